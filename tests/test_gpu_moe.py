"""Parity of the routed-expert operations (HIP, through the C ABI) against the CPU oracle:
router ids bit-exact and weights to 1e-5, grouping bit-exact, the combine bit-exact in its
float order, and the whole routed FFN layer to 1e-3 (Qwen3-30B-A3B-like shapes)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu
Q4_K = ops.TYPE_Q4_K


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


@pytest.mark.parametrize("tokens,experts,used", [(1, 128, 8), (16, 128, 8), (512, 128, 8), (33, 60, 4), (7, 256, 1),
                                                 (5, 8, 8)])
def test_router_matches_oracle(device, tokens, experts, used):
    logits = synth.rng(7 + tokens).standard_normal((tokens, experts), dtype=np.float32)
    want_ids, want_w = oracle.route(logits, used)
    ids, w = ops.moe_router(dev(logits, device), used)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    np.testing.assert_allclose(w.cpu().numpy(), want_w, rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(w.cpu().numpy().sum(axis=1), 1.0, rtol=1e-5)


def test_router_ties_and_degenerate_rows(device):
    """tests/unit/qwen38_fast_test.cc:975-1037 of the reference: ties go to the lower index;
    rows of NaN or -inf pick experts 0 .. used - 1 with zero weights."""
    experts, used = 128, 8
    logits = np.zeros((6, experts), dtype=np.float32)
    logits[0, [5, 9, 100]] = 2.0  # three tied leaders, then the zeros in index order
    logits[1, :] = -np.inf
    logits[2, 17] = np.nan
    logits[3, :] = np.inf
    logits[4, :] = -np.inf
    logits[4, [3, 70]] = [1.0, 1.5]  # two finite experts: the rest by index with zero weight
    logits[5] = np.linspace(-3, 3, experts, dtype=np.float32)
    want_ids, want_w = oracle.route(logits, used)
    ids, w = ops.moe_router(dev(logits, device), used)
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    assert np.array_equal(ids, want_ids)
    assert list(ids[0][:3]) == [5, 9, 100] and list(ids[0][3:]) == [0, 1, 2, 3, 4]
    for row in (1, 2, 3):
        assert list(ids[row]) == list(range(used)) and np.all(w[row] == 0)
    assert list(ids[4][:2]) == [70, 3]
    np.testing.assert_allclose(w, want_w, rtol=1e-5, atol=1e-9)
    ids2, w2 = ops.moe_router(dev(logits[5:6], device), used, normalize=False, scale=2.5)
    _, want2 = oracle.route(logits[5:6], used, normalize=False, scale=2.5)
    np.testing.assert_allclose(w2.cpu().numpy(), want2, rtol=1e-5)


@pytest.mark.parametrize("tokens,experts,used", [(1, 128, 8), (16, 128, 8), (512, 128, 8), (130, 7, 3), (1024, 128, 8),
                                                 (2000, 64, 6), (700, 300, 5), (1100, 256, 8)])
def test_route_groups_pairs_by_expert_in_token_order(device, tokens, experts, used):
    """Small problems are grouped by one workgroup, larger ones (more than 8192 slots, or more
    run counters than fit LDS) by the count / scan / assign launches."""
    g = synth.rng(11 + tokens)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    order, offsets = oracle.expert_sort(ids, experts)
    route = ops.moe_route(dev(ids, device), experts)
    assert np.array_equal(route.offsets.cpu().numpy(), offsets)
    position = route.position.cpu().numpy()
    # order[row] is the pair at that row: position is its inverse.
    assert np.array_equal(position[order], np.arange(tokens * used))
    assert np.array_equal(route.token.cpu().numpy(), order // used)
    assert np.array_equal(route.expert.cpu().numpy(), ids.reshape(-1)[order])
    counts = np.diff(offsets)
    padded = np.concatenate([[0], np.cumsum((counts + 127) // 128 * 128)])
    assert np.array_equal(route.scale_rows.cpu().numpy(), padded)


def test_route_marks_ids_outside_the_experts(device):
    ids = np.array([[0, 5], [9, 1], [-1, 0]], dtype=np.int32)
    route = ops.moe_route(dev(ids, device), 4)
    position = route.position.cpu().numpy()
    assert position[1] == -1 and position[2] == -1 and position[4] == -1
    assert np.array_equal(route.offsets.cpu().numpy(), [0, 2, 3, 3, 3])


def test_combine_is_the_ordered_float_sum(device):
    tokens, used, width = 9, 8, 2048
    g = synth.rng(21)
    x = g.standard_normal((tokens, used, width), dtype=np.float32)
    w = g.random((tokens, used), dtype=np.float32)
    want = oracle.expert_reduce(x, w)
    got = ops.moe_combine(dev(x.reshape(-1, width), device), dev(w, device)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    closed = (x.astype(np.float64) * w[:, :, None]).sum(axis=1)
    np.testing.assert_allclose(got, closed, rtol=1e-5, atol=1e-5)
    # Sorted rows: the same sum through a permutation.
    perm = g.permutation(tokens * used).astype(np.int32)
    shuffled = np.zeros_like(x.reshape(-1, width))
    shuffled[perm] = x.reshape(-1, width)
    got2 = ops.moe_combine(dev(shuffled, device), dev(w, device), dev(perm, device)).cpu().numpy()
    assert np.array_equal(got2.view(np.uint32), want.view(np.uint32))


def test_gathering_quantizer_is_the_quantizer(device):
    x = synth.activations(10, 768, 31)
    rows = np.array([3, 3, 0, 9, 5], dtype=np.int32)
    got = ops.quantize_q8_1_rows(dev(x, device), dev(rows, device)).cpu().numpy()
    assert np.array_equal(got, oracle.q8_1_quantize(x[rows]))


@pytest.mark.parametrize("tokens", [1, 16, 40, 512])
def test_routed_ffn_layer_matches_oracle_stage_by_stage(device, tokens):
    """Qwen3-30B-A3B-like: 128 experts, top-8, hidden 2048, expert FFN 768, Q4_K. 40 and 512 tokens
    take the sorted path (320 and 4096 pairs: about 2.5 and 32 rows an expert, the latter two and more
    passes of the matrix-core form), 1 and 16 the routed mat-vec. Every stage is compared with
    the oracle over identical input bytes (the second product over the device's own quantized
    h: a float rounding of h can move one of its Q8_1 codes by a step, which is a different
    input, not an error of the product). exec.cc:966-1002,1819-1856 of the reference."""
    t, hidden, ffn, experts, used = Q4_K, 2048, 768, 128, 8
    qk, bs = 256, 144
    gate_up = synth.q4_k_weights(experts * 2 * ffn, hidden, 41).reshape(experts, -1)
    down = synth.q4_k_weights(experts * hidden, ffn, 42).reshape(experts, -1)
    logits = synth.rng(43 + tokens).standard_normal((tokens, experts), dtype=np.float32)
    x = synth.activations(tokens, hidden, 44)
    keep = {}
    got, ids, w = ops.moe_ffn(t, dev(logits, device), dev(x, device), dev(gate_up, device), dev(down, device), hidden,
                              ffn, experts, used, keep=keep)
    want_ids, want_w = oracle.route(logits, used)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    threads = oracle.max_threads()
    up = gate_up.reshape(-1)[ffn * (hidden // qk) * bs:]
    want_h = oracle.vecq(t, up, oracle.q8_1_quantize(x), hidden, ffn, gate=gate_up, ids=want_ids, tokens=tokens,
                         used=used, stride_expert=2 * ffn * (hidden // qk), glu=oracle.GLU_SWIGLU, experts=experts,
                         threads=threads).reshape(tokens * used, ffn)
    h = keep["h"].cpu().numpy().reshape(-1, ffn)
    hq = keep["hq"].cpu().numpy()
    y = keep["y"].cpu().numpy().reshape(-1, hidden)
    pairs = np.arange(tokens * used)
    if "route" in keep:  # sorted rows: row r holds pair order[r]
        order, _ = oracle.expert_sort(want_ids, experts)
        assert np.array_equal(keep["route"].position.cpu().numpy()[order], pairs)
        pairs = order
    # 1e-3 of each value, of those under a hundredth of the RMS 1e-5 of the RMS: h is a product of two sums of
    # 2048 terms that cancel, and the matrix-core form adds a row's sub-blocks one after the other where the
    # oracle adds pairs (the reference's own check, tests/unit/dsv4_fast_test.cc:419, allows 2e-5 absolute).
    ok, worst = rel_close(h, want_h[pairs], 1e-3, floor=1e-2)
    assert ok, worst
    assert np.array_equal(hq, oracle.q8_1_quantize(h))
    blocks = oracle.padded_k(ffn) // 32
    unsorted_hq = np.zeros_like(hq)
    unsorted_hq[pairs] = hq
    want_y = oracle.vecq(t, down, unsorted_hq, ffn, hidden, ids=want_ids, tokens=tokens, used=used,
                         stride_expert=hidden * (ffn // qk), y_token=blocks * used, y_slot=blocks, experts=experts,
                         threads=threads).reshape(tokens * used, hidden)
    ok, worst = rel_close(y, want_y[pairs], 1e-3)
    assert ok, worst
    unsorted_y = np.zeros_like(y)
    unsorted_y[pairs] = y
    want = oracle.expert_reduce(unsorted_y.reshape(tokens, used, hidden), w.cpu().numpy())
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    # Without a request for the intermediates the products quantize their activations
    # themselves: the same bits out.
    plain, _, _ = ops.moe_ffn(t, dev(logits, device), dev(x, device), dev(gate_up, device), dev(down, device), hidden,
                              ffn, experts, used)
    assert np.array_equal(plain.cpu().numpy().view(np.uint32), got.cpu().numpy().view(np.uint32))
    # End to end against the all-CPU layer: the quantization steps bound it, not float order.
    cpu_hq = oracle.q8_1_quantize(want_h)
    cpu_y = oracle.vecq(t, down, cpu_hq, ffn, hidden, ids=want_ids, tokens=tokens, used=used,
                        stride_expert=hidden * (ffn // qk), y_token=blocks * used, y_slot=blocks, experts=experts,
                        threads=threads)
    cpu = oracle.expert_reduce(cpu_y, want_w).astype(np.float64)
    nmse = np.sum((got.cpu().numpy() - cpu) ** 2) / np.sum(cpu ** 2)
    assert nmse <= 1e-6, nmse


def test_sorted_rows_equal_the_routed_product(device):
    """The sorted form's flat variant computes each (token, slot) row with the routed form's arithmetic, bit for
    bit; its default (the matrix cores) the same exact sub-block sums in another float order."""
    t, hidden, ffn, experts, used, tokens = Q4_K, 1024, 256, 16, 4, 12
    gate_up = synth.q4_k_weights(experts * 2 * ffn, hidden, 51).reshape(experts, -1)
    g = synth.rng(52)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    x = synth.activations(tokens, hidden, 53)
    gd = dev(gate_up, device)
    up = gd.view(-1)[ffn * (hidden // 256) * 144:]
    stride = 2 * ffn * (hidden // 256)
    q8 = ops.quantize_q8_1(dev(x, device))
    routed = ops.vecq(t, up, q8, hidden, ffn, gate=gd, ids=dev(ids, device), tokens=tokens, used=used,
                      stride_expert=stride, glu=ops.GLU_SWIGLU).cpu().numpy().reshape(tokens * used, ffn)
    route = ops.moe_route(dev(ids, device), experts)
    sq8 = ops.quantize_q8_1_rows(dev(x, device), route.token)
    position = route.position.cpu().numpy()
    sorted_rows = ops.vecq_sorted(t, up, sq8, route.offsets, hidden, ffn, experts, gate=gd, stride_expert=stride,
                                  glu=ops.GLU_SWIGLU, variant=7).cpu().numpy()
    assert np.array_equal(sorted_rows[position].view(np.uint32), routed.view(np.uint32))
    default = ops.vecq_sorted(t, up, sq8, route.offsets, hidden, ffn, experts, gate=gd, stride_expert=stride,
                              glu=ops.GLU_SWIGLU).cpu().numpy()
    ok, worst = rel_close(default[position], routed, 1e-5, floor=1.0)
    assert ok, worst


def nvfp4_operand(g, rows, k, padded_rows=None):
    """Random NVFP4 rows: codes uint8 [rows, k / 2] and UE4M3 scales (finite, moderate) in atoms for padded_rows rows."""
    padded_rows = (rows + 127) // 128 * 128 if padded_rows is None else padded_rows
    codes = g.integers(0, 256, size=(rows, k // 2), dtype=np.uint8)
    scales = g.integers(0x20, 0x50, size=padded_rows * (k // 16), dtype=np.uint8)  # 2^-3 .. 2^3
    return codes, scales


@pytest.mark.parametrize("counts,n,k", [([5, 0, 70, 1, 130], 96, 256), ([64, 64], 64, 64), ([3], 200, 1024),
                                        ([17, 33, 0, 0, 129, 2, 64, 11], 768, 2048),
                                        # 128 experts as the reference's layers have them, most without a row
                                        ([(7 * e) % 41 if e % 5 == 0 else (1 if e % 17 == 3 else 0) for e in range(128)], 256, 512)])
def test_grouped_nvfp4_gemm_matches_its_definition(device, counts, n, k):
    """llmp.moe.gemm (RunGroupedGemm, src/kernels/ggml/moe_cutlass.h:48-76 of the reference): experts with no rows,
    one row, partial tiles of rows and of columns, more rows than a tile; D in BF16 within one rounding of the F64
    product of the decoded operands (both operands decode exactly; F32 accumulation)."""
    g = synth.rng(91 + n + k)
    groups = len(counts)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    sf_rows = np.concatenate([[0], np.cumsum((np.array(counts) + 127) // 128 * 128)]).astype(np.int32)
    rows = int(offsets[-1])
    a_codes, a_scales = nvfp4_operand(g, rows, k, padded_rows=int(sf_rows[-1]))
    codes_bytes, scales_bytes = n * (k // 2), (n + 127) // 128 * 128 * (k // 16)
    scales_offset = (codes_bytes + 255) // 256 * 256
    expert_stride = (scales_offset + scales_bytes + 255) // 256 * 256
    weights = np.zeros((groups, expert_stride), dtype=np.uint8)
    b_codes, b_scales = [], []
    for e in range(groups):
        c, s = nvfp4_operand(g, n, k)
        weights[e, :codes_bytes] = c.reshape(-1)
        weights[e, scales_offset:scales_offset + scales_bytes] = s
        b_codes.append(c)
        b_scales.append(s)
    want = oracle.grouped_nvfp4_gemm(a_codes, a_scales, offsets, sf_rows, b_codes, b_scales, n, k)
    guard = torch.full((rows + 2, n), -7.0, dtype=torch.bfloat16, device=device)
    got = ops.moe_gemm(dev(a_codes, device), dev(a_scales, device), dev(offsets, device), dev(sf_rows, device),
                       dev(weights, device), expert_stride, 0, scales_offset, n, k, out=guard[1:rows + 1])
    got = got.float().cpu().numpy().astype(np.float64)
    rms = np.sqrt(np.mean(want * want))
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-5 * rms), float(np.max(np.abs(got - want)))
    assert torch.all(guard[0] == -7.0) and torch.all(guard[rows + 1] == -7.0)  # nothing outside the rows is written


def test_grouped_nvfp4_gemm_scales_that_are_not_numbers(device):
    """A UE4M3 scale byte from 0x7F on is NaN (src/kernels/reference/decode.cc:407-411 of the reference): exactly the
    outputs whose row or column holds one are NaN, the others are as without it."""
    g = synth.rng(77)
    counts, n, k = [20, 40], 128, 256
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    sf_rows = np.array([0, 128, 256], dtype=np.int32)
    rows = int(offsets[-1])
    a_codes, a_scales = nvfp4_operand(g, rows, k, padded_rows=256)
    codes_bytes, scales_bytes = n * (k // 2), 128 * (k // 16)
    weights = np.zeros((2, codes_bytes + scales_bytes), dtype=np.uint8)
    b_codes, b_scales = [], []
    for e in range(2):
        c, s = nvfp4_operand(g, n, k)
        b_codes.append(c)
        b_scales.append(s)
    sf = lambda row, block: (((row // 128) * (k // 64)) + block // 4) * 512 + (row % 32) * 16 + ((row % 128) // 32) * 4 + block % 4
    a_scales[sf(128 + 7, 5)] = 0x7F   # group 1's row 7
    a_scales[sf(3, 0)] = 0x93         # group 0's row 3
    b_scales[1][sf(100, 15)] = 0xFF   # expert 1's column 100
    b_scales[0][sf(0, 9)] = 0x80      # expert 0's column 0
    for e in range(2):
        weights[e, :codes_bytes] = b_codes[e].reshape(-1)
        weights[e, codes_bytes:] = b_scales[e]
    want = oracle.grouped_nvfp4_gemm(a_codes, a_scales, offsets, sf_rows, b_codes, b_scales, n, k)
    got = ops.moe_gemm(dev(a_codes, device), dev(a_scales, device), dev(offsets, device), dev(sf_rows, device),
                       dev(weights, device), codes_bytes + scales_bytes, 0, codes_bytes, n, k)
    got = got.float().cpu().numpy().astype(np.float64)
    expect_nan = np.zeros((rows, n), dtype=bool)
    expect_nan[3, :] = expect_nan[20 + 7, :] = True
    expect_nan[:20, 0] = expect_nan[20:, 100] = True
    assert np.array_equal(np.isnan(want), expect_nan) and np.array_equal(np.isnan(got), expect_nan)
    fine = ~expect_nan
    assert np.all(np.abs(got[fine] - want[fine]) <= 2.0 ** -8 * np.abs(want[fine]) + 1e-5 * np.sqrt(np.mean(want[fine] ** 2)))


def test_grouped_nvfp4_gemm_refusals(device):
    lib = ops._lib.load()
    g = ops._lib.GroupedGemm()
    import ctypes as C
    assert lib.llmp_hip_grouped_gemm_available() == 1 and lib.llmp_hip_grouped_gemm_scratch(128, 256) == 0
    g.groups, g.n, g.k = 2, 64, 96
    assert lib.llmp_hip_grouped_gemm_run(C.byref(g), 256, None) > 0 and b"64-value" in lib.llmp_hip_last_error()
    g.k = 128
    assert lib.llmp_hip_grouped_gemm_run(C.byref(g), 256, None) > 0 and b"null" in lib.llmp_hip_last_error()


@pytest.mark.parametrize("launches", [2, 1])
@pytest.mark.parametrize("hidden,ffn,experts,used,x_dtype", [(2048, 768, 128, 8, "f32"), (1024, 512, 16, 4, "bf16"), (512, 256, 8, 1, "f32")])
def test_one_token_layer_in_one_launch_equals_the_four_operations(device, launches, hidden, ffn, experts, used, x_dtype):
    """llmp_hip_moe_token (router, gate/up with the GLU, down, ordered weighted sum in one launch, or its two halves as
    two): the router's ids and weights and the layer's output are bit for bit those of llmp.moe.router,
    llmp_hip_vecq_fused twice and llmp.moe.combine, and within 1e-3 of the oracle's layer; three calls in a row over the
    same meeting words (no reset between them) give the same bits, and no workgroup ever gave up waiting."""
    t = Q4_K
    gate_up = synth.q4_k_weights(experts * 2 * ffn, hidden, 401).reshape(experts, -1)
    down = synth.q4_k_weights(experts * hidden, ffn, 402).reshape(experts, -1)
    logits = synth.rng(403).standard_normal((1, experts), dtype=np.float32)
    x = synth.activations(1, hidden, 404)
    if x_dtype == "bf16":
        x = synth.bf16_to_f32(synth.bf16_bits(x))
    gd, dd, ld = dev(gate_up, device), dev(down, device), dev(logits, device)
    xd = dev(x, device) if x_dtype == "f32" else dev(x, device).to(torch.bfloat16)
    want, ids, weights = ops.moe_ffn(t, ld, xd if x_dtype == "f32" else dev(x, device), gd, dd, hidden, ffn, experts, used)
    state = ops.MoeTokenState(used, ffn, device)
    outs = []
    for _ in range(3):
        outs.append(ops.moe_token(t, ld.view(-1), xd.view(-1), gd, dd, hidden, ffn, experts, used, state, launches=launches).clone())
    torch.cuda.synchronize()
    words = state.sync.cpu().numpy()
    assert words[2] == 0, "a workgroup gave up waiting at the meeting"
    assert np.all(words[4:4 + 8] == (3 if launches == 1 else 0))  # a word a workgroup: the meetings it has come to
    assert torch.equal(state.ids, ids.view(-1)) and torch.equal(state.weights.view(torch.int32), weights.view(-1).view(torch.int32))
    for got in outs:
        assert torch.equal(got.view(torch.int32), want.view(-1).view(torch.int32))
    # And the oracle's layer over the same inputs (the activated values quantized again before the down product).
    ids_c, w_c = oracle.route(logits, used)
    qk = 256
    up_c = gate_up.reshape(-1)[ffn * (hidden // qk) * 144:]
    h_c = oracle.vecq(oracle.TYPE_Q4_K, up_c, oracle.q8_1_quantize(x), hidden, ffn, gate=gate_up, ids=ids_c, tokens=1, used=used,
                      stride_expert=2 * ffn * (hidden // qk), glu=oracle.GLU_SWIGLU, experts=experts)
    hq = oracle.q8_1_quantize(h_c.reshape(used, ffn))
    blocks = oracle.padded_k(ffn) // 32
    y_c = oracle.vecq(oracle.TYPE_Q4_K, down, hq, ffn, hidden, ids=ids_c, tokens=1, used=used, stride_expert=hidden * (ffn // qk),
                      y_token=blocks * used, y_slot=blocks, experts=experts)
    ref = oracle.expert_reduce(y_c, w_c).reshape(-1)
    ok, worst = rel_close(outs[0].cpu().numpy(), ref, 2e-3, floor=1e-2)
    assert ok, worst


def test_one_token_layer_refusals(device):
    import ctypes as C
    lib = ops._lib.load()
    op = ops._lib.MoeToken()
    for name in ("logits", "x", "gate_up", "down", "out", "ids", "weights", "h", "sync"):
        setattr(op, name, 0x10000)
    op.type, op.x_type, op.experts, op.used, op.hidden, op.ffn, op.glu, op.normalize = Q4_K, ops.X_F32, 128, 8, 2048, 768, ops.GLU_SWIGLU, 1
    op.gate_up_stride, op.down_stride = 2 * 768 * 8, 2048 * 3
    for field, value, what in (("used", 9, b"picks"), ("hidden", 2000, b"super-blocks"), ("type", ops.TYPE_Q8_0, b"Q4_K"),
                               ("glu", ops.GLU_NONE, b"a GLU"), ("down_stride", 100, b"stride"), ("sync", None, b"null")):
        saved = getattr(op, field)
        setattr(op, field, value)
        assert lib.llmp_hip_moe_token(C.byref(op), 1, 256, None) == 1 and what in lib.llmp_hip_last_error(), (field, lib.llmp_hip_last_error())
        setattr(op, field, saved)
    assert lib.llmp_hip_moe_token(C.byref(op), 3, 256, None) == 1
