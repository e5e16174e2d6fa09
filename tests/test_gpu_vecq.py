"""Parity of llmp.q8_1 and llmp.vecq (HIP, through the C ABI) against the CPU oracle on
the same seeded inputs. Integer work is compared bit for bit; float outputs to a maximum
relative error of 1e-3 (the accumulation order is the only difference)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = ops.TYPE_Q8_0, ops.TYPE_Q4_K
TOL = 1e-3


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def make_weights(t, n, k, seed, plausible=True):
    if plausible:
        return synth.q8_0_weights(n, k, seed) if t == Q8_0 else synth.q4_k_weights(n, k, seed)
    return synth.random_blocks(t, n, k, seed)


@pytest.mark.parametrize("k,rows", [(4096, 1), (3840, 8), (32, 3), (544, 5)])
def test_q8_1_quantize_is_bit_exact(device, k, rows):
    x = synth.activations(rows, k, 11 + k)
    x[0, : min(k, 40)] = 0.0  # a zero block
    if rows > 1:
        x[1] *= 1e-6
    want = oracle.q8_1_quantize(x)
    got = ops.quantize_q8_1(dev(x, device)).cpu().numpy()
    assert got.shape == want.shape
    assert np.array_equal(got, want)


def test_q8_1_quantize_ties_and_near_ties_are_bit_exact(device):
    """Quotients x / d on and beside k + 1/2 (the device multiplies by a reciprocal where that cannot change the rounded
    integer and divides otherwise), scales that are powers of two and not, blocks of tiny and huge values, a block whose
    largest magnitude is subnormal: the oracle's codes, scales and sums, bit for bit."""
    g = synth.rng(77)
    rows, k = 24, 1024
    x = np.zeros((rows, k), dtype=np.float32)
    for r in range(rows):
        for b in range(k // 32):
            amax = np.float32([127.0, 63.5, 254.0, 1.0, 3.0, 100.0, 0.37, 12.7][(r + b) % 8])
            d = np.float32(amax / np.float32(127.0))
            halves = (g.integers(-126, 126, size=32).astype(np.float32) + np.float32(0.5)) * d
            nudge = g.integers(-2, 3, size=32)
            block = halves.copy()
            for _ in range(2):  # up to two units in the last place either way
                block = np.where(nudge > 0, np.nextafter(block, np.float32(np.inf)), np.where(nudge < 0, np.nextafter(block, np.float32(-np.inf)), block))
                nudge = nudge - np.sign(nudge)
            block[g.integers(0, 32)] = amax * (1 if b % 2 else -1)
            x[r, b * 32:(b + 1) * 32] = block
    x[20] *= np.float32(1e-30)
    x[21] *= np.float32(1e30)
    x[22] *= np.float32(1e-38)
    x[23, :32] = np.float32(1e-41)  # subnormal: its scale's reciprocal is not finite
    want = oracle.q8_1_quantize(x)
    got = ops.quantize_q8_1(dev(x, device)).cpu().numpy()
    assert np.array_equal(got, want)


def test_q8_1_planes_and_strides(device):
    x = synth.activations(2 * 3, 256, 5).reshape(2, 3, 256)
    wide = np.zeros((2, 3, 300), dtype=np.float32)
    wide[:, :, :256] = x
    xd = dev(wide, device)[:, :, :256]
    got = ops.quantize_q8_1(xd).cpu().numpy()
    want = oracle.q8_1_quantize(x.reshape(6, 256)).reshape(2, 3, -1)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("t,k,n,variant", [(Q8_0, 4096, 64, 0), (Q4_K, 3840, 40, 0), (Q4_K, 3840, 40, 6),
                                           (Q8_0, 96, 9, 0), (Q4_K, 256, 7, 0), (Q4_K, 256, 7, 6),
                                           (Q4_K, 2048, 300, 6), (Q8_0, 4096, 64, 6), (Q8_0, 256, 7, 6),
                                           (Q8_0, 3840, 41, 6)])
def test_block_sums_are_bit_exact(device, t, k, n, variant):
    """The int32 sums of the rows form (variant 0) and of the flat form (variant 6)."""
    w = make_weights(t, n, k, 21, plausible=False)
    q8 = oracle.q8_1_quantize(synth.activations(1, k, 22))
    want = oracle.vecq_block_sums(t, w, q8, k, n)
    got = ops.vecq_block_sums(t, dev(w, device), dev(q8, device), k, n, variant=variant).cpu().numpy()
    assert np.array_equal(got, want)


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
@pytest.mark.parametrize("k,n", [(4096, 256), (3840, 100), (512, 33), (256, 1)])
@pytest.mark.parametrize("tokens", [1, 2, 3, 4, 8, 16])
def test_dense_matches_oracle(device, t, k, n, tokens):
    w = make_weights(t, n, k, 31 + k + n)
    x = synth.activations(tokens, k, 32 + tokens)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(t, w, q8, k, n, tokens=tokens)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


@pytest.mark.parametrize("t,k,n", [(Q4_K, 15360, 37), (Q4_K, 16384, 9), (Q4_K, 13056, 70), (Q8_0, 8192, 21),
                                   (Q8_0, 14336, 12), (Q8_0, 11008, 19), (Q8_0, 32256, 5), (Q8_0, 32512, 3),
                                   (Q4_K, 20480, 11), (Q4_K, 27136, 4), (Q4_K, 27392, 3)])
@pytest.mark.parametrize("tokens", [1, 3])
def test_long_rows_match_oracle(device, t, k, n, tokens):
    """Rows whose staged activations leave room for fewer than eight waves' tiles, rows of more
    than 64 units (streamed in pieces), and rows too long for the streaming form at all."""
    w = make_weights(t, n, k, 35 + k + n)
    x = synth.activations(tokens, k, 36 + tokens)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(t, w, q8, k, n, tokens=tokens)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    # The form that quantizes in the kernel is the flat form: the same bits as the two steps through it.
    flat = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens, variant=6 if tokens == 1 else 7).cpu().numpy()
    ok, worst = rel_close(flat, want, TOL)
    assert ok, worst
    fused = ops.vecq_fused(t, dev(w, device), dev(x, device), k, n, tokens=tokens).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), flat.view(np.uint32))


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
def test_every_variant_matches_and_random_bytes_decode(device, t):
    k, n, tokens = 1024, 50, 5
    w = make_weights(t, n, k, 41, plausible=False)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 42))
    want = oracle.vecq(t, w, q8, k, n, tokens=tokens)
    for variant, name in enumerate(ops.vecq_variants()):
        units_a_wave = k // (256 if t == Q4_K else 128) // 4
        if name.endswith("tiles64") or (name.endswith("rows32") and units_a_wave < 2) or (name.endswith("rows16") and units_a_wave < 4):
            # the relaid-out variant takes whole tiles of 64 rows (and the layout it is named for); tiles of 32 and 16
            # rows take rows of two and four units a wave (a unit is 256 values of Q4_K, 128 of Q8_0)
            with pytest.raises(ops.KernelFailure):
                ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens, variant=variant)
            continue
        got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens, variant=variant).cpu().numpy()
        ok, worst = rel_close(got, want, TOL)
        assert ok, (variant, worst)


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
@pytest.mark.parametrize("glu", [ops.GLU_SWIGLU, ops.GLU_SWIGLU_CLAMP, ops.GLU_GEGLU])
@pytest.mark.parametrize("tokens", [1, 4, 8])
def test_fused_glu_matches_oracle(device, t, glu, tokens):
    k, n = 1280 if t == Q8_0 else 1280, 72
    gate = make_weights(t, n, k, 51)
    up = make_weights(t, n, k, 52)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 53))
    limit = 0.75 if glu == ops.GLU_SWIGLU_CLAMP else 0.0
    want = oracle.vecq(t, up, q8, k, n, gate=gate, tokens=tokens, glu=glu, limit=limit)
    got = ops.vecq(t, dev(up, device), dev(q8, device), k, n, gate=dev(gate, device), tokens=tokens, glu=glu,
                   limit=limit).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
@pytest.mark.parametrize("xdtype", ["f32", "bf16"])
def test_fused_activation_quantization_equals_the_two_step_path(device, t, xdtype):
    """The in-LDS quantizer is the quantizer kernel's arithmetic: outputs equal the two-step path's through the
    same (flat) form bit for bit, and its default form's to float rounding."""
    k, n, tokens = 3840, 64, 4
    w = make_weights(t, n, k, 61)
    x = synth.activations(tokens, k, 62)
    if xdtype == "bf16":
        bits = synth.bf16_bits(x)
        x = synth.bf16_to_f32(bits)
        xd = dev(bits.view(np.int16), device).view(torch.bfloat16)
    else:
        xd = dev(x, device)
    q8 = ops.quantize_q8_1(dev(x, device))
    two = ops.vecq(t, dev(w, device), q8, k, n, tokens=tokens, variant=7).cpu().numpy()
    one = ops.vecq_fused(t, dev(w, device), xd, k, n, tokens=tokens).cpu().numpy()
    assert np.array_equal(one.view(np.uint32), two.view(np.uint32))
    default = ops.vecq(t, dev(w, device), q8, k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(default, two, 1e-5, floor=1.0)
    assert ok, worst


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
@pytest.mark.parametrize("tokens,used", [(1, 8), (4, 8), (16, 8), (3, 2)])
def test_routed_experts_match_oracle(device, t, tokens, used):
    k, n, experts = 512, 48, 12
    qk, bs = oracle.block_elements(t), oracle.block_bytes(t)
    w = make_weights(t, experts * n, k, 71).reshape(experts, n * (k // qk) * bs)
    g = synth.rng(72)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 73))
    stride_expert = n * (k // qk)
    want = oracle.vecq(t, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


@pytest.mark.parametrize("t", [Q8_0, Q4_K])
@pytest.mark.parametrize("routing", ["one expert", "one a pair", "two experts, unequal"])
def test_routed_pairs_that_share_an_expert(device, t, routing):
    """The pairs that name an expert share its rows (every pair's workgroups at work on a share of them, each
    against all of the expert's tokens): whatever the picks, a pair's values are the oracle's and, bit for bit, those
    of its own token alone through its expert as a dense product."""
    tokens, used, k, n = 16, 8, 1024, 203  # 128 pairs; several tiles a share, the last partial
    experts = {"one expert": 3, "one a pair": 128, "two experts, unequal": 5}[routing]
    qk, bs = oracle.block_elements(t), oracle.block_bytes(t)
    w = make_weights(t, experts * n, k, 91).reshape(experts, n * (k // qk) * bs)
    pair = np.arange(tokens * used)
    if routing == "one expert":
        ids = np.full(tokens * used, 2)
    elif routing == "one a pair":
        ids = synth.rng(92).permutation(experts)[pair]
    else:
        ids = np.where(pair % 7 == 3, 4, 1)  # 18 pairs name one, 110 the other
    ids = ids.reshape(tokens, used).astype(np.int32)
    x = synth.activations(tokens, k, 93)
    q8 = oracle.q8_1_quantize(x)
    stride_expert = n * (k // qk)
    want = oracle.vecq(t, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    wd, q8d = dev(w, device), dev(q8, device)
    got = ops.vecq(t, wd, q8d, k, n, ids=dev(ids, device), tokens=tokens, used=used, stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    for token, slot in ((0, 0), (5, 3), (15, 7)):
        alone = ops.vecq(t, wd[ids[token, slot]].contiguous(), q8d[token:token + 1].contiguous(), k, n, tokens=1).cpu().numpy()
        assert np.array_equal(alone.reshape(n).view(np.uint32), got[token, slot].view(np.uint32)), (token, slot)


@pytest.mark.parametrize("t,k", [(Q8_0, 9216), (Q4_K, 18432)])
def test_routed_and_sorted_long_rows_match_oracle(device, t, k):
    """Rows streamed in pieces, under routing ids and under sorted-row offsets."""
    n, experts, tokens, used = 13, 5, 3, 2
    qk, bs = oracle.block_elements(t), oracle.block_bytes(t)
    w = make_weights(t, experts * n, k, 75).reshape(experts, n * (k // qk) * bs)
    g = synth.rng(76)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 77))
    stride_expert = n * (k // qk)
    want = oracle.vecq(t, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    # The same pairs as rows sorted by expert.
    order = np.argsort(ids.reshape(-1), kind="stable")
    offsets = np.concatenate([[0], np.cumsum(np.bincount(ids.reshape(-1), minlength=experts))]).astype(np.int32)
    rows = np.ascontiguousarray(q8.reshape(tokens, -1)[order // used])
    sorted_out = ops.vecq_sorted(t, dev(w, device), dev(rows, device), dev(offsets, device), k, n, experts,
                                 stride_expert=stride_expert).cpu().numpy()
    assert np.array_equal(sorted_out.view(np.uint32), got.reshape(tokens * used, n)[order].view(np.uint32))


def same_sums(t, a, b):
    """Q8_0: the matrix-core kernel repeats the flat kernel's float operations and its summation tree, bit for bit.
    Q4_K: its sub-block sums are the same exact integers, scaled and added in another order (one fma a sub-block
    on the matrix cores' F32 results): the two forms agree to float rounding."""
    if t == Q8_0:
        return np.array_equal(a.view(np.uint32), b.view(np.uint32)), 0.0
    return rel_close(a, b, 1e-5, floor=1.0)


@pytest.mark.parametrize("t,k,n,tokens", [(Q4_K, 2816, 50, 5), (Q4_K, 256, 17, 2), (Q4_K, 6144, 32, 16),
                                          (Q4_K, 2048, 130, 9), (Q4_K, 8192, 40, 8), (Q4_K, 768, 100, 13),
                                          (Q8_0, 4096, 50, 5), (Q8_0, 256, 17, 2),
                                          (Q8_0, 3840, 20, 16), (Q8_0, 1792, 130, 9), (Q8_0, 768, 33, 3)])
def test_matrix_core_form_against_the_flat_form_and_the_oracle(device, t, k, n, tokens):
    """The matrix-core kernels (variant 9) against the flat form's four-token passes (one-token arithmetic) and the
    oracle: dense with and without a GLU, grouped matrices, and routed experts."""
    mma, flat = 9, 7
    qk = oracle.block_elements(t)
    gate, up = make_weights(t, n, k, 301), make_weights(t, n, k, 302)
    x = synth.activations(tokens, k, 303)
    q8 = ops.quantize_q8_1(dev(x, device))
    wd, gd = dev(up, device), dev(gate, device)
    for kw, okw in ((dict(), dict()), (dict(gate=gd, glu=ops.GLU_SWIGLU), dict(gate=gate, glu=oracle.GLU_SWIGLU))):
        a = ops.vecq(t, wd, q8, k, n, tokens=tokens, variant=mma, **kw).cpu().numpy()
        b = ops.vecq(t, wd, q8, k, n, tokens=tokens, variant=flat, **kw).cpu().numpy()
        ok, worst = same_sums(t, a, b)
        assert ok, (kw.keys(), worst)
        want = oracle.vecq(t, up, q8.cpu().numpy(), k, n, tokens=tokens, **okw)
        ok, worst = rel_close(a.reshape(tokens, n), want.reshape(tokens, n), TOL)
        assert ok, (kw.keys(), worst)
    # Three matrices, every token through each (per-slot activations).
    groups = 3
    w3 = dev(make_weights(t, groups * n, k, 304).reshape(groups, -1), device)
    q83 = ops.quantize_q8_1(dev(synth.activations(tokens * groups, k, 305), device))
    y_row = ops.padded_k(k) // 32
    kw = dict(tokens=tokens, used=groups, stride_expert=n * (k // qk), y_token=y_row * groups, y_slot=y_row)
    a = ops.vecq(t, w3, q83, k, n, variant=mma, **kw).cpu().numpy()
    b = ops.vecq(t, w3, q83, k, n, variant=flat, **kw).cpu().numpy()
    ok, worst = same_sums(t, a, b)
    assert ok, worst
    # Routed: two picks a token out of five experts.
    experts, used = 5, 2
    w5 = dev(make_weights(t, experts * n, k, 306).reshape(experts, -1), device)
    g = synth.rng(307)
    ids = dev(np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32), device)
    kw = dict(ids=ids, tokens=tokens, used=used, stride_expert=n * (k // qk))
    a = ops.vecq(t, w5, q8, k, n, variant=mma, **kw).cpu().numpy()
    b = ops.vecq(t, w5, q8, k, n, variant=flat, **kw).cpu().numpy()
    ok, worst = same_sums(t, a, b)
    assert ok, worst


@pytest.mark.parametrize("variant,tokens", [(9, 16), (10, 8)])
@pytest.mark.parametrize("k,n,glu", [(2816, 50, False), (3840, 70, True), (8192, 20, True), (1024, 133, False)])
def test_matrix_core_forms_values_depend_on_their_own_token_alone(device, variant, tokens, k, n, glu):
    """src/kernels/ggml/vecq.cu:688-693 of the reference, within each matrix-core form (9: the 16 x 16 instruction,
    up to sixteen tokens; 10: a weight row a lane, up to eight): a (token, row) value is the same bits whatever
    tokens are computed beside it, however many (the kernels stage groups of four, eight or sixteen tokens by the
    count) and in whatever order."""
    t = Q4_K
    gate, up = make_weights(t, n, k, 311), make_weights(t, n, k, 312)
    x = synth.activations(16, k, 313)[:tokens]
    x[5] *= 30.0
    q8 = ops.quantize_q8_1(dev(x, device))
    wd = dev(up, device)
    kw = dict(gate=dev(gate, device), glu=ops.GLU_GEGLU) if glu else {}
    full = ops.vecq(t, wd, q8, k, n, tokens=tokens, variant=variant, **kw).cpu().numpy().reshape(tokens, n)
    for count in (2, 3, 4, 7, 8, 9, 13):
        if count > tokens:
            continue
        part = ops.vecq(t, wd, q8[:count].contiguous(), k, n, tokens=count, variant=variant, **kw).cpu().numpy()
        assert np.array_equal(part.reshape(count, n).view(np.uint32), full[:count].view(np.uint32)), count
    order = synth.rng(314).permutation(tokens)
    mixed = ops.vecq(t, wd, q8[torch.from_numpy(order).to(device)].contiguous(), k, n, tokens=tokens, variant=variant, **kw)
    assert np.array_equal(mixed.cpu().numpy().reshape(tokens, n).view(np.uint32), full[order].view(np.uint32))


@pytest.mark.parametrize("variant,k,tokens", [(9, 512, 16), (10, 1024, 8), (10, 1024, 3)])
def test_matrix_core_forms_sub_block_sums_are_exact_integers(device, variant, k, tokens):
    """With d = 1, dmin = 0 and unit block scales a Q4_K product is the integer sum over sub-blocks of
    sc * sum(q * code): every partial sum stays below 2^24, so F32 holds it exactly and the kernel must return
    exactly the integer (a matrix-core product that rounded inside a sub-block would not)."""
    n = 48
    g = synth.rng(321)
    w = synth.q4_k_weights(n, k, 322).reshape(n, k // 256, 144).copy()
    w[:, :, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    w[:, :, 2:4] = 0
    w[:, :, 4:16] &= 0x07  # scales and minimums below 8: four super-blocks of 8 x 32 x 7 x 15 x 127 stay below 2^24
    sc = w[:, :, 4:8].astype(np.int64) & 63  # sub-blocks 0 .. 3; 4 .. 7 are the low nibbles of bytes 12 .. 15
    sc = np.concatenate([sc, w[:, :, 12:16].astype(np.int64) & 15], axis=2)  # [n, nsb, 8]
    assert sc.max() <= 7
    qs = w[:, :, 16:].reshape(n, k // 256, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, k // 256, 8, 32).astype(np.int64)
    codes = g.integers(-127, 128, size=(tokens, k // 32, 32), dtype=np.int64)
    q8 = np.zeros((tokens, ops.padded_k(k) // 32, 36), dtype=np.uint8)
    q8[:, :k // 32, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    q8[:, :k // 32, 4:] = codes.astype(np.int8).view(np.uint8)
    sums = np.einsum("rbgk,tbgk->trbg", q, codes.reshape(tokens, k // 256, 8, 32))
    want = np.einsum("trbg,rbg->tr", sums, sc)
    assert np.abs(want).max() < 2 ** 24
    got = ops.vecq(Q4_K, dev(w.reshape(-1), device), dev(q8, device), k, n, tokens=tokens, variant=variant).cpu().numpy()
    assert np.array_equal(got.reshape(tokens, n).astype(np.int64), want)
    assert np.array_equal(got.reshape(tokens, n), want.astype(np.float32))


@pytest.mark.parametrize("k,n,tokens", [(1024, 17, 2), (2816, 130, 5), (6144, 64, 8), (16384, 70, 4), (3840, 200, 7),
                                        (15360, 70, 8), (20480, 130, 6), (32768, 64, 3), (9472, 20, 8)])
def test_row_a_lane_form_matches_oracle(device, k, n, tokens):
    """Variant 10 (Q4_K, a weight row a lane, 2 to 8 tokens): dense with and without a GLU, rows that end within a
    tile of 64, three grouped matrices, more than eight tokens, rows whose tokens are staged a span at a time (15360 and 20480 values at 5 to
    8 tokens, 32768 at 3, 9472 in two uneven spans); and what it refuses: routed products, one token, 17, short
    rows."""
    t, rows = Q4_K, 10
    gate, up = make_weights(t, n, k, 331), make_weights(t, n, k, 332)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 333))
    names = ops.vecq_variants()
    assert names[rows] == "rows pass8"
    for kw, okw in ((dict(), dict()), (dict(gate=dev(gate, device), glu=ops.GLU_GEGLU), dict(gate=gate, glu=oracle.GLU_GEGLU))):
        want = oracle.vecq(t, up, q8, k, n, tokens=tokens, **okw)
        got = ops.vecq(t, dev(up, device), dev(q8, device), k, n, tokens=tokens, variant=rows, **kw).cpu().numpy()
        ok, worst = rel_close(got.reshape(tokens, n), want.reshape(tokens, n), TOL, floor=1e-2 if kw else 1e-3)
        assert ok, (kw.keys(), worst)
        # The tiles by name: 64 rows, and 32 and 16 where every wave has two and four super-blocks of a row.
        for parts, name in ((1, "rows pass8 rows64"), (2, "rows pass8 rows32"), (4, "rows pass8 rows16")):
            # (37 super-blocks a row are quarters of 9 and 10; eight tokens of them are staged in spans, and no span of
            # whole four-unit pieces leaves the shortest quarter four units for the last span.)
            if k // 256 // 4 < parts or (k == 9472 and tokens == 8 and parts == 4):
                with pytest.raises(ops.KernelFailure):
                    ops.vecq(t, dev(up, device), dev(q8, device), k, n, tokens=tokens, variant=names.index(name), **kw)
                continue
            got = ops.vecq(t, dev(up, device), dev(q8, device), k, n, tokens=tokens, variant=names.index(name), **kw)
            ok, worst = rel_close(got.cpu().numpy().reshape(tokens, n), want.reshape(tokens, n), TOL, floor=1e-2 if kw else 1e-3)
            assert ok, (name, kw.keys(), worst)
            two = ops.vecq(t, dev(up, device), dev(q8, device), k, n, tokens=2, variant=names.index(name), **kw)
            assert torch.equal(two.view(torch.int32), got[:2].view(torch.int32)), name
    groups = 3
    w3 = make_weights(t, groups * n, k, 334).reshape(groups, -1)
    q83 = oracle.q8_1_quantize(synth.activations(tokens * groups, k, 335))
    y_row = ops.padded_k(k) // 32
    kw = dict(tokens=tokens, used=groups, stride_expert=n * (k // 256), y_token=y_row * groups, y_slot=y_row)
    want = oracle.vecq(t, w3, q83, k, n, **kw)
    got = ops.vecq(t, dev(w3, device), dev(q83, device), k, n, variant=rows, **kw).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    ids = dev(np.zeros((tokens, 1), dtype=np.int32), device)
    # Rows apart (a pitch of two super-blocks more) and fewer rows than the matrix holds, through every tile that takes
    # the shape: the values of the packed matrix's rows.
    nsb = k // 256
    pitched = torch.zeros((n, nsb + 2, 144), dtype=torch.uint8, device=device)
    pitched[:, :nsb] = dev(up, device).view(n, nsb, 144)
    packed = ops.vecq(t, dev(up, device), dev(q8, device), k, n, tokens=tokens, variant=names.index("rows pass8 rows64"))
    for name in ("rows pass8", "rows pass8 rows64", "rows pass8 rows32", "rows pass8 rows16"):
        try:
            apart = ops.vecq(t, pitched.view(-1), dev(q8, device), k, n - 5, tokens=tokens, stride_row=nsb + 2, variant=names.index(name))
        except ops.KernelFailure as refused:  # a tile the rows are too short for (checked above)
            assert refused.rejected and name.endswith(("rows32", "rows16")), name
            continue
        ok, worst = rel_close(apart.cpu().numpy().reshape(tokens, n - 5), packed.cpu().numpy().reshape(tokens, n)[:, :n - 5], TOL)
        assert ok, (name, worst)
        if name.endswith("rows64"):
            assert torch.equal(apart.view(torch.int32), packed[:, :, :n - 5].contiguous().view(torch.int32))
    # Nine tokens and more (to the operation's 16) are launches of eight or fewer each: every token the bits it has among eight.
    many = min(tokens + 9, 16)
    x_many = synth.activations(many, k, 339)
    q8_many = dev(oracle.q8_1_quantize(x_many), device)
    got = ops.vecq(t, dev(up, device), q8_many, k, n, tokens=many, variant=rows)
    share = -(-many // -(-many // 8))
    for first in range(0, many, share):
        some = min(share, many - first)
        alone = ops.vecq(t, dev(up, device), dev(oracle.q8_1_quantize(x_many[first:first + some]), device), k, n, tokens=some, variant=rows)
        assert torch.equal(alone.view(torch.int32), got[first:first + some].view(torch.int32)), first
    ok, worst = rel_close(got.cpu().numpy().reshape(many, n), oracle.vecq(t, up, oracle.q8_1_quantize(x_many), k, n, tokens=many).reshape(many, n), TOL)
    assert ok, worst
    for bad in (dict(tokens=tokens, ids=ids, used=1, stride_expert=n * (k // 256)), dict(tokens=1), dict(tokens=17)):
        with pytest.raises(ops.KernelFailure):
            ops.vecq(t, dev(up, device), dev(oracle.q8_1_quantize(synth.activations(bad["tokens"], k, 336)), device), k, n,
                     variant=rows, **bad)
    with pytest.raises(ops.KernelFailure):  # three super-blocks a row: fewer than the workgroup's four waves
        ops.vecq(t, dev(make_weights(t, 8, 768, 337), device), dev(oracle.q8_1_quantize(synth.activations(2, 768, 338)), device),
                 768, 8, tokens=2, variant=rows)


def test_grouped_matrices_read_their_own_rows(device):
    t, k, n, groups, tokens = Q8_0, 256, 24, 3, 2
    qk, bs = 32, 34
    w = make_weights(t, groups * n, k, 81).reshape(groups, -1)
    x = synth.activations(tokens * groups, k, 82)
    q8 = oracle.q8_1_quantize(x)  # [tokens * groups, blocks]: row t * groups + g
    y_row = ops.padded_k(k) // 32
    kw = dict(tokens=tokens, used=groups, stride_expert=n * (k // qk), y_token=y_row * groups, y_slot=y_row)
    want = oracle.vecq(t, w, q8, k, n, **kw)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, **kw).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


def test_tokens_are_independent_and_zero_rows_give_zero(device):
    """tests/unit/dsv4_fast_test.cc:462-493 of the reference: through the flat form each token's sums are its
    one-token product's bit for bit; through the default form of four tokens (a weight row a lane) a token's sums
    are the same bits whatever tokens stand beside it, and close to its one-token product's; a zero input row
    gives zeros in both."""
    t, k, n, tokens = Q4_K, 2816, 96, 4
    gate = make_weights(t, n, k, 91)
    up = make_weights(t, n, k, 92)
    x = synth.activations(tokens, k, 93) * 0.5
    x[0] = 0.0
    x[3] *= 10
    wd, gd = dev(up, device), dev(gate, device)
    q8 = ops.quantize_q8_1(dev(x, device))
    got = ops.vecq(t, wd, q8, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU).cpu().numpy()
    flat = ops.vecq(t, wd, q8, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU, variant=7).cpu().numpy()
    assert np.all(got[0] == 0) and np.all(flat[0] == 0)
    for i in range(tokens):
        solo_q8 = ops.quantize_q8_1(dev(x[i:i + 1], device))
        solo = ops.vecq(t, wd, solo_q8, k, n, gate=gd, tokens=1, glu=ops.GLU_GEGLU).cpu().numpy()
        assert np.array_equal(solo[0].view(np.uint32), flat[i].view(np.uint32)), i
        ok, worst = rel_close(got[i], solo[0], 1e-5, floor=1.0)
        assert ok, (i, worst)
        # Token i beside another token, in the other place: the default form's own bits again.
        j = (i + 1) % tokens
        pair_q8 = ops.quantize_q8_1(dev(x[[j, i]], device))
        pair = ops.vecq(t, wd, pair_q8, k, n, gate=gd, tokens=2, glu=ops.GLU_GEGLU).cpu().numpy()
        assert np.array_equal(pair[1].view(np.uint32), got[i].view(np.uint32)), i
        assert np.array_equal(pair[0].view(np.uint32), got[j].view(np.uint32)), i


def test_guard_bytes_stay_untouched_and_refusals_queue_nothing(device):
    """tests/unit/dsv4_fast_test.cc:391-399,494-502 of the reference."""
    t, k, n = Q8_0, 512, 30
    w = dev(make_weights(t, n, k, 95), device)
    q8 = ops.quantize_q8_1(dev(synth.activations(1, k, 96), device))
    buf = torch.full((64 + n + 64,), float("nan"), dtype=torch.float32, device=device)
    buf.view(torch.int32).fill_(0x25A5A5A5)
    out = buf[64:64 + n].view(1, 1, n)
    ops.vecq(t, w, q8, k, n, out=out)
    guard = buf.view(torch.int32).cpu().numpy()
    assert np.all(guard[:64] == 0x25A5A5A5) and np.all(guard[64 + n:] == 0x25A5A5A5)
    before = buf.clone()
    with pytest.raises(ops.KernelFailure) as e:
        ops.vecq(t, w, q8, k, n, glu=ops.GLU_GEGLU, out=out)  # a GLU without gate weights
    assert e.value.rejected
    with pytest.raises(ops.KernelFailure):
        ops.vecq(t, w, q8, k, n, tokens=17, out=out)
    with pytest.raises(ops.KernelFailure):
        ops.vecq(t, w, q8, 500, n, out=out)
    torch.cuda.synchronize()
    assert torch.equal(before.view(torch.int32), buf.view(torch.int32))


# ---- the legacy 4/5-bit blocks through the streaming form (eight blocks a lane)

Q4_0 = ops.TYPE_Q4_0
LEGACY = [ops.TYPE_Q4_0, ops.TYPE_Q4_1, ops.TYPE_Q5_0, ops.TYPE_Q5_1, ops.TYPE_IQ4_NL]  # IQ4_NL: Q4_0's bytes, a codebook


@pytest.mark.parametrize("t", LEGACY)
@pytest.mark.parametrize("k,n", [(4096, 96), (256, 5), (2816, 33), (15360, 12), (20480, 7)])
@pytest.mark.parametrize("tokens", [1, 3, 4, 9])
def test_legacy_blocks_dense_match_oracle(device, t, k, n, tokens):
    """The blocks of tests/unit/dsv4_fast_test.cc:141-164: dw * (sum * d8 - 8 or 16 * s8), or
    sum * f16(dw * d8) + f16(m * s8), the activation block's stored sum included; IQ4_NL's
    (dw * d8) * sum over its codebook's values (src/kernels/ggml/vecq.cu:375-396). Rows of one
    tile, of fewer waves, and in pieces."""
    w = synth.legacy_weights(t, n, k, 401 + k + n)
    x = synth.activations(tokens, k, 402 + tokens)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(t, w, q8, k, n, tokens=tokens)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    # The form that quantizes in the kernel is the flat form: the same bits as the two steps through it.
    flat = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=tokens, variant=6 if tokens == 1 else 7).cpu().numpy()
    ok, worst = rel_close(flat, want, TOL)
    assert ok, worst
    fused = ops.vecq_fused(t, dev(w, device), dev(x, device), k, n, tokens=tokens).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), flat.view(np.uint32))
    # A token's values do not depend on the tokens beside it (one token a pass and four).
    alone = ops.vecq(t, dev(w, device), dev(q8[tokens - 1:], device), k, n).cpu().numpy()
    assert np.array_equal(alone[0].view(np.uint32), got[tokens - 1].view(np.uint32))


@pytest.mark.parametrize("t", LEGACY)
def test_legacy_block_sums_and_random_bytes(device, t):
    k, n = 2048, 19
    w = synth.random_blocks(t, n, k, 411)
    q8 = oracle.q8_1_quantize(synth.activations(2, k, 412))
    want = oracle.vecq_block_sums(t, w, q8[:1], k, n)
    got = ops.vecq_block_sums(t, dev(w, device), dev(q8[:1], device), k, n).cpu().numpy()
    assert np.array_equal(got, want)
    y = ops.vecq(t, dev(w, device), dev(q8, device), k, n, tokens=2).cpu().numpy()
    ok, worst = rel_close(y, oracle.vecq(t, w, q8, k, n, tokens=2), TOL)
    assert ok, worst


@pytest.mark.parametrize("t", LEGACY)
@pytest.mark.parametrize("tokens", [1, 5])
def test_legacy_blocks_glu_and_routed_match_oracle(device, t, tokens):
    k, n, experts, used = 1024, 40, 6, 2
    gate, up = synth.legacy_weights(t, n, k, 421), synth.legacy_weights(t, n, k, 422)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 423))
    want = oracle.vecq(t, up, q8, k, n, gate=gate, tokens=tokens, glu=oracle.GLU_SWIGLU)
    got = ops.vecq(t, dev(up, device), dev(q8, device), k, n, gate=dev(gate, device), tokens=tokens,
                   glu=ops.GLU_SWIGLU).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    w = synth.legacy_weights(t, experts * n, k, 424).reshape(experts, -1)
    g = synth.rng(425)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    stride_expert = n * (k // 32)
    want = oracle.vecq(t, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


def test_q4_0_refuses_what_the_streaming_form_does_not_take(device):
    k, n = 288, 4  # whole 32-value blocks, not whole 256
    w = synth.legacy_weights(Q4_0, n, k, 431)
    q8 = oracle.q8_1_quantize(synth.activations(1, k, 432))
    with pytest.raises(ops.KernelFailure):
        ops.vecq(Q4_0, dev(w, device), dev(q8, device), k, n)
    with pytest.raises(ops.KernelFailure):  # the rows form has no Q4_0
        ops.vecq(Q4_0, dev(synth.legacy_weights(Q4_0, n, 256, 433), device), dev(q8, device), 256, n, variant=0)


# ---- Q5_K through the streaming form (a 176-byte super-block a lane)

Q5_K = ops.TYPE_Q5_K


@pytest.mark.parametrize("k,n", [(4096, 96), (256, 5), (3840, 33), (15360, 12), (20480, 7)])
@pytest.mark.parametrize("tokens", [1, 3, 4, 9])
def test_q5_k_dense_matches_oracle(device, k, n, tokens):
    """Q4_K's products with a fifth bit a code (src/format/encoding.cc:116, src/kernels/ggml/vecq.cu:74-75 of the
    reference): rows of one tile, of fewer waves, and in pieces; quantizing in the kernel gives the same bits, and a
    token's values do not depend on the tokens beside it."""
    w = synth.q5_k_weights(n, k, 601 + k + n)
    x = synth.activations(tokens, k, 602 + tokens)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(Q5_K, w, q8, k, n, tokens=tokens)
    got = ops.vecq(Q5_K, dev(w, device), dev(q8, device), k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    fused = ops.vecq_fused(Q5_K, dev(w, device), dev(x, device), k, n, tokens=tokens).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), got.view(np.uint32))
    alone = ops.vecq(Q5_K, dev(w, device), dev(q8[tokens - 1:], device), k, n).cpu().numpy()
    assert np.array_equal(alone[0].view(np.uint32), got[tokens - 1].view(np.uint32))


def test_q5_k_block_sums_and_random_bytes(device):
    k, n = 2048, 19
    w = synth.random_blocks(Q5_K, n, k, 611)
    q8 = oracle.q8_1_quantize(synth.activations(2, k, 612))
    want = oracle.vecq_block_sums(Q5_K, w, q8[:1], k, n)
    got = ops.vecq_block_sums(Q5_K, dev(w, device), dev(q8[:1], device), k, n).cpu().numpy()
    assert np.array_equal(got, want)
    y = ops.vecq(Q5_K, dev(w, device), dev(q8, device), k, n, tokens=2).cpu().numpy()
    ok, worst = rel_close(y, oracle.vecq(Q5_K, w, q8, k, n, tokens=2), TOL)
    assert ok, worst


@pytest.mark.parametrize("tokens", [1, 5])
def test_q5_k_glu_and_routed_match_oracle(device, tokens):
    k, n, experts, used = 1024, 40, 6, 2
    gate, up = synth.q5_k_weights(n, k, 621), synth.q5_k_weights(n, k, 622)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 623))
    want = oracle.vecq(Q5_K, up, q8, k, n, gate=gate, tokens=tokens, glu=oracle.GLU_GEGLU)
    got = ops.vecq(Q5_K, dev(up, device), dev(q8, device), k, n, gate=dev(gate, device), tokens=tokens,
                   glu=ops.GLU_GEGLU).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    w = synth.q5_k_weights(experts * n, k, 624).reshape(experts, -1)
    g = synth.rng(625)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    stride_expert = n * (k // 256)
    want = oracle.vecq(Q5_K, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(Q5_K, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


def test_q5_k_refuses_the_other_forms(device):
    k, n = 512, 8
    w = synth.q5_k_weights(n, k, 631)
    q8 = oracle.q8_1_quantize(synth.activations(1, k, 632))
    with pytest.raises(ops.KernelFailure):  # the rows form has no Q5_K
        ops.vecq(Q5_K, dev(w, device), dev(q8, device), k, n, variant=0)


# ---- Q6_K through the streaming form (a 210-byte block a lane, every dword put together from two)

Q6_K = ops.TYPE_Q6_K


@pytest.mark.parametrize("k,n", [(4096, 96), (2048, 40), (8192, 10), (14336, 7), (5120, 6), (256, 32), (3840, 24),
                                 (1280, 40), (768, 8)])
@pytest.mark.parametrize("tokens", [1, 3, 4, 9])
def test_q6_k_dense_matches_oracle(device, k, n, tokens):
    """src/format/encoding.cc:117, src/kernels/ggml/vecq.cu:76-77 of the reference: tiles that are whole 16-byte chunks
    and tiles of 60, 63 and 24 blocks that start 0 to 14 bytes past a boundary, lanes whose block starts 0 or 2 bytes
    into a dword; quantizing in the kernel gives the same bits, and a token's values do not depend on the tokens
    beside it."""
    w = synth.q6_k_weights(n, k, 701 + k + n)
    x = synth.activations(tokens, k, 702 + tokens)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(Q6_K, w, q8, k, n, tokens=tokens)
    got = ops.vecq(Q6_K, dev(w, device), dev(q8, device), k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    fused = ops.vecq_fused(Q6_K, dev(w, device), dev(x, device), k, n, tokens=tokens).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), got.view(np.uint32))
    alone = ops.vecq(Q6_K, dev(w, device), dev(q8[tokens - 1:], device), k, n).cpu().numpy()
    assert np.array_equal(alone[0].view(np.uint32), got[tokens - 1].view(np.uint32))


def test_q6_k_block_sums_and_random_bytes(device):
    k, n = 2048, 24
    w = synth.random_blocks(Q6_K, n, k, 711)
    q8 = oracle.q8_1_quantize(synth.activations(2, k, 712))
    want = oracle.vecq_block_sums(Q6_K, w, q8[:1], k, n)
    got = ops.vecq_block_sums(Q6_K, dev(w, device), dev(q8[:1], device), k, n).cpu().numpy()
    assert np.array_equal(got, want)
    y = ops.vecq(Q6_K, dev(w, device), dev(q8, device), k, n, tokens=2).cpu().numpy()
    ok, worst = rel_close(y, oracle.vecq(Q6_K, w, q8, k, n, tokens=2), TOL)
    assert ok, worst


@pytest.mark.parametrize("tokens", [1, 5])
@pytest.mark.parametrize("k", [1024, 3840])
def test_q6_k_glu_and_routed_match_oracle(device, tokens, k):
    n, experts, used = 40, 6, 2
    gate, up = synth.q6_k_weights(n, k, 721), synth.q6_k_weights(n, k, 722)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 723))
    want = oracle.vecq(Q6_K, up, q8, k, n, gate=gate, tokens=tokens, glu=oracle.GLU_SWIGLU)
    got = ops.vecq(Q6_K, dev(up, device), dev(q8, device), k, n, gate=dev(gate, device), tokens=tokens,
                   glu=ops.GLU_SWIGLU).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    w = synth.q6_k_weights(experts * n, k, 724).reshape(experts, -1)
    g = synth.rng(725)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    stride_expert = n * (k // 256)
    want = oracle.vecq(Q6_K, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(Q6_K, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


def test_q6_k_refuses_tiles_that_are_not_whole_chunks(device):
    q8 = oracle.q8_1_quantize(synth.activations(1, 3840, 732))
    with pytest.raises(ops.KernelFailure):  # 3 rows of 15 blocks: the matrix ends within a 16-byte chunk
        ops.vecq(Q6_K, dev(synth.q6_k_weights(3, 3840, 731), device), dev(q8, device), 3840, 3)
    q8 = oracle.q8_1_quantize(synth.activations(1, 5120, 734))
    with pytest.raises(ops.KernelFailure):  # three rows of 20 blocks: the last tile would end within a chunk
        ops.vecq(Q6_K, dev(synth.q6_k_weights(3, 5120, 733), device), dev(q8, device), 5120, 3)
    q8 = oracle.q8_1_quantize(synth.activations(1, 4096, 736))
    with pytest.raises(ops.KernelFailure):  # the rows form has no Q6_K
        ops.vecq(Q6_K, dev(synth.q6_k_weights(8, 4096, 735), device), dev(q8, device), 4096, 8, variant=0)


@pytest.mark.parametrize("t", [ops.TYPE_Q5_K, ops.TYPE_Q6_K, ops.TYPE_IQ4_NL])
@pytest.mark.parametrize("k", [2048, 3840])
def test_sorted_rows_equal_routed_pairs_for_the_added_types(device, t, k):
    """Rows sorted by expert (the offsets of llmp.moe.route) against the same pairs under routing ids, bit for bit, and
    the routed product against the oracle."""
    n, experts, tokens, used = 16, 5, 6, 2
    if t == ops.TYPE_IQ4_NL and k % 256:
        pytest.skip("rows of whole 256 values")
    make = {ops.TYPE_Q5_K: synth.q5_k_weights, ops.TYPE_Q6_K: synth.q6_k_weights,
            ops.TYPE_IQ4_NL: lambda n_, k_, seed: synth.legacy_weights(ops.TYPE_IQ4_NL, n_, k_, seed)}[t]
    w = make(experts * n, k, 801).reshape(experts, -1)
    g = synth.rng(802)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 803))
    stride_expert = n * (k // oracle.block_elements(t))
    want = oracle.vecq(t, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(t, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    order = np.argsort(ids.reshape(-1), kind="stable")
    offsets = np.concatenate([[0], np.cumsum(np.bincount(ids.reshape(-1), minlength=experts))]).astype(np.int32)
    rows = np.ascontiguousarray(q8.reshape(tokens, -1)[order // used])
    sorted_out = ops.vecq_sorted(t, dev(w, device), dev(rows, device), dev(offsets, device), k, n, experts,
                                 stride_expert=stride_expert).cpu().numpy()
    assert np.array_equal(sorted_out.view(np.uint32), got.reshape(tokens * used, n)[order].view(np.uint32))


# ---- MXFP4 through the streaming form (eight 17-byte blocks a lane)

MXFP4 = ops.TYPE_MXFP4


@pytest.mark.parametrize("k,n", [(4096, 96), (512, 5), (2560, 33), (15360, 12), (20480, 7)])
@pytest.mark.parametrize("tokens", [1, 3, 4, 9])
def test_mxfp4_dense_matches_oracle(device, k, n, tokens):
    """src/kernels/ggml/vecq.cu:421-437 over the values of src/kernels/reference/decode.cc:239-248:
    (2^(e - 127) / 2 * d8) * sum(twice the E2M1 values * q). Rows of one tile, of fewer waves, and
    in pieces; quantized beforehand or in the kernel; a token alone or among others."""
    w = synth.mxfp4_weights(n, k, 501 + k + n)
    x = synth.activations(tokens, k, 502 + tokens)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(MXFP4, w, q8, k, n, tokens=tokens)
    got = ops.vecq(MXFP4, dev(w, device), dev(q8, device), k, n, tokens=tokens).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    fused = ops.vecq_fused(MXFP4, dev(w, device), dev(x, device), k, n, tokens=tokens).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), got.view(np.uint32))
    alone = ops.vecq(MXFP4, dev(w, device), dev(q8[tokens - 1:], device), k, n).cpu().numpy()
    assert np.array_equal(alone[0].view(np.uint32), got[tokens - 1].view(np.uint32))


def test_mxfp4_block_sums_and_every_scale_byte(device):
    """The int32 sums bit for bit over random bytes; then every scale byte there is, subnormal
    (0 and 1) and NaN (0xFF) included, one block a row so that each output is one block's term."""
    k, n = 2048, 19
    w = synth.random_blocks(MXFP4, n, k, 511)
    q8 = oracle.q8_1_quantize(synth.activations(2, k, 512))
    want = oracle.vecq_block_sums(MXFP4, w, q8[:1], k, n)
    got = ops.vecq_block_sums(MXFP4, dev(w, device), dev(q8[:1], device), k, n).cpu().numpy()
    assert np.array_equal(got, want)
    y = ops.vecq(MXFP4, dev(w, device), dev(q8, device), k, n, tokens=2).cpu().numpy()
    ok, worst = rel_close(y, oracle.vecq(MXFP4, w, q8, k, n, tokens=2), TOL)
    assert ok, worst
    k, n = 512, 256
    w = np.zeros((n, k // 32, 17), dtype=np.uint8)
    w[:, :, 0] = 127
    for r in range(n):  # row r: block r % 16 holds codes and scale byte r, the others zeros
        w[r, r % 16, 0] = r
        w[r, r % 16, 1:] = synth.rng(513 + r).integers(0, 256, size=16, dtype=np.uint8)
    w = w.reshape(n, -1)
    q8 = oracle.q8_1_quantize(synth.activations(1, k, 514) * 1e-3)
    want = oracle.vecq(MXFP4, w, q8, k, n)[0, 0]
    got = ops.vecq(MXFP4, dev(w, device), dev(q8, device), k, n).cpu().numpy().reshape(-1)
    assert np.isnan(got[255]) and np.isnan(want[255])
    # Half the scale times d8 (about 2^-15 here) is exact while it is a normal float: one rounding,
    # the same bits. Below that (scale bytes under 20) the product is subnormal and loses bits.
    assert np.array_equal(got[20:255].view(np.uint32), want[20:255].view(np.uint32))
    assert np.allclose(got[:20], want[:20], rtol=0.1, atol=1e-44) and np.all(np.sign(got[:20]) == np.sign(want[:20]))


@pytest.mark.parametrize("tokens", [1, 5])
def test_mxfp4_glu_and_routed_match_oracle(device, tokens):
    k, n, experts, used = 1024, 40, 6, 2
    gate, up = synth.mxfp4_weights(n, k, 521), synth.mxfp4_weights(n, k, 522)
    q8 = oracle.q8_1_quantize(synth.activations(tokens, k, 523))
    want = oracle.vecq(MXFP4, up, q8, k, n, gate=gate, tokens=tokens, glu=oracle.GLU_SWIGLU)
    got = ops.vecq(MXFP4, dev(up, device), dev(q8, device), k, n, gate=dev(gate, device), tokens=tokens,
                   glu=ops.GLU_SWIGLU).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    w = synth.mxfp4_weights(experts * n, k, 524).reshape(experts, -1)
    g = synth.rng(525)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    stride_expert = n * (k // 32)
    want = oracle.vecq(MXFP4, w, q8, k, n, ids=ids, tokens=tokens, used=used, stride_expert=stride_expert, experts=experts)
    got = ops.vecq(MXFP4, dev(w, device), dev(q8, device), k, n, ids=dev(ids, device), tokens=tokens, used=used,
                   stride_expert=stride_expert).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst


def test_mxfp4_refuses_what_the_streaming_form_does_not_take(device):
    k, n = 768, 4  # whole 256 values, not whole 512: a row would start off a 16-byte boundary
    w = synth.mxfp4_weights(n, k, 531)
    q8 = oracle.q8_1_quantize(synth.activations(1, k, 532))
    with pytest.raises(ops.KernelFailure):
        ops.vecq(MXFP4, dev(w, device), dev(q8, device), k, n)
    with pytest.raises(ops.KernelFailure):  # the rows form has no MXFP4
        ops.vecq(MXFP4, dev(synth.mxfp4_weights(n, 512, 533), device), dev(q8, device), 512, n, variant=0)


@pytest.mark.parametrize("tokens,glu", [(2, ops.GLU_NONE), (4, ops.GLU_GEGLU), (8, ops.GLU_SWIGLU)])
def test_relaid_out_rows_equal_the_row_a_lane_form_bit_for_bit(device, tokens, glu):
    """llmp_hip_relayout_q4_k_tiles64 permutes whole blocks inside 64-row tiles and its inverse puts them back; the
    variant that reads the result multiplies the same blocks with the same arithmetic as the row-a-lane form over the
    reference's layout: equal bits, and the oracle's values. Dense and grouped (two matrices, two input rows)."""
    k, n, used = 1280, 192, 2
    names = ops.vecq_variants()
    rows_variant, tiled_variant = names.index("rows pass8 rows64"), names.index("rows pass8 tiles64")
    up = make_weights(Q4_K, used * n, k, 301)
    gate = make_weights(Q4_K, used * n, k, 302) if glu != ops.GLU_NONE else None
    q8 = oracle.q8_1_quantize(synth.activations(tokens * used, k, 303))
    ud, qd = dev(up, device), dev(q8, device)
    gd = dev(gate, device) if gate is not None else None
    ut = ops.relayout_q4_k_tiles64(ud, used * n, k)
    gt = ops.relayout_q4_k_tiles64(gd, used * n, k) if gd is not None else None
    assert not torch.equal(ut, ud)
    assert torch.equal(ops.relayout_q4_k_tiles64(ut, used * n, k, inverse=True), ud)
    # What the layout is: block (row, sb) at block (sb, row % 64) of its tile.
    nsb = k // 256
    native, tiled = up.reshape(-1, nsb, 144), ut.cpu().numpy().reshape(-1, nsb, 64, 144)
    for row, sb in ((0, 0), (63, nsb - 1), (64, 1), (used * n - 1, 2)):
        assert np.array_equal(tiled[row // 64, sb, row % 64], native[row, sb])
    blocks = oracle.padded_k(k) // 32
    common = dict(tokens=tokens, used=used, stride_expert=n * nsb, y_token=blocks * used, y_slot=blocks, glu=glu)
    want = ops.vecq(Q4_K, ud, qd, k, n, gate=gd, variant=rows_variant, **common)
    got = ops.vecq(Q4_K, ut, qd, k, n, gate=gt, variant=tiled_variant, **common)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    ref = oracle.vecq(Q4_K, up, q8, k, n, gate=gate, tokens=tokens, used=used, stride_expert=n * nsb, y_token=blocks * used,
                      y_slot=blocks, glu=glu)
    ok, worst = rel_close(got.cpu().numpy(), ref, TOL)
    assert ok, worst
    # Rows that are not whole tiles are refused, nothing queued.
    with pytest.raises(ops.KernelFailure) as refused:
        ops.vecq(Q4_K, ut, qd, k, n - 8, gate=gt, variant=tiled_variant, **common)
    assert refused.value.rejected


@pytest.mark.parametrize("tokens,glu,k", [(2, ops.GLU_NONE, 640), (4, ops.GLU_GEGLU, 1536), (8, ops.GLU_SWIGLU, 1536), (7, ops.GLU_NONE, 4096),
                                           (8, ops.GLU_NONE, 14336), (6, ops.GLU_SWIGLU, 9472)])
def test_q8_0_rows_form_over_relaid_out_weights(device, tokens, glu, k):
    """llmp_hip_relayout_q8_0_tiles64 (codes and scales apart, 64-row tiles, four blocks a piece) and the row-a-lane
    variant that reads it for Q8_0: the layout is what the header says, the inverse gives the file's bytes back, the
    products are the oracle's (integer block sums on the matrix instruction are exact; what is left is the order of
    the float sums, 1e-3), a token's values do not depend on the tokens beside it, and shapes the form does not take
    are refused. Dense and grouped (two matrices, two input rows)."""
    n, used = 192, 2
    tiled_variant = ops.vecq_variants().index("rows pass8 tiles64")
    up = make_weights(Q8_0, used * n, k, 311)
    gate = make_weights(Q8_0, used * n, k, 312) if glu != ops.GLU_NONE else None
    q8 = oracle.q8_1_quantize(synth.activations(tokens * used, k, 313))
    ud, qd = dev(up, device), dev(q8, device)
    ut = ops.relayout_q8_0_tiles64(ud, used * n, k)
    gt = ops.relayout_q8_0_tiles64(dev(gate, device), used * n, k) if gate is not None else None
    assert not torch.equal(ut, ud)
    assert torch.equal(ops.relayout_q8_0_tiles64(ut, used * n, k, inverse=True), ud)
    units = k // 128
    native = up.reshape(-1, units, 4, 34)                      # [row][unit][block][d, 32 codes]
    tiled = ut.cpu().numpy().reshape(-1, units, 8704)          # [tile][unit][piece]
    for row, unit in ((0, 0), (63, units - 1), (64, 1), (used * n - 1, 2), (77, 3)):
        piece, r = tiled[row // 64, unit], row % 64
        for b in range(4):
            assert np.array_equal(piece[8192 + r * 8 + 2 * b:8192 + r * 8 + 2 * b + 2], native[row, unit, b, :2])
            for half in range(2):
                c = 2 * b + half
                at = r * 128 + ((c ^ (r & 7)) << 4)
                assert np.array_equal(piece[at:at + 16], native[row, unit, b, 2 + 16 * half:18 + 16 * half])
    blocks = oracle.padded_k(k) // 32
    common = dict(used=used, stride_expert=n * (k // 32), y_token=blocks * used, y_slot=blocks, glu=glu)
    got = ops.vecq(Q8_0, ut, qd, k, n, gate=gt, variant=tiled_variant, tokens=tokens, **common)
    ref = oracle.vecq(Q8_0, up, q8, k, n, gate=gate, tokens=tokens, **common)
    ok, worst = rel_close(got.cpu().numpy(), ref, TOL)
    assert ok, worst
    # The default form over the file's layout computes the same definition.
    same = ops.vecq(Q8_0, ud, qd, k, n, gate=dev(gate, device) if gate is not None else None, tokens=tokens, **common)
    ok, worst = rel_close(got.cpu().numpy(), same.cpu().numpy(), TOL)
    assert ok, worst
    # Two of the tokens alone (another instance of the kernel where the count crosses four): the same bits.
    pair = ops.vecq(Q8_0, ut, qd, k, n, gate=gt, variant=tiled_variant, tokens=2, **common)
    assert torch.equal(pair.view(torch.int32), got[:2].view(torch.int32))
    for bad in (dict(nrows=n - 8), dict(tokens=1), dict(tokens=9)):
        with pytest.raises(ops.KernelFailure) as refused:
            ops.vecq(Q8_0, ut, qd, k, bad.get("nrows", n), gate=gt, variant=tiled_variant, tokens=bad.get("tokens", tokens), **common)
        assert refused.value.rejected
    # The row-a-lane form over the file's layout (rows of whole 256 values) in tiles of 64 rows: the same arithmetic,
    # the same bits. In tiles of 32 and 16 rows (and the launcher's choice among the three) the sums meet in another
    # order: the oracle's values, and a token's own whatever the tokens beside it.
    rows_variant = ops.vecq_variants().index("rows pass8 rows64")
    gd = dev(gate, device) if gate is not None else None
    if k % 256 == 0:
        native = ops.vecq(Q8_0, ud, qd, k, n, gate=gd, variant=rows_variant, tokens=tokens, **common)
        assert torch.equal(native.view(torch.int32), got.view(torch.int32))
        for name in ("rows pass8", "rows pass8 rows32", "rows pass8 rows16"):
            narrow_variant = ops.vecq_variants().index(name)
            if k // 512 < (4 if name.endswith("rows16") else 2 if name.endswith("rows32") else 1):
                continue  # a wave's quarter of a row is at least a piece: two units are 1024 values a row, four 2048
            narrow = ops.vecq(Q8_0, ud, qd, k, n, gate=gd, variant=narrow_variant, tokens=tokens, **common)
            ok, worst = rel_close(narrow.cpu().numpy(), ref, TOL)
            assert ok, (name, worst)
            two = ops.vecq(Q8_0, ud, qd, k, n, gate=gd, variant=narrow_variant, tokens=2, **common)
            assert torch.equal(two.view(torch.int32), narrow[:2].view(torch.int32)), name
        # Fewer rows than whole tiles, and rows apart (a pitch of eight blocks more): the form's own edges.
        pitched = torch.zeros((used * n, k // 32 + 8, 34), dtype=torch.uint8, device=device)
        pitched[:, :k // 32] = ud.view(used * n, k // 32, 34)
        wide = dict(common, stride_expert=n * (k // 32 + 8))
        short = ops.vecq(Q8_0, pitched.view(-1), qd, k, n - 24, variant=rows_variant, tokens=tokens, stride_row=k // 32 + 8, **dict(wide, glu=ops.GLU_NONE))
        plain = got if glu == ops.GLU_NONE else ops.vecq(Q8_0, ut, qd, k, n, variant=tiled_variant, tokens=tokens, **dict(common, glu=ops.GLU_NONE))
        assert torch.equal(short.view(torch.int32), plain[:, :, :n - 24].contiguous().view(torch.int32))
        # The same edges in the narrower tiles (the launcher's choice here): the oracle's values.
        narrow_short = ops.vecq(Q8_0, pitched.view(-1), qd, k, n - 24, tokens=tokens, stride_row=k // 32 + 8,
                                variant=ops.vecq_variants().index("rows pass8"), **dict(wide, glu=ops.GLU_NONE))
        ok, worst = rel_close(narrow_short.cpu().numpy(), plain[:, :, :n - 24].cpu().numpy(), TOL)
        assert ok, worst
    else:
        with pytest.raises(ops.KernelFailure):
            ops.vecq(Q8_0, ud, qd, k, n, gate=gd, variant=rows_variant, tokens=tokens, **common)
