"""Parity at the benchmark's own geometries: the launches `bench.py` times are the launches checked
here, at full size, against the CPU oracle over the same seeded inputs (the oracle finishes each in
well under a second on the host cores). Integer intermediates bit for bit; float outputs to a
maximum relative error of 1e-3 (accumulation order only).

Follows tests/unit/dsv4_fast_test.cc:1441-1633 (the products at a model's real shapes) and
tests/unit/exl3_trellis_test.cc:519-564 (the linear against the decoded rows) of the reference."""
import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu

Q8_0, Q4_K = ops.TYPE_Q8_0, ops.TYPE_Q4_K
TOL = 1e-3
# A GLU output is a product of two sums of thousands of terms that cancel: where it comes out under a hundredth of
# the output's RMS it is held to 1e-5 of the RMS (FP32 accumulation in another order than the oracle's doubles moves
# it by about 1e-6 of the RMS; the reference's own check, tests/unit/dsv4_fast_test.cc:419, allows 2e-5 absolute).
GLU_FLOOR = 1e-2


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def halves(a, device):
    return dev(np.ascontiguousarray(a).view(np.int16), device).view(torch.float16)


def test_config_1_q8_0_4096_x_4096(device):
    """GGML Q8_0 mat-vec, N = K = 4096, one F32 token through llmp.q8_1: the quantized activations and the
    int32 block sums bit for bit, y within 1e-3, on the default variant and every other that takes the shape."""
    n = k = 4096
    w = synth.q8_0_weights(n, k, 201)
    x = synth.activations(1, k, 202)
    q8 = oracle.q8_1_quantize(x)
    q8_got = ops.quantize_q8_1(dev(x, device))
    assert np.array_equal(q8_got.cpu().numpy(), q8)
    sums = ops.vecq_block_sums(Q8_0, dev(w, device), q8_got, k, n).cpu().numpy()
    assert np.array_equal(sums, oracle.vecq_block_sums(Q8_0, w, q8, k, n))
    want = oracle.vecq(Q8_0, w, q8, k, n, threads=oracle.max_threads())
    wd = dev(w, device)
    got = ops.vecq(Q8_0, wd, q8_got, k, n).cpu().numpy()
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    fused = ops.vecq_fused(Q8_0, wd, dev(x, device), k, n).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), got.view(np.uint32))
    for variant, name in enumerate(ops.vecq_variants()):
        try:
            other = ops.vecq(Q8_0, wd, q8_got, k, n, variant=variant).cpu().numpy()
        except ops.KernelFailure as refused:  # a variant the shape cannot take: nothing was queued
            assert refused.rejected, name
            continue
        ok, worst = rel_close(other, want, TOL)
        assert ok, (name, worst)


@pytest.mark.parametrize("tokens", [1, 4, 8])
def test_config_2_q4_k_gate_up_geglu_3840_x_15360(device, tokens):
    """The fused gate/up pair at decode, K = 3840 (15 super-blocks a row: 60 of a wave's 64 lanes), N = 2 x 15360,
    bf16 activations at batch 1, 4 and 8: q8_1 bit for bit, GEGLU(gate) * up within 1e-3 of the oracle; the form
    that quantizes in the kernel gives the same bits; each token's values are those of its own one-token launch."""
    k, n = 3840, 15360
    gate, up = synth.q4_k_weights(n, k, 101), synth.q4_k_weights(n, k, 102)
    x = synth.bf16_to_f32(synth.bf16_bits(synth.activations(tokens, k, 103)))
    q8 = oracle.q8_1_quantize(x)
    q8_got = ops.quantize_q8_1(dev(x, device))
    assert np.array_equal(q8_got.cpu().numpy(), q8)
    want = oracle.vecq(Q4_K, up, q8, k, n, gate=gate, tokens=tokens, glu=oracle.GLU_GEGLU, threads=oracle.max_threads())
    gd, ud = dev(gate, device), dev(up, device)
    got = ops.vecq(Q4_K, ud, q8_got, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU).cpu().numpy()
    assert got.shape[-1] == n
    ok, worst = rel_close(got.reshape(tokens, n), want.reshape(tokens, n), TOL, floor=GLU_FLOOR)
    assert ok, worst
    xd = dev(x, device).to(torch.bfloat16)
    fused = ops.vecq_fused(Q4_K, ud, xd, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU).cpu().numpy()
    ok, worst = rel_close(fused.reshape(tokens, n), want.reshape(tokens, n), TOL, floor=GLU_FLOOR)
    assert ok, worst
    if tokens <= 4:  # the flat form at these counts: the bits of the two steps through it
        flat = ops.vecq(Q4_K, ud, q8_got, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU, variant=6 if tokens == 1 else 7)
        assert np.array_equal(fused.view(np.uint32), flat.cpu().numpy().view(np.uint32))
    # vecq.cu:688-693: a (token, row) value does not depend on the tokens scheduled beside it.
    again = ops.vecq(Q4_K, ud, q8_got, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))
    if tokens > 1:
        shuffled = q8_got.flip(0).contiguous()
        flipped = ops.vecq(Q4_K, ud, shuffled, k, n, gate=gd, tokens=tokens, glu=ops.GLU_GEGLU).cpu().numpy()
        assert np.array_equal(flipped.reshape(tokens, n)[::-1].view(np.uint32), got.reshape(tokens, n).view(np.uint32))


@pytest.mark.parametrize("t,k,n", [(Q4_K, 15360, 3840), (Q8_0, 14336, 4096)])
@pytest.mark.parametrize("tokens", [1, 2, 4, 8, 16])
def test_down_projection_at_full_size(device, t, k, n, tokens):
    """Config 2's down projection (15360 -> 3840, Q4_K: rows of 60 super-blocks, 60 tiles of 64 rows) and a Q8_0 one of
    the same kind (14336 -> 4096) at 1 to 16 tokens: the default forms (the flat form at one token, the row-a-lane form
    in tiles of 16 rows at 2 to 8, eight tokens in spans, sixteen in two launches) within 1e-3 of the oracle, and the
    same shape through the flat form's four-token passes, an independent kernel, within 1e-3 as well; a token's values
    do not move with the tokens beside it."""
    w = (synth.q4_k_weights if t == Q4_K else synth.q8_0_weights)(n, k, 111)
    x = synth.activations(tokens, k, 112)
    q8 = oracle.q8_1_quantize(x)
    want = oracle.vecq(t, w, q8, k, n, tokens=tokens, threads=oracle.max_threads()).reshape(tokens, n)
    wd, qd = dev(w, device), dev(q8, device)
    got = ops.vecq(t, wd, qd, k, n, tokens=tokens)
    ok, worst = rel_close(got.cpu().numpy().reshape(tokens, n), want, TOL)
    assert ok, worst
    flat = ops.vecq(t, wd, qd, k, n, tokens=tokens, variant=ops.vecq_variants().index("flat pass4" if tokens > 1 else "flat pass1"))
    ok, worst = rel_close(flat.cpu().numpy().reshape(tokens, n), want, TOL)
    assert ok, worst
    if tokens > 1:
        flipped = ops.vecq(t, wd, qd.flip(0).contiguous(), k, n, tokens=tokens)
        assert torch.equal(flipped.flip(0).view(torch.int32), got.view(torch.int32))
    if tokens in (4, 8):  # among fewer tokens (another instance of the kernel, the whole row staged at once): the same bits
        fewer = ops.vecq(t, wd, qd[:tokens // 2].contiguous(), k, n, tokens=tokens // 2)
        assert torch.equal(fewer.view(torch.int32), got[:tokens // 2].view(torch.int32))


def test_config_2_block_sums_at_full_size(device):
    """The eight products and eight sums of every super-block of the 15360 x 3840 gate matrix, bit for bit."""
    k, n = 3840, 15360
    gate = synth.q4_k_weights(n, k, 101)
    q8 = oracle.q8_1_quantize(synth.bf16_to_f32(synth.bf16_bits(synth.activations(1, k, 103))))
    got = ops.vecq_block_sums(Q4_K, dev(gate, device), dev(q8, device), k, n).cpu().numpy()
    assert np.array_equal(got, oracle.vecq_block_sums(Q4_K, gate, q8, k, n))


@pytest.mark.parametrize("m", [1, 16])
def test_config_5_exl3_4096_x_14336(device, m):
    """The EXL3 linear at 4 bits a weight with the 3INST codebook, K = 4096, N = 14336, one and sixteen rows: the
    transformed input within one F16 step of the oracle's, the product over the device's own transformed input
    within 1e-3, and the reference's bound against the F64 product of the decoded rows on a sample of columns."""
    k, n, bits, codebook = 4096, 14336, 4, ops.EXL3_3INST
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 208)
    x = synth.rng(209).standard_normal((m, k)).astype(np.float16)
    keep = {}
    got = ops.exl3_linear(dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook,
                          halves(x, device), keep=keep).cpu().numpy()
    a_had = keep["a_had"].cpu().numpy().view(np.uint16)
    want_had = oracle.exl3_input(suh.view(np.uint16), k, x.view(np.uint16))
    ulps = np.abs(a_had.view(np.int16).astype(np.int32) - want_had.view(np.int16).astype(np.int32))
    assert ulps.max() <= 1 and np.count_nonzero(ulps) <= 0.01 * ulps.size
    want = oracle.exl3_product(trellis, svh.view(np.uint16), k, n, bits, codebook, a_had, threads=oracle.max_threads())
    ok, worst = rel_close(got, want, TOL)
    assert ok, worst
    first, count = 5 * 128, 256  # two Hadamard blocks of columns
    rows = oracle.exl3_rows(trellis, suh.view(np.uint16), svh.view(np.uint16), k, n, bits, codebook, first=first,
                            count=count).astype(np.float64)
    ref = x.astype(np.float64) @ rows.T
    for r in range(m):
        part = got[r, first:first + count]
        assert np.sqrt(np.mean((part - ref[r]) ** 2)) <= 2.0 ** -8 * np.sqrt(np.mean(ref[r] ** 2))
    half = ops.exl3_linear(dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook,
                           halves(x, device), f32=False).cpu().numpy()
    assert np.array_equal(half.view(np.uint16), got.astype(np.float16).view(np.uint16))


def crowded_ids(counts, tokens, used, seed):
    """ids [tokens][used] whose pairs name expert e counts[e] times, in a seeded order."""
    pairs = np.concatenate([np.full(c, e, dtype=np.int32) for e, c in enumerate(counts)])
    assert pairs.size == tokens * used
    return synth.rng(seed).permutation(pairs).reshape(tokens, used)


@pytest.mark.parametrize("t,glu", [(Q4_K, True), (Q4_K, False), (Q8_0, False), (Q8_0, True)])
def test_sorted_rows_of_many_passes_match_oracle_and_the_routed_product(device, t, glu):
    """Experts with 17, 33, 40 and 38 rows: the matrix-core form takes an expert's rows sixteen a pass, so these
    run two and three passes. Against the oracle, 1e-3, and against the routed product of the same 128 pairs (its
    form is the one-token arithmetic)."""
    hidden, ffn, tokens, used = 2048, 768, 16, 8
    counts = [17, 33, 40, 0, 38]
    experts = len(counts)
    qk, bs = (256, 144) if t == Q4_K else (32, 34)
    per = ffn * (hidden // qk)  # blocks a matrix
    make = synth.q4_k_weights if t == Q4_K else synth.q8_0_weights
    weights = make(experts * (2 if glu else 1) * ffn, hidden, 71).reshape(experts, -1)
    ids = crowded_ids(counts, tokens, used, 72)
    x = synth.activations(tokens, hidden, 73)
    q8 = oracle.q8_1_quantize(x)
    stride = (2 if glu else 1) * per
    up = weights.reshape(-1)[per * bs:] if glu else weights
    want = oracle.vecq(t, up, q8, hidden, ffn, gate=weights if glu else None, ids=ids, tokens=tokens, used=used,
                       stride_expert=stride, glu=oracle.GLU_SWIGLU if glu else oracle.GLU_NONE, experts=experts,
                       threads=oracle.max_threads()).reshape(tokens * used, ffn)
    wd = dev(weights, device)
    upd = wd.view(-1)[per * bs:] if glu else wd
    kw = dict(gate=wd, glu=ops.GLU_SWIGLU) if glu else {}
    route = ops.moe_route(dev(ids, device), experts)
    assert np.array_equal(np.diff(route.offsets.cpu().numpy()), counts)
    sq8 = ops.quantize_q8_1_rows(dev(x, device), route.token)
    position = route.position.cpu().numpy()
    for variant in (-1, 7):  # the default (matrix cores) and the flat form's four-token passes
        got = ops.vecq_sorted(t, upd, sq8, route.offsets, hidden, ffn, experts, stride_expert=stride, variant=variant,
                              **kw).cpu().numpy()
        ok, worst = rel_close(got[position], want, TOL, floor=GLU_FLOOR if glu else 1e-3)
        assert ok, (variant, worst)
    routed = ops.vecq(t, upd, dev(q8, device), hidden, ffn, ids=dev(ids, device), tokens=tokens, used=used,
                      stride_expert=stride, **kw).cpu().numpy().reshape(tokens * used, ffn)
    ok, worst = rel_close(routed, want, TOL, floor=GLU_FLOOR if glu else 1e-3)
    assert ok, worst
    default = ops.vecq_sorted(t, upd, sq8, route.offsets, hidden, ffn, experts, stride_expert=stride, **kw).cpu().numpy()
    ok, worst = rel_close(default[position], routed, 1e-5, floor=1.0)  # two forms of the same sums: float order only
    assert ok, worst


def test_sorted_rows_beyond_the_routed_form(device):
    """700 pairs over six experts, one of them with 300 rows (nineteen passes) and one with none; the down
    projection's shape (K = 768: three super-blocks a row) and the gate/up shape."""
    experts, tokens, used = 6, 100, 7
    counts = [300, 1, 0, 150, 16, 233]
    ids = crowded_ids(counts, tokens, used, 81)
    for k, n, glu in ((768, 2048, False), (2048, 768, True)):
        per = n * (k // 256)
        weights = synth.q4_k_weights(experts * (2 if glu else 1) * n, k, 82 + k).reshape(experts, -1)
        x = synth.activations(tokens * used, k, 83)  # a row a pair: the down projection's per-slot activations
        q8 = oracle.q8_1_quantize(x)
        blocks = oracle.padded_k(k) // 32
        stride = (2 if glu else 1) * per
        up = weights.reshape(-1)[per * 144:] if glu else weights
        want = oracle.vecq(Q4_K, up, q8, k, n, gate=weights if glu else None, ids=ids, tokens=tokens, used=used,
                           stride_expert=stride, y_token=blocks * used, y_slot=blocks,
                           glu=oracle.GLU_SWIGLU if glu else oracle.GLU_NONE, experts=experts,
                           threads=oracle.max_threads()).reshape(tokens * used, n)
        wd = dev(weights, device)
        upd = wd.view(-1)[per * 144:] if glu else wd
        kw = dict(gate=wd, glu=ops.GLU_SWIGLU) if glu else {}
        route = ops.moe_route(dev(ids, device), experts)
        order, _ = oracle.expert_sort(ids, experts)
        sq8 = dev(q8[order], device)  # row r of the sorted activations is pair order[r]'s
        got = ops.vecq_sorted(Q4_K, upd, sq8, route.offsets, k, n, experts, stride_expert=stride, **kw).cpu().numpy()
        ok, worst = rel_close(got, want[order], TOL, floor=GLU_FLOOR if glu else 1e-3)
        assert ok, (k, worst)
