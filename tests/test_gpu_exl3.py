"""Parity of the EXL3 operations (HIP, through the C ABI) against the CPU oracle: reconstructed
weights bit for bit (every rate, the three codebooks), the transforms within F16/F32 rounding,
and the packed linear to a maximum relative error of 1e-3."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def halves(a, device):
    return dev(a.view(np.int16), device).view(torch.float16)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("codebook", [ops.EXL3_3INST, ops.EXL3_MCG, ops.EXL3_MUL1])
def test_reconstruct_is_the_rotated_decode_bit_for_bit(device, bits, codebook):
    """tests/unit/exl3_trellis_test.cc:446-465 of the reference."""
    k, n = 128, 256
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 100 + bits)
    want = oracle.exl3_rotated(trellis, k, n, bits, codebook)
    got = ops.exl3_reconstruct(dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), want)
    part = ops.exl3_reconstruct(dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook,
                                column=64, columns=96)
    assert np.array_equal(part.cpu().numpy().view(np.uint16), want[:, 64:160])


def test_every_state_of_every_codebook(device):
    """All 65,536 states: a 4-bit trellis whose stream walks them is not needed; a tile's positions
    see 256 states each, so 4096 random tiles cover the space densely; the golden vectors pin the rest."""
    k, n, bits = 1024, 1024, 4
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 7)
    for codebook in (ops.EXL3_3INST, ops.EXL3_MCG, ops.EXL3_MUL1):
        want = oracle.exl3_rotated(trellis, k, n, bits, codebook)
        got = ops.exl3_reconstruct(dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
        assert np.array_equal(got.cpu().numpy().view(np.uint16), want)


@pytest.mark.parametrize("bits,codebook", [(4, ops.EXL3_3INST), (3, ops.EXL3_MCG), (6, ops.EXL3_MUL1), (1, ops.EXL3_3INST),
                                           (8, ops.EXL3_MCG)])
def test_fused_reconstruction_is_the_weights(device, bits, codebook):
    """ReconstructOperands::fused (tests/unit/exl3_trellis_test.cc:467-518 of the reference): the weights with both
    transforms and side vectors applied, against the oracle's W in F64. The reference's bounds (relative L2 of a
    128 x 128 block 2^-7, any value within 2^-4 of its block's RMS) are for F16 butterflies; this kernel's transforms
    are F32 with one rounding to F16, so every value is also held to one F16 step of the oracle's (and F32's own error, which is of the block's size, not the value's)."""
    k, n = 384, 512
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 300 + bits)
    want = oracle.exl3_rows(trellis, suh, svh, k, n, bits, codebook).T  # [k][n]
    args = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
    got16 = ops.exl3_reconstruct(*args, fused=True)
    got = got16.float().cpu().numpy().astype(np.float64)
    for kb in range(0, k, 128):
        for nb in range(0, n, 128):
            w, g = want[kb:kb + 128, nb:nb + 128], got[kb:kb + 128, nb:nb + 128]
            rms = np.sqrt(np.mean(w.astype(np.float64) ** 2))
            assert np.sqrt(np.mean((g - w) ** 2)) / rms <= 2.0 ** -7
            assert np.abs(g - w).max() / rms <= 2.0 ** -4
    step = np.maximum(np.spacing(np.abs(want).astype(np.float16)).astype(np.float64), 2.0 ** -24)
    assert np.all(np.abs(got - want) <= step + 2e-6 * np.abs(want).max())  # F32's own error is of the block's size
    assert np.mean(got.astype(np.float16) != want.astype(np.float16)) < 2e-3  # ties and F32's last bits
    # A slice is the same columns of the whole.
    part = ops.exl3_reconstruct(*args, column=128, columns=256, fused=True)
    assert torch.equal(part, got16[:, 128:384])
    for column, columns in ((64, 128), (0, 64), (384, 256)):
        with pytest.raises(ops.KernelFailure):
            ops.exl3_reconstruct(*args, column=column, columns=columns, fused=True)


def hadamard_rows(x):
    idx = np.arange(128)
    h = np.where(np.array([[bin(i & j).count("1") % 2 for j in idx] for i in idx]) == 0, 1.0, -1.0)
    out = np.zeros_like(x, dtype=np.float64)
    for b in range(0, x.shape[1], 128):
        out[:, b:b + 128] = x[:, b:b + 128].astype(np.float64) @ h
    return out


def test_hadamard_transforms(device):
    g = synth.rng(9)
    rows, columns = 5, 384
    x = g.standard_normal((rows, columns)).astype(np.float16)
    scale = (g.choice([-1.0, 1.0], columns) * g.uniform(0.5, 1.5, columns)).astype(np.float16)
    r = 0.088388347648
    want_in = hadamard_rows(x.astype(np.float64) * scale.astype(np.float64)) * r
    got_in = ops.exl3_hadamard(halves(x, device), halves(scale, device), input_scale=True).float().cpu().numpy()
    np.testing.assert_allclose(got_in, want_in, rtol=2e-3, atol=2e-3)
    want_out = hadamard_rows(x) * r * scale.astype(np.float64)
    got_out = ops.exl3_hadamard(halves(x, device), halves(scale, device), input_scale=False).float().cpu().numpy()
    np.testing.assert_allclose(got_out, want_out, rtol=2e-3, atol=2e-3)
    xf = g.standard_normal((rows, columns)).astype(np.float32)
    got_f = ops.exl3_hadamard(dev(xf, device), halves(scale, device), input_scale=False).cpu().numpy()
    np.testing.assert_allclose(got_f, hadamard_rows(xf) * r * scale.astype(np.float64), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("m", [1, 2, 5, 16])
@pytest.mark.parametrize("bits,codebook", [(4, ops.EXL3_3INST), (4, ops.EXL3_MCG), (3, ops.EXL3_3INST), (6, ops.EXL3_MCG),
                                           (8, ops.EXL3_MUL1)])
def test_linear_matches_oracle(device, m, bits, codebook):
    k, n = 1024, 512
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 21 + bits)
    x = synth.rng(22 + m).standard_normal((m, k)).astype(np.float16)
    keep = {}
    got = ops.exl3_linear(dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook,
                          halves(x, device), keep=keep).cpu().numpy()
    # Stage one: the transformed input, F16. The device sums in F32, the oracle in F64, so a value
    # may round to the neighbouring F16 (rarely); nothing moves further.
    a_had = keep["a_had"].cpu().numpy().view(np.uint16)
    want_had = oracle.exl3_input(suh.view(np.uint16), k, x.view(np.uint16))
    ulps = np.abs(a_had.view(np.int16).astype(np.int32) - want_had.view(np.int16).astype(np.int32))
    assert ulps.max() <= 1 and np.count_nonzero(ulps) <= 0.01 * ulps.size
    # Stage two over identical transformed inputs: accumulation order only, 1e-3.
    want = oracle.exl3_product(trellis, svh.view(np.uint16), k, n, bits, codebook, a_had, threads=oracle.max_threads())
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst
    # And the reference's own bound against the F64 product with the decoded rows
    # (tests/unit/exl3_trellis_test.cc:519-564): relative RMS 2^-8 a row.
    rows = oracle.exl3_rows(trellis, suh.view(np.uint16), svh.view(np.uint16), k, n, bits, codebook).astype(np.float64)
    ref = x.astype(np.float64) @ rows.T
    for r in range(m):
        assert np.sqrt(np.mean((got[r] - ref[r]) ** 2)) <= 2.0 ** -8 * np.sqrt(np.mean(ref[r] ** 2))


def test_linear_rows_are_independent_and_f16_output_rounds_once(device):
    k, n, bits, codebook = 512, 256, 4, ops.EXL3_3INST
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 31)
    x = synth.rng(32).standard_normal((16, k)).astype(np.float16)
    args = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
    full = ops.exl3_linear(*args, halves(x, device)).cpu().numpy()
    solo = ops.exl3_linear(*args, halves(x[3:4], device)).cpu().numpy()
    assert np.array_equal(solo[0].view(np.uint32), full[3].view(np.uint32))
    half = ops.exl3_linear(*args, halves(x, device), f32=False).cpu().numpy()
    assert np.array_equal(half.view(np.uint16), full.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("m", [17, 40, 144])
def test_linear_of_more_than_sixteen_rows_runs_in_passes(device, m):
    """The packed path is upstream's choice through 144 rows (src/kernels/exl3/validate.h:254-256 of the
    reference): here sixteen rows a pass. Against the oracle over the device's transformed input, and each pass
    bit for bit the launch of its sixteen (or fewer) rows alone."""
    k, n, bits, codebook = 1024, 512, 4, ops.EXL3_3INST
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 71)
    x = synth.rng(72 + m).standard_normal((m, k)).astype(np.float16)
    args = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
    keep = {}
    got = ops.exl3_linear(*args, halves(x, device), keep=keep).cpu().numpy()
    a_had = keep["a_had"].cpu().numpy().view(np.uint16)
    want_had = oracle.exl3_input(suh.view(np.uint16), k, x.view(np.uint16))
    ulps = np.abs(a_had.view(np.int16).astype(np.int32) - want_had.view(np.int16).astype(np.int32))
    assert ulps.max() <= 1 and np.count_nonzero(ulps) <= 0.01 * ulps.size
    want = oracle.exl3_product(trellis, svh.view(np.uint16), k, n, bits, codebook, a_had, threads=oracle.max_threads())
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst
    for first in range(0, m, 16):
        alone = ops.exl3_linear(*args, halves(x[first:first + 16], device)).cpu().numpy()
        assert np.array_equal(alone.view(np.uint32), got[first:first + 16].view(np.uint32)), first
    if m == 40:
        up = synth.exl3_weights(k, n, bits, 73)
        second = (dev(up[0], device), halves(up[1], device), halves(up[2], device), k, n, bits, codebook)
        both = ops.exl3_multi_linear(args, second, halves(x, device)).cpu().numpy()
        assert np.array_equal(both[0].view(np.uint32), got.view(np.uint32))
        alone = ops.exl3_linear(*second, halves(x, device)).cpu().numpy()
        assert np.array_equal(both[1].view(np.uint32), alone.view(np.uint32))


@pytest.mark.parametrize("m,k,n,bits,codebook", [(200, 1024, 512, 4, ops.EXL3_3INST), (300, 256, 384, 3, ops.EXL3_MCG),
                                                 (1, 128, 128, 5, ops.EXL3_MUL1), (130, 128, 32768 + 256, 2, ops.EXL3_3INST)])
@pytest.mark.parametrize("fused", [True, False])
def test_reconstruction_paths_of_the_linear(device, m, k, n, bits, codebook, fused):
    """ReconstructedLinear (src/kernels/exl3/linear.cc:87-190 of the reference; its test
    tests/unit/exl3_trellis_test.cc:519-564): the weights reconstructed to F16 a slice at a time, a plain F16 product
    with F32 sums a slice; partial tiles of rows, two slices of columns. Against the F64 product with the decoded
    rows within the reference's bounds (2^-8 of a row's RMS; any output within 2^-5 of it), and stage by stage over
    the device's own reconstructed weights (and transformed input): what is left is the order of F32 sums, 1e-3."""
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 500 + bits)
    x = synth.rng(501 + m).standard_normal((m, k)).astype(np.float16)
    args = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
    got = ops.exl3_linear_reconstructed(*args, halves(x, device), f32=True, fused=fused).cpu().numpy().astype(np.float64)
    rows = oracle.exl3_rows(trellis, suh.view(np.uint16), svh.view(np.uint16), k, n, bits, codebook).astype(np.float64)
    ref = x.astype(np.float64) @ rows.T
    for r in range(m):
        rms = np.sqrt(np.mean(ref[r] ** 2))
        assert np.sqrt(np.mean((got[r] - ref[r]) ** 2)) <= 2.0 ** -8 * rms
        assert np.abs(got[r] - ref[r]).max() <= 2.0 ** -5 * rms
    if fused:
        w = np.concatenate([ops.exl3_reconstruct(*args, column=c, columns=min(32768, n - c), fused=True).float().cpu().numpy()
                            for c in range(0, n, 32768)], axis=1).astype(np.float64)
        want = x.astype(np.float64) @ w
        ok, worst = rel_close(got, want, 1e-3)
        assert ok, worst
    else:
        # The same definition as the packed path's: its output over the same rows agrees to the sums' order and the
        # rounding of the transformed input (one F16 step of a value in a hundred).
        packed = np.concatenate([ops.exl3_linear(*args, halves(x[i:i + 16], device)).cpu().numpy() for i in range(0, m, 16)])
        ok, worst = rel_close(got, packed.astype(np.float64), 2e-3)
        assert ok, worst
    half = ops.exl3_linear_reconstructed(*args, halves(x, device), f32=False, fused=fused).float().cpu().numpy()
    for r in range(0, m, 7):
        rms = np.sqrt(np.mean(ref[r] ** 2))
        assert np.sqrt(np.mean((half[r] - ref[r]) ** 2)) <= 2.0 ** -8 * rms


def test_reconstruction_path_refusals(device):
    k, n = 256, 256
    trellis, suh, svh = synth.exl3_weights(k, n, 4, 41)
    args = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, 4, 0)
    x = halves(synth.rng(1).standard_normal((8, k)).astype(np.float16), device)
    with pytest.raises(ops.KernelFailure) as e:
        ops.exl3_linear_reconstructed(*args, x, w=torch.empty(1024, dtype=torch.uint8, device=device))
    assert e.value.rejected and "scratch" in e.value.detail
    with pytest.raises(ops.KernelFailure):
        ops.exl3_linear_reconstructed(*args, x[:0])


def test_refusals(device):
    trellis, suh, svh = synth.exl3_weights(128, 128, 4, 41)
    x = halves(np.zeros((2, 128), dtype=np.float16), device)
    # An in-place linear (a_had and y on x) is refused before anything is queued (validate.cc:120-126).
    op = ops.Exl3Linear()
    op.weights = ops._exl3_weights(dev(trellis, device), halves(suh, device), halves(svh, device), 128, 128, 4, 0)
    op.x, op.a_had, op.y, op.f32, op.m = x.data_ptr(), x.data_ptr(), x.data_ptr(), 0, 2
    scratch = torch.empty(1 << 16, dtype=torch.uint8, device=device)
    lib = ops._lib.load()
    with pytest.raises(ops.KernelFailure) as e:
        ops._lib.check(lib.llmp_hip_exl3_linear(C.byref(op), scratch.data_ptr(), scratch.numel(), None))
    assert e.value.rejected and "overlaps" in e.value.detail
    with pytest.raises(ops.KernelFailure):
        ops.exl3_reconstruct(dev(trellis, device), halves(suh, device), halves(svh, device), 128, 128, 9, 0)
    with pytest.raises(ops.KernelFailure):
        ops.exl3_reconstruct(dev(trellis, device), halves(suh, device), halves(svh, device), 128, 128, 4, 0, column=8,
                             columns=16)


@pytest.mark.parametrize("m", [1, 3, 16])
@pytest.mark.parametrize("codebooks", [(ops.EXL3_3INST, ops.EXL3_3INST), (ops.EXL3_MCG, ops.EXL3_MUL1)])
@pytest.mark.parametrize("f32", [True, False])
def test_multi_linear_is_the_two_linears(device, m, codebooks, f32):
    """exl3.multi_linear (tests/unit/exl3_trellis_test.cc:664-716 of the reference): gate and up over one
    input, the first linear's rows then the second's, each against its own reference. Here each half
    is bit for bit the single linear's output (the same arithmetic in one launch), whose parity
    with the oracle the tests above hold; one half is checked against the oracle directly as well."""
    k, n, bits = 1024, 384, 4
    gate, up = synth.exl3_weights(k, n, bits, 51), synth.exl3_weights(k, n, bits, 52)
    x = synth.rng(53 + m).standard_normal((m, k)).astype(np.float16)
    first = (dev(gate[0], device), halves(gate[1], device), halves(gate[2], device), k, n, bits, codebooks[0])
    second = (dev(up[0], device), halves(up[1], device), halves(up[2], device), k, n, bits, codebooks[1])
    keep = {}
    got = ops.exl3_multi_linear(first, second, halves(x, device), f32=f32, keep=keep)
    assert got.shape == (2, m, n)
    word = torch.int32 if f32 else torch.int16
    for i, side in enumerate((first, second)):
        alone = {}
        want = ops.exl3_linear(*side, halves(x, device), f32=f32, keep=alone)
        assert torch.equal(got[i].view(word), want.view(word))
        assert torch.equal(keep["a_had"][i].view(torch.int16), alone["a_had"].view(torch.int16))
    if f32:
        a_had = keep["a_had"][1].cpu().numpy().view(np.uint16)
        want = oracle.exl3_product(up[0], up[2].view(np.uint16), k, n, bits, codebooks[1], a_had,
                                   threads=oracle.max_threads())
        ok, worst = rel_close(got[1].cpu().numpy(), want, 1e-3)
        assert ok, worst


def test_multi_linear_refusals(device):
    a, b = synth.exl3_weights(128, 128, 4, 61), synth.exl3_weights(128, 128, 3, 62)
    x = halves(np.zeros((2, 128), dtype=np.float16), device)
    first = (dev(a[0], device), halves(a[1], device), halves(a[2], device), 128, 128, 4, 0)
    second = (dev(b[0], device), halves(b[1], device), halves(b[2], device), 128, 128, 3, 0)
    with pytest.raises(ops.KernelFailure) as e:  # the two linears share k, n and the rate
        ops.exl3_multi_linear(first, second, x)
    assert e.value.rejected
