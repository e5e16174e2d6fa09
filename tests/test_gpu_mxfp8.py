"""Parity of the MXFP8 operations (HIP, through the C ABI) against the CPU oracle: the
quantizer's codes and scales and the swizzle bit for bit; the vector product to 1e-3; the
GEMM to 2e-2 against the float-accumulated product of the same quantized operands (and far
closer in aggregate)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def mixed_rows(rows, k, seed):
    g = synth.rng(seed)
    x = (g.standard_normal((rows, k)) * np.exp(g.uniform(-6, 6, (rows, 1)))).astype(np.float32)
    x[0, :32] = 0.0
    x[0, 40] = 448.0
    x[0, 41] = -1e9
    if rows > 1:
        x[1, :] *= 1e-30
    return x


@pytest.mark.parametrize("rows,k", [(1, 128), (5, 256), (130, 384), (2048, 4096)])
def test_quantize_is_bit_exact(device, rows, k):
    x = mixed_rows(rows, k, 3 + rows)
    want_codes, want_scales = oracle.mxfp8_quantize(x)
    codes, scales = ops.mxfp8_quantize(dev(x, device))
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(scales.cpu().numpy(), want_scales)


def test_quantize_takes_bf16_and_strided_rows(device):
    rows, k = 9, 256
    x = synth.bf16_to_f32(synth.bf16_bits(mixed_rows(rows, k, 5)))
    want_codes, want_scales = oracle.mxfp8_quantize(x)
    wide = torch.zeros((rows, k + 64), dtype=torch.bfloat16, device=device)
    wide[:, :k] = dev(x, device).to(torch.bfloat16)
    codes, scales = ops.mxfp8_quantize(wide[:, :k])
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(scales.cpu().numpy(), want_scales)


def test_every_float_to_e4m3_code(device):
    """All 256 codes' values, the midpoints between neighbours and the saturation edge through the
    device's conversion (a block whose scale is 2^0)."""
    values = np.array([oracle.lib.orc_e4m3_to_f32(c) for c in range(0x7F)], dtype=np.float64)
    mids = (values[:-1] + values[1:]) / 2
    probe = np.concatenate([values, mids, np.nextafter(mids.astype(np.float32), 1e9), [448.0, 300.0]]).astype(np.float32)
    probe = np.concatenate([probe, -probe])
    rows = -(-probe.size // 31)
    x = np.zeros((rows, 128), dtype=np.float32)
    for r in range(rows):
        chunk = probe[r * 31:(r + 1) * 31]
        x[r, 0] = 448.0  # pins the block's scale to 2^0
        x[r, 1:1 + chunk.size] = chunk
    want_codes, want_scales = oracle.mxfp8_quantize(x)
    codes, scales = ops.mxfp8_quantize(dev(x, device))
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(scales.cpu().numpy(), want_scales)


def test_swizzle_is_bit_exact(device):
    g = synth.rng(7)
    plain = g.integers(0, 255, size=(300, 12), dtype=np.uint8)
    assert np.array_equal(ops.mxfp8_swizzle(dev(plain, device)).cpu().numpy(), oracle.mxfp8_swizzle(plain))


@pytest.mark.parametrize("tokens", [1, 3, 8, 16])
def test_vector_product_matches_oracle(device, tokens):
    g = synth.rng(9)
    n, k = 200, 2560
    w = (g.standard_normal((n, k)) * 0.02).astype(np.float32)
    codes, atoms = oracle.mxfp8_quantize(w)
    blocks = k // 32
    plain = np.array([[atoms[oracle.lib.orc_scale_atom_offset(r, b, blocks)] for b in range(blocks)] for r in range(n)],
                     dtype=np.uint8)
    x = synth.activations(tokens, k, 10)
    want = oracle.mxfp8_gemv(codes, plain, x)
    got = ops.mxfp8_gemv(dev(codes, device), dev(plain, device), dev(x, device)).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst
    solo = ops.mxfp8_gemv(dev(codes, device), dev(plain, device), dev(x[:1], device)).cpu().numpy()
    assert np.array_equal(solo[0].view(np.uint32), got[0].view(np.uint32))  # a column is its lone product


def quantized_operands(m, n, k, seed):
    g = synth.rng(seed)
    a = synth.bf16_to_f32(synth.bf16_bits(g.standard_normal((m, k), dtype=np.float32)))
    w = (g.standard_normal((n, k), dtype=np.float32) * 0.02)
    return a, w, oracle.mxfp8_quantize(a), oracle.mxfp8_quantize(w)


@pytest.mark.parametrize("m,n,k", [(128, 128, 128), (256, 384, 512), (100, 260, 256), (1, 4, 128), (130, 136, 1024)])
@pytest.mark.parametrize("bf16", [False, True])
def test_gemm_matches_the_product_of_the_quantized_operands(device, m, n, k, bf16):
    a, w, (ac, asc), (wc, wsc) = quantized_operands(m, n, k, 20 + m)
    want = oracle.mxfp8_gemm(ac, asc, wc, wsc, threads=oracle.max_threads())
    got = ops.mxfp8_gemm(dev(ac, device), dev(asc, device), dev(wc, device), dev(wsc, device), bf16=bf16)
    got = got.float().cpu().numpy()
    scale = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    # The stated bound: 2e-2 of each value (floored at 2e-2 of the output's RMS).
    assert np.all(np.abs(got - want) <= 2e-2 * np.maximum(np.abs(want), 2e-2 * scale))
    nmse = np.sum((got - want.astype(np.float64)) ** 2) / np.sum(want.astype(np.float64) ** 2)
    # tests/unit/qwen38_fast_test.cc:755-778 of the reference asks 1e-10 / 1e-5 of its tensor cores; the
    # block-scaled MFMA rounds inside its 128-term sums, measured about 2e-10 at one K step.
    assert nmse <= (1e-5 if bf16 else 1e-8), nmse
    exact = a.astype(np.float64) @ w.astype(np.float64).T
    assert np.sum((got - exact) ** 2) / np.sum(exact ** 2) <= 3e-3


@pytest.mark.parametrize("m,n,k", [(520, 400, 384), (300, 700, 128), (257, 260, 256), (600, 392, 640)])
@pytest.mark.parametrize("bf16", [False, True])
def test_gemm_workgroups_that_take_several_tiles(device, m, n, k, bf16):
    """A workgroup goes through its tiles one after the other, the next tile's first steps asked for while the last
    steps of this one are multiplied (with one or two K steps a tile, two or three tiles ahead). Whichever workgroup
    takes a tile, its sums are the same: one, two, three or five workgroups against a workgroup a tile, bit for bit,
    and that against the oracle."""
    a, w, (ac, asc), (wc, wsc) = quantized_operands(m, n, k, 60 + m)
    ops_in = (dev(ac, device), dev(asc, device), dev(wc, device), dev(wsc, device))
    each = ops.mxfp8_gemm(*ops_in, bf16=bf16, compute_units=4096).cpu()
    want = oracle.mxfp8_gemm(ac, asc, wc, wsc, threads=oracle.max_threads())
    got = each.float().numpy()
    scale = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.all(np.abs(got - want) <= 2e-2 * np.maximum(np.abs(want), 2e-2 * scale))
    for cus in (1, 2, 3, 5):
        few = ops.mxfp8_gemm(*ops_in, bf16=bf16, compute_units=cus).cpu()
        assert torch.equal(few.view(torch.int16 if bf16 else torch.int32), each.view(torch.int16 if bf16 else torch.int32)), cus


@pytest.mark.parametrize("bf16", [False, True])
def test_gemm_nan_codes_and_scales_stay_in_their_rows_and_columns(device, bf16):
    """E4M3's NaN code (0x7F) in an activation row, and an undefined scale (0xFF) on a weight row: every output of
    that row (that column) is a NaN, in F32 and after the bf16 packing, and every other output keeps its bits."""
    m, n, k = 130, 200, 256
    a, w, (ac, asc), (wc, wsc) = quantized_operands(m, n, k, 77)
    clean = ops.mxfp8_gemm(dev(ac, device), dev(asc, device), dev(wc, device), dev(wsc, device), bf16=bf16).float().cpu().numpy()
    ac2 = ac.copy()
    ac2[5, 131] = 0x7F
    wsc2 = wsc.copy()
    wsc2[oracle.lib.orc_scale_atom_offset(9, 3, k // 32)] = 0xFF
    got = ops.mxfp8_gemm(dev(ac2, device), dev(asc, device), dev(wc, device), dev(wsc2, device), bf16=bf16).float().cpu().numpy()
    bad = np.zeros((m, n), dtype=bool)
    bad[5, :] = True
    bad[:, 9] = True
    assert np.all(np.isnan(got[bad]))
    assert np.array_equal(got[~bad].view(np.uint32), clean[~bad].view(np.uint32))


def test_gemm_full_size_sampled(device):
    """The headline prefill shape, M 2048, K 4096, N 12288: sampled entries against the oracle's dot, and
    linearity in the activations' scales (doubling a row's scales doubles its outputs exactly)."""
    m, n, k = 2048, 12288, 4096
    g = synth.rng(31)
    ac = g.integers(0, 256, size=(m, k), dtype=np.uint8)
    ac[(ac & 0x7F) == 0x7F] = 0x3A
    wc = g.integers(0, 256, size=(n, k), dtype=np.uint8)
    wc[(wc & 0x7F) == 0x7F] = 0x3A
    asc = oracle.mxfp8_swizzle(g.integers(118, 126, size=(m, k // 32), dtype=np.uint8))
    wsc = oracle.mxfp8_swizzle(g.integers(112, 120, size=(n, k // 32), dtype=np.uint8))
    da, dasc, dw, dwsc = dev(ac, device), dev(asc, device), dev(wc, device), dev(wsc, device)
    got = ops.mxfp8_gemm(da, dasc, dw, dwsc, bf16=False).cpu().numpy()
    rows = g.integers(0, m, size=300)
    cols = g.integers(0, n, size=300)
    want = np.array([oracle.mxfp8_dot(ac, asc, int(i), wc, wsc, int(j)) for i, j in zip(rows, cols)])
    scale = np.sqrt(np.mean(want ** 2))
    assert np.all(np.abs(got[rows, cols] - want) <= 2e-2 * np.maximum(np.abs(want), 2e-2 * scale))
    assert np.sum((got[rows, cols] - want) ** 2) / np.sum(want ** 2) <= 1e-8
    doubled = asc.copy()
    blocks = k // 32
    for b in range(blocks):
        doubled[oracle.lib.orc_scale_atom_offset(7, b, blocks)] += 1
    got2 = ops.mxfp8_gemm(da, dev(doubled, device), dw, dwsc, bf16=False).cpu().numpy()
    assert np.array_equal(got2[7], 2 * got[7]) and np.array_equal(got2[8], got[8])


def test_gemm_refusals(device):
    z = torch.zeros(128 * 128, dtype=torch.uint8, device=device)
    with pytest.raises(ops.KernelFailure) as e:
        ops.mxfp8_gemm(z.view(128, 128)[:, :96], z, z.view(128, 128)[:, :96], z)
    assert e.value.rejected
