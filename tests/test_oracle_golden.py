"""Pins of the CPU oracle: the reference's own golden vectors and independent derivations
(numpy IEEE conversions, closed forms, brute force), so that a dropped term, a wrong index or
a transposed operand in oracle/oracle.c fails here. No GPU."""
import math

import numpy as np
import pytest

import oracle
from oracle import lib

# ---------------------------------------------------------------- conversions


def test_f16_decode_is_ieee_exhaustively():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.orc_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_and_bf16_encode_round_to_nearest_even():
    """tests/unit/reference_decode_test.cc:138-141 of the reference: its sample list, then
    random bit patterns, against numpy's float16 and the bfloat16 closed form."""
    samples = [0x00000000, 0x80000000, 0x7F800000, 0xFF800000, 0x477FE000, 0x477FEFFF, 0x477FF000, 0x38800000,
               0x387FFFFF, 0x33000000, 0x33000001, 0x32FFFFFF, 0x337FFFFF, 0x00000001, 0x3F800000]
    g = np.random.Generator(np.random.PCG64(3))
    samples += [int(v) for v in g.integers(0, 2 ** 32, size=20000, dtype=np.uint64)]
    u = np.array(samples, dtype=np.uint32)
    f = u.view(np.float32)
    keep = ~np.isnan(f)
    with np.errstate(over="ignore"):
        want16 = f.astype(np.float16).view(np.uint16)
    for x, w16, ok in zip(f, want16, keep):
        if not ok:
            assert math.isnan(lib.orc_f16_to_f32(lib.orc_f32_to_f16(float(x))))
            continue
        assert lib.orc_f32_to_f16(float(x)) == int(w16), hex(np.float32(x).view(np.uint32))
        xb = int(np.float32(x).view(np.uint32))
        assert lib.orc_f32_to_bf16(float(x)) == ((xb + 0x7FFF + ((xb >> 16) & 1)) >> 16) & 0xFFFF
    assert lib.orc_bf16_to_f32(0x3FC0) == 1.5


def e4m3_closed_form(b):
    """tests/unit/qwen38_ops_test.cc:101-110 of the reference."""
    e, m = (b >> 3) & 15, b & 7
    if e == 15 and m == 7:
        return math.nan
    v = m * 2.0 ** -9 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
    return -v if b & 0x80 else v


def test_e4m3_and_e8m0_decode():
    for b in range(256):
        want = e4m3_closed_form(b)
        got = lib.orc_e4m3_to_f32(b)
        assert (math.isnan(got) and math.isnan(want)) or got == want
        if b == 0xFF:
            assert math.isnan(lib.orc_e8m0_to_f32(b))
        else:
            assert lib.orc_e8m0_to_f32(b) == math.ldexp(1.0, b - 127)
    assert lib.orc_e4m3_to_f32(0x7E) == 448.0 and lib.orc_e4m3_to_f32(0x01) == 2.0 ** -9


def test_e4m3_encode_is_nearest_even_and_saturates():
    """Brute force: every float maps to the nearest finite E4M3 value, ties to the even code."""
    values = np.array([e4m3_closed_form(b) for b in range(0x7F)])  # positive finite codes, ascending
    g = np.random.Generator(np.random.PCG64(4))
    xs = np.concatenate([g.uniform(-500, 500, 4000), g.uniform(-0.05, 0.05, 4000), values, (values[:-1] + values[1:]) / 2,
                         [448.0, 449.0, 464.0, 465.0, 1e9, -1e9, 0.0]]).astype(np.float32)
    for x in xs:
        got = lib.orc_f32_to_e4m3(float(x))
        a = abs(float(x))
        if a >= 448.0:
            want = 0x7E
        else:
            d = np.abs(values - a)
            best = np.flatnonzero(d == d.min())
            want = int(best[0]) if len(best) == 1 else int([c for c in best if c % 2 == 0][0])
        want |= 0x80 if np.signbit(x) else 0
        assert got == want, (float(x), hex(got), hex(want))
    assert lib.orc_f32_to_e4m3(float("nan")) & 0x7F == 0x7F


# ---------------------------------------------------------------------- Q8_1


def test_q8_1_layout_and_values_against_numpy():
    """Block = {f16 d; f16 s; i8 qs[32]} (src/format/encoding.cc:112 of the reference), d = amax / 127,
    q = round-half-away(x / d), zero blocks past k (src/ir/op.h:400-405)."""
    g = np.random.Generator(np.random.PCG64(5))
    x = g.standard_normal((3, 96)).astype(np.float32)
    x[0, :32] = 0
    x[1, 40] = 1000.0
    got = oracle.q8_1_quantize(x)
    assert got.shape == (3, 512 // 32 * 36)
    for r in range(3):
        blocks = got[r].reshape(-1, 36)
        assert not blocks[3:].any()
        for b in range(3):
            v = x[r, b * 32:(b + 1) * 32]
            amax = np.abs(v).max()
            d = np.float32(amax) / np.float32(127.0)
            assert blocks[b, 0:2].view(np.float16)[0] == np.float16(d)
            q = np.zeros(32) if amax == 0 else np.trunc(np.abs(v / d) + np.float32(0.5)) * np.sign(v)
            # (|v / d| + 0.5 truncated is round-half-away unless the sum rounds up: not at these magnitudes)
            assert np.array_equal(blocks[b, 4:].view(np.int8), q.astype(np.int8))
            assert abs(float(blocks[b, 2:4].view(np.float16)[0]) - float(v.sum())) <= 2e-3 * max(1.0, abs(v.sum()))
    # Decode is d * q (tests/unit/reference_decode_test.cc:207-224).
    back = oracle.q8_1_decode(got[2], 96)
    assert np.abs(back - x[2]).max() <= np.abs(x[2]).max() / 127 * 0.51


def test_q8_1_flavours_differ_only_by_rounding_ties():
    x = np.random.Generator(np.random.PCG64(6)).standard_normal((64, 4096)).astype(np.float32)
    a = oracle.q8_1_quantize(x, oracle.Q8_DEVICE).reshape(64, -1, 36)
    b = oracle.q8_1_quantize(x, oracle.Q8_GGML_CPU).reshape(64, -1, 36)
    assert np.array_equal(a[:, :, 0:2], b[:, :, 0:2])  # the same scale
    diff = a[:, :, 4:].view(np.int8).astype(int) - b[:, :, 4:].view(np.int8).astype(int)
    assert np.abs(diff).max() <= 1
    assert np.count_nonzero(diff) <= 1e-4 * diff.size  # a handful of codes per million


# ------------------------------------------------------------- weight blocks


def q4_k_decode_numpy(block):
    """An independent Q4_K decode: ggml's get_scale_min_k4 packing, nibble j of byte
    (g / 2) * 32 + i (tests/unit/dsv4_fast_test.cc:176-193 of the reference)."""
    d, dmin = block[0:4].view(np.float16).astype(np.float32)
    s = block[4:16].astype(int)
    qs = block[16:].astype(int)
    out = np.zeros(256, dtype=np.float64)
    for g in range(8):
        if g < 4:
            sc, m = s[g] & 63, s[g + 4] & 63
        else:
            sc, m = (s[g + 4] & 15) | ((s[g - 4] >> 6) << 4), (s[g + 4] >> 4) | ((s[g] >> 6) << 4)
        codes = (qs[(g // 2) * 32:(g // 2) * 32 + 32] >> (4 * (g % 2))) & 15
        out[g * 32:(g + 1) * 32] = float(d) * sc * codes - float(dmin) * m
    return out


def test_q4_k_and_q8_0_decode_and_block_sums_by_brute_force():
    from llmp_amd import synth
    k = 512
    for t in (oracle.TYPE_Q4_K, oracle.TYPE_Q8_0):
        w = synth.random_blocks(t, 5, k, 7)
        x = np.random.Generator(np.random.PCG64(8)).standard_normal((1, k)).astype(np.float32)
        q8 = oracle.q8_1_quantize(x)
        dec = oracle.decode_rows(t, w, k)
        a = q8[0].reshape(-1, 36)
        aq = a[:, 4:].view(np.int8).astype(np.int64)
        ad = a[:, 0:2].view(np.float16).astype(np.float64).reshape(-1)
        sums = oracle.vecq_block_sums(t, w, q8, k, 5)
        y = oracle.vecq(t, w, q8, k, 5)[0, 0]
        for r in range(5):
            if t == oracle.TYPE_Q4_K:
                blocks = w[r].reshape(-1, 144)
                want = np.concatenate([q4_k_decode_numpy(b) for b in blocks])
                codes = np.stack([((b[16:].astype(int)[(g // 2) * 32:(g // 2) * 32 + 32] >> (4 * (g % 2))) & 15)
                                  for b in blocks for g in range(8)])
                prod = (codes * aq[:k // 32]).sum(axis=1).reshape(-1, 8)
                assert np.array_equal(sums[r, :, :8], prod)
                assert np.array_equal(sums[r, :, 8:], aq[:k // 32].sum(axis=1).reshape(-1, 8))
            else:
                blocks = w[r].reshape(-1, 34)
                wq = blocks[:, 2:].view(np.int8).astype(np.int64)
                wd = blocks[:, 0:2].view(np.float16).astype(np.float64).reshape(-1)
                want = (wq * wd[:, None]).reshape(-1)
                assert np.array_equal(sums[r, :, 0], (wq * aq[:k // 32]).sum(axis=1))
            np.testing.assert_allclose(dec[r], want, rtol=1e-6, atol=1e-12)
            # The product is the FP64 dot of decoded weights and decoded activations.
            act = (aq[:k // 32] * ad[:k // 32, None]).reshape(-1)
            np.testing.assert_allclose(y[r], float(np.dot(want, act)), rtol=2e-6, atol=1e-9)


def test_q5_k_decode_sums_and_products_by_brute_force_and_known_answers():
    """Q5_K (src/format/encoding.cc:116 of the reference: 256 values in 176 bytes; ggml's dequantize_row_q5_K):
    Q4_K's header and nibbles after 32 bytes whose bit g of byte i is the fifth bit of value i of sub-block g.
    Parity unpinned: ggml is not vendored and the reference holds no Q5_K vector; this pins the oracle's C against
    numpy's reading of the published layout, the fifth bits alone against Q4_K (a block with qh = 0 is the Q4_K
    block of the same header and nibbles; with qh = 0xFF every code is 16 more), and a hand-built block."""
    from llmp_amd import synth
    t, k, n = oracle.TYPE_Q5_K, 512, 5
    assert oracle.block_bytes(t) == 176 and oracle.block_elements(t) == 256
    w = synth.random_blocks(t, n, k, 71)
    x = np.random.Generator(np.random.PCG64(72)).standard_normal((1, k)).astype(np.float32)
    q8 = oracle.q8_1_quantize(x)
    a = q8[0].reshape(-1, 36)
    aq = a[:, 4:].view(np.int8).astype(np.int64)
    ad = a[:, 0:2].view(np.float16).astype(np.float64).reshape(-1)
    dec, sums, y = oracle.decode_rows(t, w, k), oracle.vecq_block_sums(t, w, q8, k, n), oracle.vecq(t, w, q8, k, n)[0, 0]
    for r in range(n):
        rows, codes = [], []
        for b in w[r].reshape(-1, 176):
            four = np.concatenate([b[0:16], b[48:176]])           # the Q4_K block of the same header and nibbles
            base = q4_k_decode_numpy(four)
            d = float(b[0:2].view(np.float16)[0])
            s = b[4:16].astype(int)
            for g in range(8):
                sc = s[g] & 63 if g < 4 else (s[g + 4] & 15) | ((s[g - 4] >> 6) << 4)
                fifth = (b[16:48].astype(int) >> g) & 1
                base[g * 32:(g + 1) * 32] += d * sc * 16.0 * fifth
                codes.append(((b[48:].astype(int)[(g // 2) * 32:(g // 2) * 32 + 32] >> (4 * (g % 2))) & 15) + 16 * fifth)
            rows.append(base)
        want = np.concatenate(rows)
        np.testing.assert_allclose(dec[r], want, rtol=1e-5, atol=1e-9)
        prod = (np.stack(codes) * aq[:k // 32]).sum(axis=1).reshape(-1, 8)
        assert np.array_equal(sums[r, :, :8], prod)
        assert np.array_equal(sums[r, :, 8:], aq[:k // 32].sum(axis=1).reshape(-1, 8))
        act = (aq[:k // 32] * ad[:k // 32, None]).reshape(-1)
        np.testing.assert_allclose(y[r], float(np.dot(want, act)), rtol=2e-6, atol=1e-9)
    # qh = 0: the Q4_K block; qh = 0xFF: every code 16 more.
    five = synth.random_blocks(t, 1, 256, 73)
    five[0, 16:48] = 0
    four = np.concatenate([five[0, 0:16], five[0, 48:176]])[None, :]
    assert np.array_equal(oracle.decode_rows(t, five, 256), oracle.decode_rows(oracle.TYPE_Q4_K, four, 256))
    q1 = oracle.q8_1_quantize(x[:, :256])
    low = oracle.vecq_block_sums(t, five, q1, 256, 1)
    assert np.array_equal(low, oracle.vecq_block_sums(oracle.TYPE_Q4_K, four, q1, 256, 1))
    five[0, 16:48] = 0xFF
    high = oracle.vecq_block_sums(t, five, q1, 256, 1)
    assert np.array_equal(high[0, 0, :8], low[0, 0, :8] + 16 * low[0, 0, 8:])
    # Hand-built: d = 1, dmin = 0, every sub-scale 1 (bytes 4..7 = 1, bytes 12..15 = 1), nibbles 3, the fifth bit of
    # sub-block 2 alone set: its values 19, all others 3. Every q = 1 with d8 = 0.5: 0.5 * (7 * 96 + 608) = 640.
    b = np.zeros((1, 176), dtype=np.uint8)
    b[0, 0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    b[0, 4:8], b[0, 12:16] = 1, 1
    b[0, 16:48] = 1 << 2
    b[0, 48:] = 0x33
    got = oracle.decode_rows(t, b, 256)[0]
    assert np.array_equal(got, np.where((np.arange(256) // 32) == 2, 19.0, 3.0))
    q = np.zeros((1, 8 * 36), dtype=np.uint8)
    for g in range(8):
        q[0, g * 36:g * 36 + 2] = np.array([0.5], dtype=np.float16).view(np.uint8)
        q[0, g * 36 + 4:g * 36 + 36] = 1
    assert oracle.vecq(t, b, q, 256, 1)[0, 0, 0] == 640.0


def q6_k_decode_numpy(block):
    """ggml's dequantize_row_q6_K, its loops as published (two halves of 128, four groups of 32 each from the same 32
    bytes of qh), apart from the oracle's index form."""
    ql, qh, sc = block[0:128].astype(int), block[128:192].astype(int), block[192:208].view(np.int8).astype(int)
    d = float(block[208:210].view(np.float16)[0])
    y = np.zeros(256, dtype=np.float64)
    for half in range(2):
        lo, hi, s, o = ql[64 * half:], qh[32 * half:], sc[8 * half:], 128 * half
        for l in range(32):
            i = l // 16
            q1 = ((lo[l] & 0xF) | (((hi[l] >> 0) & 3) << 4)) - 32
            q2 = ((lo[l + 32] & 0xF) | (((hi[l] >> 2) & 3) << 4)) - 32
            q3 = ((lo[l] >> 4) | (((hi[l] >> 4) & 3) << 4)) - 32
            q4 = ((lo[l + 32] >> 4) | (((hi[l] >> 6) & 3) << 4)) - 32
            y[o + l], y[o + l + 32] = d * s[i] * q1, d * s[i + 2] * q2
            y[o + l + 64], y[o + l + 96] = d * s[i + 4] * q3, d * s[i + 6] * q4
    return y


def test_q6_k_decode_sums_and_products_by_brute_force_and_known_answers():
    """Q6_K (src/format/encoding.cc:117 of the reference: 256 values in 210 bytes). Parity unpinned: ggml is not
    vendored and the reference holds no Q6_K vector; this pins the oracle's C against numpy's reading of the published
    loops, the int32 sums and the product against the FP64 dot of decoded weights and activations, and a hand-built
    block."""
    from llmp_amd import synth
    t, k, n = oracle.TYPE_Q6_K, 512, 5
    assert oracle.block_bytes(t) == 210 and oracle.block_elements(t) == 256
    x = np.random.Generator(np.random.PCG64(82)).standard_normal((1, k)).astype(np.float32)
    q8 = oracle.q8_1_quantize(x)
    a = q8[0].reshape(-1, 36)
    aq = a[:, 4:].view(np.int8).astype(np.int64)
    ad = a[:, 0:2].view(np.float16).astype(np.float64).reshape(-1)
    act = (aq[:k // 32] * ad[:k // 32, None]).reshape(-1)
    for w in (synth.random_blocks(t, n, k, 81), synth.q6_k_weights(n, k, 83)):
        dec, sums, y = oracle.decode_rows(t, w, k), oracle.vecq_block_sums(t, w, q8, k, n), oracle.vecq(t, w, q8, k, n)[0, 0]
        for r in range(n):
            blocks = w[r].reshape(-1, 210)
            want = np.concatenate([q6_k_decode_numpy(b) for b in blocks])
            np.testing.assert_allclose(dec[r], want, rtol=1e-6, atol=1e-12)
            for i, b in enumerate(blocks):
                d, sc = float(b[208:210].view(np.float16)[0]), b[192:208].view(np.int8).astype(np.float64)
                codes = np.rint(want[256 * i:256 * (i + 1)].reshape(16, 16) / (d * sc[:, None] + (sc[:, None] == 0)))
                codes = np.where(sc[:, None] == 0, 0, codes).astype(np.int64)
                got = sums[r, i].astype(np.int64)
                flat = aq[8 * i:8 * i + 8].reshape(16, 16)
                live = sc != 0
                assert np.array_equal(got[live], (codes * flat).sum(axis=1)[live])
            np.testing.assert_allclose(y[r], float(np.dot(want, act)), rtol=2e-6, atol=1e-9)
    # Hand-built: d = 0.5, every scale 2, ql = 0x21 everywhere, qh = 0xE4 (bits 2t, 2t + 1 = t): group t of a half has
    # codes (1 or 2) + 16 t - 32: t = 0, 1 take the low nibble 1, t = 2, 3 the high nibble 2.
    b = np.zeros((1, 210), dtype=np.uint8)
    b[0, 0:128], b[0, 128:192], b[0, 192:208] = 0x21, 0xE4, 2
    b[0, 208:210] = np.array([0.5], dtype=np.float16).view(np.uint8)
    code = np.array([1 - 32, 1 + 16 - 32, 2 + 32 - 32, 2 + 48 - 32])
    want = np.tile(np.repeat(code, 32), 2).astype(np.float64)
    assert np.array_equal(oracle.decode_rows(t, b, 256)[0], want)
    q = np.zeros((1, 8 * 36), dtype=np.uint8)
    for g in range(8):
        q[0, g * 36:g * 36 + 2] = np.array([0.25], dtype=np.float16).view(np.uint8)
        q[0, g * 36 + 4:g * 36 + 36] = 3
    assert np.array_equal(oracle.vecq_block_sums(t, b, q, 256, 1)[0, 0], np.tile(np.repeat(code, 2), 2) * 48)
    assert oracle.vecq(t, b, q, 256, 1)[0, 0, 0] == 0.5 * 0.25 * 2 * 48 * 2 * 2 * code.sum()


def legacy_block_numpy(t, block, a):
    """tests/unit/dsv4_fast_test.cc:141-164 restated with numpy, apart from the oracle's C:
    (codes, int sum, product) of one legacy block and one Q8_1 block."""
    affine, five = t in (3, 7), t in (6, 7)
    prefix = 4 if affine else 2
    high = int(block[prefix:prefix + 4].view(np.uint32)[0]) if five else 0
    nib = block[prefix + (4 if five else 0):].astype(np.int64)
    codes = np.concatenate([nib & 15, nib >> 4])
    if five:
        codes = codes + 16 * ((high >> np.arange(32)) & 1)
    q = a[4:].view(np.int8).astype(np.int64)
    total = int((codes * q).sum())
    dw, da, sa = (float(v) for v in (block[0:2].view(np.float16)[0], a[0:2].view(np.float16)[0],
                                    a[2:4].view(np.float16)[0]))
    if affine:
        m = float(block[2:4].view(np.float16)[0])
        scale = float(np.float16(np.float32(dw) * np.float32(da)))
        minimum = float(np.float16(np.float32(m) * np.float32(sa)))
        return codes, total, total * scale + minimum
    return codes, total, dw * (total * da - (16.0 if five else 8.0) * sa)


def test_legacy_blocks_decode_sums_and_products_by_brute_force():
    from llmp_amd import synth
    k, n = 256, 4
    x = np.random.Generator(np.random.PCG64(18)).standard_normal((1, k)).astype(np.float32)
    q8 = oracle.q8_1_quantize(x)
    acts = q8[0].reshape(-1, 36)
    for t in (oracle.TYPE_Q4_0, oracle.TYPE_Q4_1, oracle.TYPE_Q5_0, oracle.TYPE_Q5_1):
        size = oracle.block_bytes(t)
        assert size == synth.LEGACY_BYTES[t] and oracle.block_elements(t) == 32
        for w in (synth.random_blocks(t, n, k, 17 + t), synth.legacy_weights(t, n, k, 19 + t)):
            sums = oracle.vecq_block_sums(t, w, q8, k, n)
            y = oracle.vecq(t, w, q8, k, n)[0, 0]
            dec = oracle.decode_rows(t, w, k)
            for r in range(n):
                want, row = 0.0, []
                for b, block in enumerate(w[r].reshape(-1, size)):
                    codes, total, product = legacy_block_numpy(t, block, acts[b])
                    assert sums[r, b, 0] == total
                    want += product
                    d = float(block[0:2].view(np.float16)[0])
                    m = float(block[2:4].view(np.float16)[0]) if t in (3, 7) else 0.0
                    offset = 0 if t in (3, 7) else 16 if t in (6, 7) else 8
                    row.append(np.float32(d) * (codes - offset).astype(np.float32) + np.float32(m))
                np.testing.assert_allclose(dec[r], np.concatenate(row), rtol=1e-6, atol=1e-12)
                np.testing.assert_allclose(y[r], want, rtol=1e-6, atol=1e-9)


def test_iq4_nl_codebook_blocks_by_brute_force_and_known_answers():
    """IQ4_NL (src/format/encoding.cc:126: 32 values in 18 bytes; src/kernels/ggml/vecq.cu:375-396 of the
    reference: (dw * d8) * sum(value[code] * q)). Parity unpinned: the codebook is ggml's kvalues_iq4nl, which the
    reference does not vendor and for which it holds no vector; this pins the oracle's layout and arithmetic
    against numpy and a hand-built block, and the codebook against what is published of it (sixteen rising int8
    values from -127 to 113 that sum to -94, the ninth being 1)."""
    from llmp_amd import synth
    values = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.int64)
    t, k, n = oracle.TYPE_IQ4_NL, 256, 4
    assert oracle.block_bytes(t) == 18 and oracle.block_elements(t) == 32
    # The codebook as the oracle decodes it: d = 1, code i = i % 16 in both halves.
    w = np.zeros((1, 18), dtype=np.uint8)
    w[0, 0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    w[0, 2:] = np.arange(16, dtype=np.uint8) * 17
    book = oracle.decode_rows(t, w, 32)[0]
    assert np.array_equal(book[:16], book[16:]) and np.all(np.diff(book[:16]) > 0)
    assert book[0] == -127 and book[8] == 1 and book[15] == 113 and book[:16].sum() == -94
    assert np.array_equal(book[:16], values)
    # Every q = 2, d8 = 0.25: sum = 2 * 2 * -94 = -376; (1 * 0.25) * -376 = -94.
    q8 = np.zeros((1, 36), dtype=np.uint8)
    q8[0, 0:2] = np.array([0.25], dtype=np.float16).view(np.uint8)
    q8[0, 2:4] = np.array([3.0], dtype=np.float16).view(np.uint8)  # the stored sum plays no part
    q8[0, 4:36] = np.full(32, 2, dtype=np.int8).view(np.uint8)
    assert oracle.vecq_block_sums(t, w, q8, 32, 1)[0, 0, 0] == -376
    assert oracle.vecq(t, w, q8, 32, 1)[0, 0, 0] == -94.0
    # Random bytes and plausible blocks against numpy.
    x = np.random.Generator(np.random.PCG64(58)).standard_normal((1, k)).astype(np.float32)
    q8 = oracle.q8_1_quantize(x)
    acts = q8[0].reshape(-1, 36)
    for w in (synth.random_blocks(t, n, k, 59), synth.legacy_weights(t, n, k, 60)):
        sums = oracle.vecq_block_sums(t, w, q8, k, n)
        y = oracle.vecq(t, w, q8, k, n)[0, 0]
        dec = oracle.decode_rows(t, w, k)
        for r in range(n):
            want, row = 0.0, []
            for b, block in enumerate(w[r].reshape(-1, 18)):
                nib = block[2:].astype(np.int64)
                v = values[np.concatenate([nib & 15, nib >> 4])]
                total = int((v * acts[b][4:].view(np.int8).astype(np.int64)).sum())
                assert sums[r, b, 0] == total
                d = float(block[0:2].view(np.float16)[0])
                want += d * float(acts[b][0:2].view(np.float16)[0]) * total
                row.append(np.float32(d) * v.astype(np.float32))
            np.testing.assert_allclose(dec[r], np.concatenate(row), rtol=1e-6, atol=1e-12)
            np.testing.assert_allclose(y[r], want, rtol=1e-6, atol=1e-9)


def test_hand_built_legacy_blocks_have_known_answers():
    # Q4_0: d = 0.5, code i = i % 16 in both halves (byte i = i | i << 4); activation d = 0.25,
    # every q = 2, s = 3. sum = 2 * 2 * (0 + .. + 15) = 480; 0.5 * (480 * 0.25 - 8 * 3) = 48.
    w = np.zeros((1, 18), dtype=np.uint8)
    w[0, 0:2] = np.array([0.5], dtype=np.float16).view(np.uint8)
    w[0, 2:] = np.arange(16, dtype=np.uint8) * 17
    q8 = np.zeros((1, 16 * 36), dtype=np.uint8)
    q8[0, 0:2] = np.array([0.25], dtype=np.float16).view(np.uint8)
    q8[0, 2:4] = np.array([3.0], dtype=np.float16).view(np.uint8)
    q8[0, 4:36] = np.full(32, 2, dtype=np.int8).view(np.uint8)
    assert oracle.vecq_block_sums(oracle.TYPE_Q4_0, w, q8, 32, 1)[0, 0, 0] == 480
    assert oracle.vecq(oracle.TYPE_Q4_0, w, q8, 32, 1)[0, 0, 0] == 48.0
    assert np.array_equal(oracle.decode_rows(oracle.TYPE_Q4_0, w, 32)[0], 0.5 * (np.arange(32) % 16 - 8))
    # Q5_0 with the high bits of values 0..7 set: codes 16..23 there; offset 16.
    w5 = np.zeros((1, 22), dtype=np.uint8)
    w5[0, 0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    w5[0, 2:6] = np.array([0xFF], dtype=np.uint32).view(np.uint8)
    w5[0, 6:] = np.arange(16, dtype=np.uint8) * 17
    total = 2 * (2 * sum(range(16)) + 16 * 8)
    assert oracle.vecq_block_sums(oracle.TYPE_Q5_0, w5, q8, 32, 1)[0, 0, 0] == total
    assert oracle.vecq(oracle.TYPE_Q5_0, w5, q8, 32, 1)[0, 0, 0] == np.float32(total * 0.25 - 16 * 3)


def test_mxfp4_values_layout_and_products():
    """MXFP4 as the reference's own CPU decoder has it (src/kernels/reference/decode.cc:239-248,
    417-428) and its known answers (tests/unit/reference_decode_test.cc:465-484: bytes of 0x22
    are ones, scale bytes 0x00 / 0x7F / 0xFE are 2^-127 / 1 / 2^127, 0xFF is NaN); the product
    of src/kernels/ggml/vecq.cu:421-437 against a numpy restatement and a hand-built block."""
    from llmp_amd import synth
    # The E2M1 values, by the format's definition: sign, two exponent bits, one mantissa bit,
    # bias 1, subnormal at exponent 0.
    for code in range(16):
        e, m = (code >> 1) & 3, code & 1
        magnitude = 0.5 * m if e == 0 else (1.0 + 0.5 * m) * 2.0 ** (e - 1)
        assert oracle.lib.orc_e2m1_to_f32(code) == (-magnitude if code & 8 else magnitude)
    assert [oracle.lib.orc_e2m1_to_f32(c) for c in range(8)] == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert oracle.block_bytes(oracle.TYPE_MXFP4) == 17 and oracle.block_elements(oracle.TYPE_MXFP4) == 32
    # reference_decode_test.cc:465-484
    k = 128
    row = np.concatenate([np.concatenate([[e], np.full(16, 0x22)]) for e in (0x00, 0x7F, 0xFE, 0xFF)]).astype(np.uint8)
    got = oracle.decode_rows(oracle.TYPE_MXFP4, row[None, :], k)[0]
    assert np.array_equal(got[:32], np.full(32, 2.0 ** -127, dtype=np.float32))
    assert np.array_equal(got[32:64], np.ones(32, dtype=np.float32))
    assert np.array_equal(got[64:96], np.full(32, 2.0 ** 127, dtype=np.float32))
    assert np.all(np.isnan(got[96:]))
    # Layout: byte j of a block holds values j (low nibble) and j + 16.
    block = np.zeros(17, dtype=np.uint8)
    block[0] = 128  # scale 2
    block[1 + 3] = 0x5 | (0xC << 4)  # value 3 = code 5 (3.0), value 19 = code 12 (-2.0)
    got = oracle.decode_rows(oracle.TYPE_MXFP4, block[None, :], 32)[0]
    want = np.zeros(32, dtype=np.float32)
    want[3], want[19] = 6.0, -4.0
    assert np.array_equal(got, want)
    # Products: numpy restatement over random bytes.
    table = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], dtype=np.int64)
    k, n = 512, 5
    x = np.random.Generator(np.random.PCG64(28)).standard_normal((1, k)).astype(np.float32)
    q8 = oracle.q8_1_quantize(x)
    acts = q8[0].reshape(-1, 36)
    for w in (synth.random_blocks(oracle.TYPE_MXFP4, n, k, 29), synth.mxfp4_weights(n, k, 30)):
        sums = oracle.vecq_block_sums(oracle.TYPE_MXFP4, w, q8, k, n)
        y = oracle.vecq(oracle.TYPE_MXFP4, w, q8, k, n)[0, 0]
        dec = oracle.decode_rows(oracle.TYPE_MXFP4, w, k)
        for r in range(n):
            total, row = 0.0, []
            for b, blk in enumerate(w[r].reshape(-1, 17)):
                codes = np.concatenate([blk[1:] & 15, blk[1:] >> 4]).astype(np.int64)
                q = acts[b][4:].view(np.int8).astype(np.int64)
                s = int((table[codes] * q).sum())
                assert sums[r, b, 0] == s
                scale = 2.0 ** (int(blk[0]) - 127)
                total += scale * 0.5 * float(acts[b][0:2].view(np.float16)[0]) * s
                row.append((table[codes] * 0.5 * scale).astype(np.float32))
            np.testing.assert_array_equal(dec[r], np.concatenate(row))
            np.testing.assert_allclose(y[r], total, rtol=1e-6, atol=1e-12)
        # The product is the decoded weights times the decoded activations.
        dense = dec.astype(np.float64) @ oracle.q8_1_decode(q8[0], k).astype(np.float64)
        np.testing.assert_allclose(y, dense, rtol=1e-5, atol=1e-9)
    # By hand: scale byte 126 (0.5), codes i % 16 in both halves; activation d = 0.25, q = 2 against
    # codes 0..7 (twice their values add up to 36) and -2 against codes 8..15 (-36):
    # sum = 2 halves * (2 * 36 + -2 * -36) = 288; times 0.5 / 2 * 0.25 = 18.
    w = np.zeros((1, 17), dtype=np.uint8)
    w[0, 0] = 126
    w[0, 1:] = np.arange(16, dtype=np.uint8) * 17
    q8 = np.zeros((1, 16 * 36), dtype=np.uint8)
    q8[0, 0:2] = np.array([0.25], dtype=np.float16).view(np.uint8)
    q = np.where(np.arange(32) % 16 < 8, 2, -2).astype(np.int8)
    q8[0, 4:36] = q.view(np.uint8)
    assert oracle.vecq_block_sums(oracle.TYPE_MXFP4, w, q8, 32, 1)[0, 0, 0] == 288
    assert oracle.vecq(oracle.TYPE_MXFP4, w, q8, 32, 1)[0, 0, 0] == 18.0


def test_decode_products_values_and_layouts():
    """The decode products' oracle (orc_decode_value, orc_decode_vector) against the reference's known
    answers and independent restatements: NVFP4 bytes of 0x22 are ones times their block scale in
    all four layouts, undefined scales NaN (tests/unit/reference_decode_test.cc:407-462); every
    layout of an encoding holds the same values; the product is the decoded matrix times x."""
    from llmp_amd import synth
    scales8 = [0x00, 0x01, 0x38, 0x7E, 0x7F, 0x80, 0xB8, 0xFF]
    for b in range(256):  # decode.cc:407-411
        v = oracle.lib.orc_ue4m3_to_f32(b)
        assert np.isnan(v) == (b >= 0x7F)
        if b < 0x7F:
            assert v == oracle.lib.orc_e4m3_to_f32(b)
    assert oracle.lib.orc_ue4m3_to_f32(0x38) == 1.0 and oracle.lib.orc_ue4m3_to_f32(0x01) == 2.0 ** -9
    k, n, blocks = 128, 4, 8
    codes = np.full((n, k // 2), 0x22, dtype=np.uint8)
    scales = np.array([scales8[i % 8] for i in range(n * blocks)], dtype=np.uint8).reshape(n, blocks)
    atoms = np.zeros(128 * blocks, dtype=np.uint8)
    for r in range(n):
        for b in range(blocks):
            atoms[oracle.lib.orc_scale_atom_offset(r, b, blocks)] = scales[r, b]
    ggml = np.concatenate([scales.reshape(n, k // 64, 4), np.full((n, k // 64, 32), 0x22, dtype=np.uint8)],
                          axis=-1).reshape(n, -1)
    layouts = {3: {"k": k, "data": codes, "scales": scales.reshape(-1)},
               4: {"k": k, "data": codes, "scales": atoms},
               5: {"k": k, "data": np.ascontiguousarray(np.concatenate([codes, scales], axis=1))},
               6: {"k": k, "data": np.ascontiguousarray(ggml)}}
    for decoder, w in layouts.items():
        got = oracle.decode_rows_of(decoder, w)
        for i in range(n * k):
            sc = scales.reshape(-1)[i // 16]
            if sc >= 0x7F:
                assert np.isnan(got.reshape(-1)[i]), (decoder, i)
            else:
                assert got.reshape(-1)[i] == oracle.lib.orc_e4m3_to_f32(sc), (decoder, i)
    # Random weights: the layouts of one encoding hold the same values; numpy restatements.
    e2m1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float32)
    n, k = 130, 256
    w6 = synth.decode_weight(6, n, k, 41)
    codes, scales = w6["plain"]
    nib = np.stack([codes & 15, codes >> 4], axis=-1).reshape(n, k)  # value 2 i in byte i's low nibble
    ue = np.array([oracle.lib.orc_ue4m3_to_f32(b) for b in range(256)], dtype=np.float32)
    want = e2m1[nib] * np.repeat(ue[scales], 16, axis=1)
    assert np.array_equal(oracle.decode_rows_of(6, w6), want)
    for decoder in (3, 4, 5):
        w = synth.decode_weight(decoder, n, k, 41)  # the same seed: the same codes and scales
        assert np.array_equal(oracle.decode_rows_of(decoder, w), want), decoder
    for split, atoms_id, per in ((7, 8, 32), (9, 10, 32)):
        a, b = synth.decode_weight(split, n, k, 42), synth.decode_weight(atoms_id, n, k, 42)
        assert np.array_equal(oracle.decode_rows_of(split, a), oracle.decode_rows_of(atoms_id, b))
    w9 = synth.decode_weight(9, n, k, 43)
    nib = np.stack([w9["data"] & 15, w9["data"] >> 4], axis=-1).reshape(n, k)
    e8 = np.exp2(w9["scales"].reshape(n, k // 32).astype(np.float32) - 127)
    assert np.array_equal(oracle.decode_rows_of(9, w9), e2m1[nib] * np.repeat(e8, 32, axis=1))
    w0 = synth.decode_weight(0, 9, 64, 44)
    assert np.array_equal(oracle.decode_rows_of(0, w0), synth.bf16_to_f32(w0["data"].view(np.uint16)))
    w1 = synth.decode_weight(1, 9, 64, 45)
    assert np.array_equal(oracle.decode_rows_of(1, w1), w1["data"].view(np.float16).astype(np.float32))
    w2 = synth.decode_weight(2, 9, 64, 46)
    assert np.array_equal(oracle.decode_rows_of(2, w2), oracle.decode_rows(oracle.TYPE_Q8_0, w2["data"], 64))
    # The product: decoded rows times x, a window of rows, tensor scales once an output.
    w = synth.decode_weight(6, 64, 128, 47, tensor_scales=2)
    x = np.random.Generator(np.random.PCG64(48)).standard_normal((3, 128)).astype(np.float32)
    dense = oracle.decode_rows_of(6, w).astype(np.float64)
    scale = w["tensor_scale"][np.arange(64) // 32].astype(np.float64)
    want = (x.astype(np.float64) @ dense.T) * scale
    np.testing.assert_allclose(oracle.decode_vector(6, w, x), want, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(oracle.decode_vector(6, w, x, first=20, outputs=30), want[:, 20:50], rtol=1e-6, atol=1e-9)


def test_affine_decoder_against_a_numpy_restatement():
    """The affine encoding (src/kernels/reference/decode.cc:173-220): codes of 4 or 8 bits little-endian along the
    row, s * q + b rounded once or s * (q - z), scales F16 / BF16 / F32 a group; restated with numpy (the fused
    multiply-add as an exact double product and sum rounded once)."""
    from llmp_amd import synth
    n, k, group = 5, 256, 64
    for bits in (4, 8):
        for scale in ("f16", "bf16", "f32"):
            for zero_point in (False, True):
                w = synth.affine_weight(n, k, 61, bits=bits, group=group, scale=scale, zero_point=zero_point)
                got = oracle.decode_rows_of(11, w)
                codes = w["data"] if bits == 8 else np.stack([w["data"] & 15, w["data"] >> 4], axis=-1).reshape(n, k)
                kind = w["scale_type"] & 0x7F

                def floats(raw):
                    if kind == 2:
                        return synth.bf16_to_f32(raw.view(np.uint16)).reshape(n, -1)
                    return raw.view(np.float16 if kind == 1 else np.float32).astype(np.float32).reshape(n, -1)

                sc = np.repeat(floats(w["scales"]), group, axis=1)
                if zero_point:
                    z = w["biases"] if bits == 8 else np.stack([w["biases"] & 15, w["biases"] >> 4], axis=-1).reshape(n, -1)
                    z = np.repeat(z[:, :k // group].astype(np.int32), group, axis=1)
                    want = sc * (codes.astype(np.int32) - z).astype(np.float32)
                else:
                    b = np.repeat(floats(w["biases"]), group, axis=1)
                    want = (sc.astype(np.float64) * codes.astype(np.float64) + b.astype(np.float64)).astype(np.float32)
                assert np.array_equal(got, want), (bits, scale, zero_point)
    # By hand: 4-bit codes 0..15 in one group of 32 (twice), s = 0.5, b = -4: values -4 .. 3.5.
    w = {"k": 32, "data": np.array([[(2 * i % 16) | ((2 * i + 1) % 16) << 4 for i in range(16)]], dtype=np.uint8),
         "scales": np.array([0.5], dtype=np.float16).view(np.uint8).reshape(1, 2),
         "biases": np.array([-4.0], dtype=np.float16).view(np.uint8).reshape(1, 2),
         "group": 32, "bits": 4, "scale_type": 1, "scale_row_bytes": 2}
    assert np.array_equal(oracle.decode_rows_of(11, w)[0], 0.5 * (np.arange(32) % 16) - 4.0)


def test_decode_glu_products_against_closed_forms():
    """orc_decode_vector_glu: glu(gate . x, up . x) with the four functions of the reference's CPU executor
    (src/kernels/reference/exec.cc:248-262), here from scipy's erf and numpy, over the oracle's own plain products."""
    from scipy.special import erf
    from llmp_amd import synth
    n, k = 24, 128
    gate = synth.decode_weight(9, n, k, 51, tensor_scales=2)
    up = synth.decode_weight(9, n, k, 52)
    x = np.random.Generator(np.random.PCG64(53)).standard_normal((2, k)).astype(np.float32) * 0.25
    g = oracle.decode_vector(9, gate, x).astype(np.float64)
    u = oracle.decode_vector(9, up, x).astype(np.float64)
    silu = lambda v: v / (1.0 + np.exp(-v))
    forms = {0: silu(g) * u,
             1: 0.5 * g * (1.0 + erf(g / np.sqrt(2.0))) * u,
             2: 0.5 * g * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g + 0.044715 * g ** 3))) * u,
             3: silu(np.minimum(g, 0.75)) * np.clip(u, -0.75, 0.75)}
    for kind, want in forms.items():
        got = oracle.decode_vector_glu(9, gate, up, x, kind, 0.75 if kind == 3 else 0.0)
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)
    # Row windows of one stacked weight.
    both = synth.decode_weight(3, 2 * n, k, 54)
    got = oracle.decode_vector_glu(3, both, both, x, 0, gate_first=0, up_first=n, outputs=n)
    want = silu(oracle.decode_vector(3, both, x, first=0, outputs=n).astype(np.float64)) * oracle.decode_vector(3, both, x, first=n, outputs=n)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)


def kv_blocks_numpy(t, x):
    """src/kernels/ggml/kv_quant.cuh:27-69 restated with numpy float32 operations (IEEE, one
    rounding each), apart from the oracle's C."""
    f = np.float32
    out = []
    for block in x.reshape(-1, 32).astype(np.float32):
        if t == oracle.TYPE_Q8_0:
            amax = f(np.max(np.abs(block)))
            d = f(amax / f(127.0))
            inv = f(f(1.0) / d) if d != 0 else f(0.0)
            scaled = (block * inv).astype(np.float32)
            codes = np.where(scaled >= 0, np.floor(scaled + f(0.5)), np.ceil(scaled - f(0.5)))
            # roundf is half away from zero; floor(x + 0.5) in float32 can round up a value just below
            # a half step, so compare in float64, where x + 0.5 is exact.
            s64 = scaled.astype(np.float64)
            codes = np.where(s64 >= 0, np.floor(s64 + 0.5), np.ceil(s64 - 0.5))
            out.append(np.concatenate([np.array([d], dtype=np.float16).view(np.uint8),
                                       codes.astype(np.int8).view(np.uint8)]))
        else:
            first = int(np.argmax(np.abs(block)))  # the first among equals
            vmax = block[first] if np.abs(block[first]) > 0 else f(0.0)
            d = f(vmax / f(-8.0))
            inv = f(f(1.0) / d) if d != 0 else f(0.0)
            scaled = ((block * inv).astype(np.float32) + f(8.5)).astype(np.float32)
            codes = np.minimum(15, np.trunc(scaled).astype(np.int64))
            packed = (codes[:16] | (codes[16:] << 4)).astype(np.uint8)
            out.append(np.concatenate([np.array([d], dtype=np.float16).view(np.uint8), packed]))
    return np.concatenate(out)


def test_kv_cache_quantizers_by_restatement_and_properties():
    from llmp_amd import synth
    g = synth.rng(81)
    x = g.standard_normal((7, 128), dtype=np.float32) * 2.5
    x[0, :32] = 0.0
    x[1, :32] = np.tile(np.array([-3.0, 3.0], dtype=np.float32), 16)
    x[2, :32] = np.tile(np.array([3.0, -3.0], dtype=np.float32), 16)
    x[3, :32] = (np.arange(32, dtype=np.float32) - 15.5) * 0.5
    for t in (oracle.TYPE_Q8_0, oracle.TYPE_Q4_0):
        got = oracle.kv_quantize(t, x)
        for r in range(x.shape[0]):
            assert np.array_equal(got[r], kv_blocks_numpy(t, x[r])), (t, r)
        # Decoding what was stored lands within half a step of the input (a full step at Q4_0's
        # clamped upper end), and a zero block stays zero.
        dec = oracle.decode_rows(t, got, 128)
        size = oracle.block_bytes(t)
        d = np.abs(got.reshape(7, -1, size)[:, :, 0:2].copy().view(np.float16).astype(np.float32)).repeat(32, axis=2).reshape(7, 128)
        bound = d * (0.5 if t == oracle.TYPE_Q8_0 else 1.0) * 1.001 + 1e-7
        assert np.all(np.abs(dec - x) <= bound + np.abs(x) * 2e-3), t
        assert np.all(dec[0, :32] == 0.0)
    # Q4_0 takes its scale from the first value of largest magnitude: -3 first gives d = 0.375,
    # codes 0 and 15 (clamped from 16); 3 first gives d = -0.375 and the codes swap.
    q = oracle.kv_quantize(oracle.TYPE_Q4_0, x[1:3, :32])
    assert q[0, 0:2].view(np.float16)[0] == np.float16(0.375) and q[1, 0:2].view(np.float16)[0] == np.float16(-0.375)
    assert (q[0, 2] & 15, q[0, 3] & 15) == (0, 15) and (q[1, 2] & 15, q[1, 3] & 15) == (0, 15)


def test_hand_built_blocks_have_known_sums():
    w = np.zeros((1, 34), dtype=np.uint8)
    w[0, 0:2] = np.array([2.0], dtype=np.float16).view(np.uint8)
    w[0, 2:] = np.arange(1, 33, dtype=np.int8).view(np.uint8)
    q8 = np.zeros((1, 16 * 36), dtype=np.uint8)
    q8[0, 0:2] = np.array([0.5], dtype=np.float16).view(np.uint8)
    q8[0, 4:36] = np.full(32, 3, dtype=np.int8).view(np.uint8)
    assert oracle.vecq_block_sums(oracle.TYPE_Q8_0, w, q8, 32, 1)[0, 0, 0] == 3 * 528
    assert oracle.vecq(oracle.TYPE_Q8_0, w, q8, 32, 1)[0, 0, 0] == 2.0 * 0.5 * 3 * 528
    # Q4_K: sub-block g has scale g + 1 and minimum 2 g; every code 15 low, 1 high.
    b = np.zeros((1, 144), dtype=np.uint8)
    b[0, 0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    b[0, 2:4] = np.array([0.5], dtype=np.float16).view(np.uint8)
    sc = [g + 1 for g in range(8)]
    mn = [2 * g for g in range(8)]
    s = np.zeros(12, dtype=int)
    for g in range(4):
        s[g] = sc[g] | ((sc[g + 4] >> 4) << 6)
        s[g + 4] = mn[g] | ((mn[g + 4] >> 4) << 6)
        s[g + 8] = (sc[g + 4] & 15) | ((mn[g + 4] & 15) << 4)
    b[0, 4:16] = s
    b[0, 16:] = 0x1F
    a = np.zeros((1, 16 * 36), dtype=np.uint8)
    for g in range(8):
        a[0, g * 36:g * 36 + 2] = np.array([1.0], dtype=np.float16).view(np.uint8)
        a[0, g * 36 + 4:g * 36 + 36] = np.full(32, 2, dtype=np.int8).view(np.uint8)
    sums = oracle.vecq_block_sums(oracle.TYPE_Q4_K, b, a, 256, 1)[0, 0]
    assert list(sums[:8]) == [15 * 64 if g % 2 == 0 else 64 for g in range(8)]
    assert list(sums[8:]) == [64] * 8
    want = sum(1.0 * sc[g] * sums[g] - 0.5 * mn[g] * 64 for g in range(8))
    assert oracle.vecq(oracle.TYPE_Q4_K, b, a, 256, 1)[0, 0, 0] == want


def test_glu_closed_forms():
    """tests/unit/dsv4_fast_test.cc:401-408 (tanh GELU) and exec.cc:206-214,248-262 of the reference."""
    for g, u in [(0.3, -1.2), (-2.0, 0.7), (5.0, 5.0), (0.0, 3.0)]:
        gelu = 0.5 * g * (1 + math.tanh(math.sqrt(2.0 / math.acos(-1.0)) * g * (1 + 0.044715 * g * g)))
        assert oracle.glu(oracle.GLU_GEGLU, g, u) == pytest.approx(gelu * u, rel=1e-15)
        assert oracle.glu(oracle.GLU_SWIGLU, g, u) == pytest.approx(g / (1 + math.exp(-g)) * u, rel=1e-15)
        gc, uc = min(g, 1.0), max(-1.0, min(1.0, u))
        assert oracle.glu(oracle.GLU_SWIGLU_CLAMP, g, u, 1.0) == pytest.approx(gc / (1 + math.exp(-gc)) * uc, rel=1e-15)


def test_vecq_forms_route_to_the_right_rows():
    """Dense, grouped and routed indexing against an explicit loop over decoded weights."""
    from llmp_amd import synth
    t, k, n, experts = oracle.TYPE_Q8_0, 64, 6, 5
    w = synth.random_blocks(t, experts * n, k, 9).reshape(experts, -1)
    dec = oracle.decode_rows(t, w.reshape(experts * n, -1), k).reshape(experts, n, k).astype(np.float64)
    x = np.random.Generator(np.random.PCG64(10)).standard_normal((3, k)).astype(np.float32)
    q8 = oracle.q8_1_quantize(x)
    act = np.stack([oracle.q8_1_decode(q8[i], k) for i in range(3)]).astype(np.float64)
    ids = np.array([[4, 0], [1, 1], [2, 3]], dtype=np.int32)
    got = oracle.vecq(t, w, q8, k, n, ids=ids, tokens=3, used=2, stride_expert=n * (k // 32), experts=experts)
    for tok in range(3):
        for u in range(2):
            np.testing.assert_allclose(got[tok, u], dec[ids[tok, u]] @ act[tok], rtol=1e-6)
    with pytest.raises(IndexError):
        oracle.vecq(t, w, q8, k, n, ids=np.array([[5, 0]], dtype=np.int32), tokens=1, used=2,
                    stride_expert=n * (k // 32), experts=experts)


# --------------------------------------------------------------------- MXFP8


def test_mxfp8_quantize_invariants():
    """tests/unit/qwen38_fast_test.cc:179-218 of the reference: each scale the smallest power of two with
    amax <= 448 * s, each value within half an E4M3 step, padding rows' scales zero."""
    g = np.random.Generator(np.random.PCG64(11))
    rows, k = 5, 128
    x = (g.standard_normal((rows, k)) * np.exp(g.uniform(-8, 8, (rows, 1)))).astype(np.float32)
    x[0, :32] = 0
    x[1, 33] = 448.0
    x[1, 32:64] = np.clip(x[1, 32:64], -448, 448)
    codes, scales = oracle.mxfp8_quantize(x)
    blocks = k // 32
    for r in range(128):
        for b in range(blocks):
            e = scales[lib.orc_scale_atom_offset(r, b, blocks)]
            if r >= rows:
                assert e == 0
                continue
            v = x[r, b * 32:(b + 1) * 32].astype(np.float64)
            s = 2.0 ** (int(e) - 127)
            amax = np.abs(v).max()
            if amax > 0:
                assert amax <= 448 * s * (1 + 1e-6) and amax > 224 * s * (1 - 1e-6)
            q = np.array([e4m3_closed_form(int(c)) for c in codes[r, b * 32:(b + 1) * 32]]) * s
            mag = np.abs(v) / s
            step = np.where(mag < 2.0 ** -6, 2.0 ** -9, 2.0 ** (np.floor(np.log2(np.maximum(mag, 1e-300))) - 3))
            assert np.all(np.abs(q - v) <= 0.5 * step * s * (1 + 1e-6))
    assert lib.orc_mxfp8_scale_code(0.0) == 0 and lib.orc_mxfp8_scale_code(448.0) == 127
    assert lib.orc_mxfp8_scale_code(449.0) == 128 and lib.orc_mxfp8_inverse_scale(127) == 1.0


def test_scale_atoms_and_gemm_are_the_plain_block_scaled_product():
    """src/format/layout.h:108-113 and tests/unit/reference_decode_test.cc:531-568 of the reference."""
    assert lib.orc_scale_atom_offset(0, 0, 8) == 0
    assert lib.orc_scale_atom_offset(1, 0, 8) == 16 and lib.orc_scale_atom_offset(32, 0, 8) == 4
    assert lib.orc_scale_atom_offset(0, 1, 8) == 1 and lib.orc_scale_atom_offset(0, 4, 8) == 512
    assert lib.orc_scale_atom_offset(128, 0, 8) == 1024
    seen = {lib.orc_scale_atom_offset(r, b, 8) for r in range(256) for b in range(8)}
    assert seen == set(range(256 * 8))  # a bijection onto the padded area
    g = np.random.Generator(np.random.PCG64(12))
    m, n, k = 6, 9, 128  # scale atoms take rows of whole groups of four scales
    a = g.standard_normal((m, k)).astype(np.float32)
    w = (g.standard_normal((n, k)) * 0.02).astype(np.float32)
    ac, asc = oracle.mxfp8_quantize(a)
    wc, wsc = oracle.mxfp8_quantize(w)

    def dequant(codes, scales, rows):
        out = np.zeros((rows, k))
        for r in range(rows):
            for j in range(k):
                out[r, j] = e4m3_closed_form(int(codes[r, j])) * 2.0 ** (int(scales[lib.orc_scale_atom_offset(r, j // 32, k // 32)]) - 127)
        return out
    want = dequant(ac, asc, m) @ dequant(wc, wsc, n).T
    got = oracle.mxfp8_gemm(ac, asc, wc, wsc)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-7)
    assert oracle.mxfp8_dot(ac, asc, 2, wc, wsc, 3) == pytest.approx(want[2, 3], rel=1e-12)
    np.testing.assert_allclose(want, a.astype(np.float64) @ w.astype(np.float64).T, rtol=0.2, atol=0.02)
    # The swizzle of plain [n][k/32] scales is the same placement.
    plain = g.integers(100, 140, size=(n, k // 32), dtype=np.uint8)
    sw = oracle.mxfp8_swizzle(plain)
    assert all(sw[lib.orc_scale_atom_offset(r, b, k // 32)] == plain[r, b] for r in range(n) for b in range(k // 32))
    y = oracle.mxfp8_gemv(wc, np.stack([[wsc[lib.orc_scale_atom_offset(r, b, k // 32)] for b in range(k // 32)]
                                        for r in range(n)]).astype(np.uint8), a)
    np.testing.assert_allclose(y, a.astype(np.float64) @ dequant(wc, wsc, n).T, rtol=1e-5, atol=1e-7)


# ----------------------------------------------------------------------- MoE


def test_route_sort_and_reduce_against_numpy():
    g = np.random.Generator(np.random.PCG64(13))
    logits = g.standard_normal((9, 32)).astype(np.float32)
    logits[3, [4, 7]] = logits[3].max() + 1  # a tie for first: the lower index wins
    ids, w = oracle.route(logits, 4)
    for t in range(9):
        l = logits[t].astype(np.float64)
        p = np.exp(l - l.max())
        p /= p.sum()
        order = np.argsort(-p, kind="stable")[:4]
        assert list(ids[t]) == list(order)
        np.testing.assert_allclose(w[t], p[order] / p[order].sum(), rtol=1e-6)
    assert list(ids[3][:2]) == [4, 7]
    bad = np.full((1, 8), np.nan, dtype=np.float32)
    ids, w = oracle.route(bad, 3)
    assert list(ids[0]) == [0, 1, 2] and not w.any()
    tiny = np.full((1, 8), -1e4, dtype=np.float32)
    tiny[0, 0] = 0
    _, w = oracle.route(tiny, 2, normalize=False, scale=3.0)
    assert w[0, 0] == 3.0 and w[0, 1] == 0.0
    flat = np.array([3, 1, 3, 0, 1, 3], dtype=np.int32)
    order, offsets = oracle.expert_sort(flat, 4)
    assert list(order) == [3, 1, 4, 0, 2, 5] and list(offsets) == [0, 1, 3, 3, 6]
    with pytest.raises(IndexError):
        oracle.expert_sort(np.array([4], dtype=np.int32), 4)
    x = g.standard_normal((2, 3, 8)).astype(np.float32)
    ww = g.random((2, 3)).astype(np.float32)
    np.testing.assert_allclose(oracle.expert_reduce(x, ww), (x * ww[:, :, None]).sum(axis=1), rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------------- EXL3

GOLDEN = [(0x0000, 0x3A25, 0x3F60, 0xC2E8), (0x0001, 0xBB5B, 0x304E, 0x3921), (0x1234, 0xC066, 0x3E0F, 0xB89E),
          (0x8000, 0xB7F8, 0xB915, 0xBAF2), (0xBEEF, 0x424B, 0xC293, 0x3124), (0xFFFF, 0xB110, 0x3ACD, 0xB936)]


def test_exl3_codebooks_match_the_reference_golden_vectors():
    """tests/unit/reference_decode_test.cc:677-682 of the reference: six states, three codebooks."""
    for state, three_inst, mcg, mul1 in GOLDEN:
        assert lib.orc_exl3_codebook(oracle.CB_3INST, state) == three_inst
        assert lib.orc_exl3_codebook(oracle.CB_MCG, state) == mcg
        assert lib.orc_exl3_codebook(oracle.CB_MUL1, state) == mul1
    assert lib.orc_exl3_codebook(3, 0) == 0x7E00


def test_exl3_tiles_follow_the_independent_derivation():
    """tests/unit/reference_decode_test.cc:699-747 of the reference: state p is the 16 bits of the tile's
    circular MSB-first stream ending at bit (p + 1) K; position 8 L + i of a lane without bit 2 lands at row
    (L % 4) * 2 + {0, 1, 8, 9}[i % 4], column 2 (L / 8 + 4 (i / 4)), lane L + 4's one column right."""
    kk, nn = 32, 48
    for bits in range(1, 9):
        trellis = np.random.Generator(np.random.PCG64(100 + bits)).integers(0, 256, size=(kk // 16) * (nn // 16) * 32 * bits,
                                                                           dtype=np.uint8)
        want = np.zeros((kk, nn), dtype=np.uint16)
        tile_bytes = 32 * bits
        for kt in range(kk // 16):
            for nt in range(nn // 16):
                tile = trellis[(kt * (nn // 16) + nt) * tile_bytes:][:tile_bytes]
                words = tile.view(np.uint32)
                length = 256 * bits
                stream = np.array([(int(words[j // 32]) >> (31 - j % 32)) & 1 for j in range(length)])
                for p in range(256):
                    end = (p + 1) * bits
                    state = 0
                    for i in range(16):
                        state = (state << 1) | int(stream[(end + length - 16 + i) % length])
                    group = p // 8
                    partner = (group & 4) != 0
                    lane = group - 4 if partner else group
                    i = p % 8
                    row = (lane % 4) * 2 + [0, 1, 8, 9][i % 4]
                    col = 2 * (lane // 8 + 4 * (i // 4)) + (1 if partner else 0)
                    want[kt * 16 + row, nt * 16 + col] = lib.orc_exl3_codebook(oracle.CB_MCG, state)
        got = oracle.exl3_rotated(trellis, kk, nn, bits, oracle.CB_MCG)
        assert np.array_equal(got, want), bits
        part = oracle.exl3_rotated(trellis, kk, nn, bits, oracle.CB_MCG, 16, 32)
        assert np.array_equal(part, want[:, 16:48])


def test_exl3_rows_are_the_explicit_hadamard_product():
    """tests/unit/reference_decode_test.cc:754-814 of the reference: W = diag(suh) H W^ H diag(svh) / 128
    with explicit Hadamard matrices in F64, bit-equal for 3INST and MCG."""
    kk, nn = 256, 384
    idx = np.arange(128)
    h128 = np.where(np.array([[bin(i & j).count("1") % 2 for j in idx] for i in idx]) == 0, 1.0, -1.0)
    g = np.random.Generator(np.random.PCG64(200))
    for bits, codebook in [(4, oracle.CB_3INST), (3, oracle.CB_3INST), (4, oracle.CB_MCG), (6, oracle.CB_MCG)]:
        trellis = g.integers(0, 256, size=(kk // 16) * (nn // 16) * 32 * bits, dtype=np.uint8)
        suh = (g.choice([-1.0, 1.0], kk) * g.uniform(0.25, 2.0, kk)).astype(np.float16)
        svh = (g.choice([-1.0, 1.0], nn) * g.uniform(0.25, 2.0, nn)).astype(np.float16)
        rot = oracle.exl3_rotated(trellis, kk, nn, bits, codebook).view(np.float16).astype(np.float64)
        a = np.zeros_like(rot)
        for kb in range(0, kk, 128):
            a[kb:kb + 128] = h128 @ rot[kb:kb + 128]
        w = np.zeros_like(rot)
        for nb in range(0, nn, 128):
            w[:, nb:nb + 128] = a[:, nb:nb + 128] @ h128
        want = (w * suh.astype(np.float64)[:, None] * svh.astype(np.float64)[None, :] / 128.0).T.astype(np.float32)
        got = oracle.exl3_rows(trellis, suh.view(np.uint16), svh.view(np.uint16), kk, nn, bits, codebook)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        some = oracle.exl3_rows(trellis, suh.view(np.uint16), svh.view(np.uint16), kk, nn, bits, codebook, 100, 200)
        assert np.array_equal(some, got[100:300])
        # The linear over these rows: within the F16 rounding of the transformed input
        # (tests/unit/exl3_trellis_test.cc:519-564: relative RMS 2^-8 a row).
        x = g.standard_normal((2, kk)).astype(np.float16)
        y = oracle.exl3_linear(trellis, suh.view(np.uint16), svh.view(np.uint16), kk, nn, bits, codebook, x.view(np.uint16))
        ref = x.astype(np.float64) @ got.astype(np.float64).T
        for r in range(2):
            assert np.sqrt(np.mean((y[r] - ref[r]) ** 2)) <= 2.0 ** -8 * np.sqrt(np.mean(ref[r] ** 2))


def test_rope_neox_against_complex_rotations_and_yarn_closed_forms():
    """oracle.rope_neox (src/kernels/reference/exec.cc:1343-1484 of the reference) against an independent form: a
    pair (c, c + n_dims / 2) as a complex number times exp(i theta); position 0 is the identity; channels past n_dims
    pass; the frequency factor divides the angle; YaRN with every pair inside the ramp (ramp = 1) keeps the
    extrapolated angle and raises the magnitude by 1 + 0.1 ln(1 / scale), with every pair past it (ramp = 0) the
    interpolated one."""
    g = np.random.Generator(np.random.PCG64(91))
    tokens, heads, head_dim, n_dims = 5, 3, 64, 48
    x = g.standard_normal((tokens, heads, head_dim)).astype(np.float32)
    pos = np.array([0, 1, 7, 300, 4095], dtype=np.int32)
    theta_scale = np.float32(10000.0 ** (-2.0 / n_dims))
    half = n_dims // 2

    def rotate(angle, magnitude=1.0):
        z = (x[:, :, :half].astype(np.float64) + 1j * x[:, :, half:n_dims].astype(np.float64))
        z = z * np.exp(1j * angle)[:, None, :] * magnitude
        want = x.astype(np.float64).copy()
        want[:, :, :half], want[:, :, half:n_dims] = z.real, z.imag
        return want

    base = pos[:, None].astype(np.float64) * np.float64(theta_scale) ** np.arange(half)[None, :]
    got = oracle.rope_neox(x, pos, n_dims, theta_scale)
    # The angle is formed in F32 steps: at position 4095 it is good to about 4095 * 2^-23.
    np.testing.assert_allclose(got, rotate(base), atol=3e-3, rtol=0)
    np.testing.assert_allclose(got[:3], rotate(base)[:3], atol=2e-6, rtol=0)
    assert np.array_equal(got[0], x[0]) and np.array_equal(got[:, :, n_dims:], x[:, :, n_dims:])
    ff = g.uniform(0.5, 4.0, size=half).astype(np.float32)
    np.testing.assert_allclose(oracle.rope_neox(x, pos, n_dims, theta_scale, freq_factors=ff)[:3],
                               rotate(base / ff[None, :])[:3], atol=2e-6, rtol=0)
    np.testing.assert_allclose(oracle.rope_neox(x, pos, n_dims, theta_scale, freq_scale=0.25)[:3],
                               rotate(0.25 * base)[:3], atol=2e-6, rtol=0)
    inside = oracle.rope_neox(x, pos, n_dims, theta_scale, freq_scale=0.25, ext_factor=1.0, attn_factor=1.5,
                              corr_dims=(100.0, 200.0))
    np.testing.assert_allclose(inside[:3], rotate(base, 1.5 * (1.0 + 0.1 * np.log(4.0)))[:3], atol=4e-6, rtol=0)
    past = oracle.rope_neox(x, pos, n_dims, theta_scale, freq_scale=0.25, ext_factor=1.0, attn_factor=1.5,
                            corr_dims=(-200.0, -100.0))
    np.testing.assert_allclose(past[:3], rotate(0.25 * base, 1.5 * (1.0 + 0.1 * np.log(4.0)))[:3], atol=4e-6, rtol=0)
    # Rotations keep a pair's length.
    n0 = np.hypot(x[:, :, :half], x[:, :, half:n_dims])
    np.testing.assert_allclose(np.hypot(got[:, :, :half], got[:, :, half:n_dims]), n0, rtol=1e-6)


def test_grouped_nvfp4_values_and_product_by_scalar_loops():
    """llmp.moe.gemm's operands (src/kernels/ggml/moe_cutlass.h:12-46 of the reference): element 2i in byte i's low
    nibble, one UE4M3 scale per 16 elements at SfOffset in a block of rows from sf_rows[e]. The vectorised decode
    against scalar loops over the pinned conversions, known answers (bytes of 0x22 are ones, a scale byte of 0x38 is
    1.0, 0x40 is 2.0), and the product against explicit dot products."""
    g = np.random.default_rng(5)
    k, n = 128, 7
    offsets = np.array([0, 3, 3, 8], dtype=np.int32)
    sf_rows = np.array([0, 128, 128, 256], dtype=np.int32)
    a_codes = g.integers(0, 256, size=(8, k // 2), dtype=np.uint8)
    a_scales = g.integers(0, 0x7F, size=256 * (k // 16), dtype=np.uint8)
    b_codes = [g.integers(0, 256, size=(n, k // 2), dtype=np.uint8) for _ in range(3)]
    b_scales = [g.integers(0, 0x7F, size=128 * (k // 16), dtype=np.uint8) for _ in range(3)]
    ones = oracle.nvfp4_values(np.full((2, k // 2), 0x22, dtype=np.uint8), np.full(128 * (k // 16), 0x38, dtype=np.uint8), 2, k)
    assert np.array_equal(ones, np.ones((2, k)))
    twos = oracle.nvfp4_values(np.full((1, k // 2), 0x22, dtype=np.uint8), np.full(128 * (k // 16), 0x40, dtype=np.uint8), 1, k)
    assert np.array_equal(twos, 2 * np.ones((1, k)))

    def value(codes, scales, r, j, row0):
        byte = int(codes[r, j // 2])
        code = byte >> 4 if j % 2 else byte & 15
        where = ((((row0 + r) // 128) * ((k // 16) // 4)) + ((j // 16) // 4)) * 512 + (((row0 + r) % 32) * 16) + \
            ((((row0 + r) % 128) // 32) * 4) + ((j // 16) % 4)  # SfOffset, moe_cutlass.h:42-46
        return float(oracle.lib.orc_e2m1_to_f32(code)) * float(oracle.lib.orc_ue4m3_to_f32(int(scales[where])))

    got = oracle.grouped_nvfp4_gemm(a_codes, a_scales, offsets, sf_rows, b_codes, b_scales, n, k)
    for e in (0, 2):
        for r in range(offsets[e], offsets[e + 1]):
            local = r - offsets[e]
            a_row = [value(a_codes[offsets[e]:], a_scales, local, j, int(sf_rows[e])) for j in range(k)]
            for c in (0, n - 1):
                b_row = [value(b_codes[e], b_scales[e], c, j, 0) for j in range(k)]
                assert got[r, c] == pytest.approx(sum(x * y for x, y in zip(a_row, b_row)), rel=1e-12, abs=1e-12)


@pytest.mark.parametrize("t", [oracle.TYPE_Q8_0, oracle.TYPE_Q4_0])
def test_attention_over_a_quantized_cache_against_numpy_and_closed_forms(t):
    """orc_attention_quant (the reference executor's kAttention, src/kernels/reference/exec.cc:1027-1085, over Q8_0 /
    Q4_0 rows): against an independent numpy softmax attention over the rows decoded by the pinned block decoders
    (grouped heads, an F16 mask with -inf cells and finite biases, a softcap, sinks, pitched cells); and against what
    the mathematics fixes: equal keys give the mean of the seen values, one seen cell gives that cell's value, a row
    that sees nothing is zero, a large sink empties the output."""
    g = np.random.default_rng(31 + t)
    d, heads, kv_heads, rows, cells = 64, 6, 2, 3, 40
    row_bytes = d // 32 * oracle.block_bytes(t)
    keys = g.standard_normal((cells, kv_heads, d)).astype(np.float32)
    vals = g.standard_normal((cells, kv_heads, d)).astype(np.float32)
    pitch = row_bytes * kv_heads + 2 * oracle.block_bytes(t)  # a gap of two blocks after every cell
    k_cache = np.zeros((cells, pitch), dtype=np.uint8)
    v_cache = np.zeros((cells, pitch), dtype=np.uint8)
    k_cache[:, :row_bytes * kv_heads] = oracle.kv_quantize(t, keys.reshape(cells * kv_heads, d)).reshape(cells, -1)
    v_cache[:, :row_bytes * kv_heads] = oracle.kv_quantize(t, vals.reshape(cells * kv_heads, d)).reshape(cells, -1)
    kd = oracle.decode_rows(t, k_cache[:, :row_bytes * kv_heads].reshape(cells * kv_heads, row_bytes), d).reshape(cells, kv_heads, d).astype(np.float64)
    vd = oracle.decode_rows(t, v_cache[:, :row_bytes * kv_heads].reshape(cells * kv_heads, row_bytes), d).reshape(cells, kv_heads, d).astype(np.float64)
    q = g.standard_normal((heads, rows, d)).astype(np.float32)
    mask = np.full((rows + 1, cells), -np.inf, dtype=np.float16)
    for r in range(rows):
        mask[r, :cells - 7 + r] = 0.0
        mask[r, 1:cells - 7 + r:5] = -0.75
    sinks = g.standard_normal(heads).astype(np.float32)
    scale, softcap = 0.125, 3.0

    def numpy_attention(use_mask, use_sinks, cap):
        out = np.zeros((rows, heads, d))
        for h in range(heads):
            kh = h // (heads // kv_heads)
            for r in range(rows):
                s = (kd[:, kh, :] @ q[h, r].astype(np.float64)) * scale
                if cap > 0:
                    s = cap * np.tanh(s / cap)
                if use_mask:
                    s = s + mask[r].astype(np.float64)
                m = max(s.max(), float(sinks[h])) if use_sinks else s.max()
                e = np.exp(s - m)
                total = e.sum() + (np.exp(float(sinks[h]) - m) if use_sinks else 0.0)
                out[r, h] = (e / total) @ vd[:, kh, :]
        return out

    for use_mask, use_sinks, cap in ((True, False, 0.0), (True, True, softcap), (False, False, softcap)):
        got = oracle.attention_quant(t, q, k_cache, v_cache, d, heads, kv_heads, rows, cells, scale,
                                     mask=mask if use_mask else None, sinks=sinks if use_sinks else None, softcap=cap,
                                     cell_stride=pitch, head_stride=row_bytes)
        np.testing.assert_allclose(got, numpy_attention(use_mask, use_sinks, cap), rtol=2e-6, atol=2e-7)
    # Equal keys: every seen cell weighs the same, the output is the mean of the seen values.
    same = np.repeat(k_cache[:1], cells, axis=0)
    got = oracle.attention_quant(t, q, same, v_cache, d, heads, kv_heads, rows, cells, scale, mask=mask,
                                 cell_stride=pitch, head_stride=row_bytes)
    for r in range(rows):
        seen = np.isfinite(mask[r].astype(np.float64))
        w = np.exp(mask[r].astype(np.float64)[seen])
        want = (w / w.sum()) @ vd[seen][:, 0, :]
        np.testing.assert_allclose(got[r, 0], want, rtol=2e-6, atol=2e-7)
    # One seen cell: its value row, whatever the scores; none: zeros; a huge sink: nearly nothing.
    one = np.full((rows, cells), -np.inf, dtype=np.float16)
    one[:, 5] = 0.0
    one[2, :] = -np.inf
    got = oracle.attention_quant(t, q, k_cache, v_cache, d, heads, kv_heads, rows, cells, scale, mask=one,
                                 cell_stride=pitch, head_stride=row_bytes)
    np.testing.assert_allclose(got[0, 4], vd[5, 1], rtol=1e-6, atol=1e-7)
    assert np.all(got[2] == 0.0)
    big = oracle.attention_quant(t, q, k_cache, v_cache, d, heads, kv_heads, rows, cells, scale, mask=mask,
                                 sinks=np.full(heads, 80.0, dtype=np.float32), cell_stride=pitch, head_stride=row_bytes)
    assert np.abs(big).max() < 1e-20
    # Through Q8_1: the same attention over the decoded quantized queries.
    blocks = oracle.q8_1_quantize(q.reshape(heads * rows, d))
    q8 = np.stack([oracle.q8_1_decode(row, d) for row in blocks]).reshape(heads, rows, d)
    a = oracle.attention_quant(t, q, k_cache, v_cache, d, heads, kv_heads, rows, cells, scale, mask=mask, q8_1_q=True,
                               cell_stride=pitch, head_stride=row_bytes)
    b = oracle.attention_quant(t, q8, k_cache, v_cache, d, heads, kv_heads, rows, cells, scale, mask=mask,
                               cell_stride=pitch, head_stride=row_bytes)
    assert np.array_equal(a, b)
