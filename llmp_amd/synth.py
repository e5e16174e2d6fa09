"""Seeded synthetic inputs of the benchmark configurations (numpy, host side).

Weights are byte images of GGML blocks: Q8_0 {f16 d; i8 qs[32]}, Q4_K
{f16 d; f16 dmin; u8 scales[12]; u8 qs[128]} (src/format/encoding.cc:110-116
of the reference) and the legacy 4/5-bit blocks {f16 d; [f16 m;] [u32 high bits;]
u8 nibbles[16]} as tests/unit/dsv4_fast_test.cc:141-157 reads them."""
import numpy as np


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def q8_0_weights(n, k, seed):
    """[n, k/32*34] uint8: codes uniform in [-127, 127], each block's scale
    max|w| / 127 over 32 draws of N(0, 0.02)."""
    g = rng(seed)
    blocks = k // 32
    out = np.zeros((n, blocks, 34), dtype=np.uint8)
    amax = np.abs(g.standard_normal((n, blocks, 32), dtype=np.float32) * 0.02).max(axis=-1)
    out[:, :, 0:2] = (amax / 127.0).astype(np.float16).view(np.uint8).reshape(n, blocks, 2)
    out[:, :, 2:] = g.integers(-127, 128, size=(n, blocks, 32), dtype=np.int8).view(np.uint8)
    return out.reshape(n, blocks * 34)


def q4_k_weights(n, k, seed):
    """[n, k/256*144] uint8: 4-bit codes uniform 0..15, 6-bit sub-scales and minimums
    uniform 0..63, d and dmin sized so that d*63*15 and dmin*63 span the range of 256
    draws of N(0, 0.02) (about 5.6 and 2.8 standard deviations)."""
    g = rng(seed)
    blocks = k // 256
    out = np.zeros((n, blocks, 144), dtype=np.uint8)
    d = (0.02 * g.uniform(5.0, 6.2, size=(n, blocks)) / (63.0 * 15.0)).astype(np.float16)
    dmin = (0.02 * g.uniform(2.4, 3.2, size=(n, blocks)) / 63.0).astype(np.float16)
    out[:, :, 0:2] = d.view(np.uint8).reshape(n, blocks, 2)
    out[:, :, 2:4] = dmin.view(np.uint8).reshape(n, blocks, 2)
    out[:, :, 4:] = g.integers(0, 256, size=(n, blocks, 140), dtype=np.uint8)
    return out.reshape(n, blocks * 144)


def q5_k_weights(n, k, seed):
    """[n, k/256*176] uint8 of Q5_K super-blocks {f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]}:
    5-bit codes, 6-bit sub-scales and minimums uniform, d and dmin sized as for Q4_K."""
    g = rng(seed)
    blocks = k // 256
    out = np.zeros((n, blocks, 176), dtype=np.uint8)
    d = (0.02 * g.uniform(5.0, 6.2, size=(n, blocks)) / (63.0 * 31.0)).astype(np.float16)
    dmin = (0.02 * g.uniform(2.4, 3.2, size=(n, blocks)) / 63.0).astype(np.float16)
    out[:, :, 0:2] = d.view(np.uint8).reshape(n, blocks, 2)
    out[:, :, 2:4] = dmin.view(np.uint8).reshape(n, blocks, 2)
    out[:, :, 4:] = g.integers(0, 256, size=(n, blocks, 172), dtype=np.uint8)
    return out.reshape(n, blocks * 176)


def q6_k_weights(n, k, seed):
    """[n, k/256*210] uint8 of Q6_K super-blocks {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d}: 6-bit codes and
    int8 sub-scales uniform, d sized so that d * 127 * 32 spans the range of 256 draws of N(0, 0.02)."""
    g = rng(seed)
    blocks = k // 256
    out = g.integers(0, 256, size=(n, blocks, 210), dtype=np.uint8)
    d = (0.02 * g.uniform(5.0, 6.2, size=(n, blocks)) / (127.0 * 32.0)).astype(np.float16)
    out[:, :, 208:210] = d.view(np.uint8).reshape(n, blocks, 2)
    return out.reshape(n, blocks * 210)


LEGACY_BYTES = {2: 18, 3: 20, 6: 22, 7: 24, 20: 18}  # Q4_0, Q4_1, Q5_0, Q5_1; IQ4_NL (Q4_0's bytes)


def legacy_weights(t, n, k, seed):
    """[n, k/32*bytes] uint8 of a legacy block type: codes uniform, each block's scale the
    range of 32 draws of N(0, 0.02) over its code range (and a minimum at the low end)."""
    g = rng(seed)
    blocks, size = k // 32, LEGACY_BYTES[t]
    out = g.integers(0, 256, size=(n, blocks, size), dtype=np.uint8)
    levels = 31.0 if t in (6, 7) else 254.0 if t == 20 else 15.0  # IQ4_NL's codebook spans -127 .. 113
    amax = np.abs(g.standard_normal((n, blocks, 32), dtype=np.float32) * 0.02).max(axis=-1)
    out[:, :, 0:2] = (2.0 * amax / levels).astype(np.float16).view(np.uint8).reshape(n, blocks, 2)
    if t in (3, 7):
        out[:, :, 2:4] = (-amax).astype(np.float16).view(np.uint8).reshape(n, blocks, 2)
    return out.reshape(n, blocks * size)


def mxfp4_weights(n, k, seed, low=112, high=124):
    """[n, k/32*17] uint8 of MXFP4 blocks {e8m0 scale; 16 bytes of E2M1 codes}: codes uniform,
    scale bytes uniform in [low, high) (2^-15 .. 2^-4 by default: weights up to about 0.4)."""
    g = rng(seed)
    blocks = k // 32
    out = g.integers(0, 256, size=(n, blocks, 17), dtype=np.uint8)
    out[:, :, 0] = g.integers(low, high, size=(n, blocks), dtype=np.uint8)
    return out.reshape(n, blocks * 17)


def random_blocks(t, n, k, seed):
    """Every field random (any finite f16 scale up to magnitude 4, any scale byte, any code):
    the bytes a decoder must take, not a plausible quantization."""
    if t == 39:
        return mxfp4_weights(n, k, seed, 90, 150)  # 2^-37 .. 2^22: any code, no overflow
    g = rng(seed)
    if t in LEGACY_BYTES:
        blocks, size, heads = k // 32, LEGACY_BYTES[t], 2 if t in (3, 7) else 1
    elif t == 8:
        blocks, size, heads = k // 32, 34, 1
    elif t == 13:
        blocks, size, heads = k // 256, 176, 2
    elif t == 14:
        out = rng(seed).integers(0, 256, size=(n, k // 256, 210), dtype=np.uint8)
        scale = rng(seed + 1).uniform(-4.0, 4.0, size=(n, k // 256, 1)).astype(np.float16)
        out[:, :, 208:210] = scale.view(np.uint8).reshape(n, k // 256, 2)
        return out.reshape(n, k // 256 * 210)
    else:
        blocks, size, heads = k // 256, 144, 2
    out = g.integers(0, 256, size=(n, blocks, size), dtype=np.uint8)
    scale = (g.uniform(-4.0, 4.0, size=(n, blocks, heads))).astype(np.float16)
    out[:, :, 0:2 * heads] = scale.view(np.uint8).reshape(n, blocks, 2 * heads)
    return out.reshape(n, blocks * size)


def activations(tokens, k, seed, dtype=np.float32):
    return rng(seed).standard_normal((tokens, k), dtype=np.float32).astype(dtype)


def bf16_bits(x):
    """float32 -> bfloat16 bits, nearest even (src/kernels/reference/decode.cc:386-392)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def exl3_weights(k, n, bits, seed):
    """A trellis of seed-random words (every bit stream is a valid trellis), input signs
    suh = +-1 and output scales svh = +-|N(1, 0.1)|, both float16."""
    g = rng(seed)
    trellis = g.integers(0, 256, size=(k // 16) * (n // 16) * 32 * bits, dtype=np.uint8)
    suh = g.choice(np.array([-1.0, 1.0]), size=k).astype(np.float16)
    svh = (g.choice(np.array([-1.0, 1.0]), size=n) * np.abs(g.normal(1.0, 0.1, size=n))).astype(np.float16)
    return trellis, suh, svh


def decode_weight(decoder, n, k, seed, tensor_scales=0):
    """A weight of n rows of k values as decoder `decoder` (its index in the reference's DecoderId,
    src/kernels/decode/operand.h:26-41) reads it: a dict of data (uint8 [n, row_bytes]), k, and where the
    layout has them scales (uint8, flat) and, with `tensor_scales` > 0, that many F32 tensor scales. Codes are
    uniform bytes; block scales are kept in a range whose products stay finite."""
    g = rng(seed)
    w = {"k": k}

    def atoms(scales, blocks):  # [n, blocks] -> CUTLASS's scale atoms (src/format/layout.h)
        rows = (n + 127) // 128 * 128
        out = np.zeros(rows * blocks, dtype=np.uint8)
        r, b = np.meshgrid(np.arange(n), np.arange(blocks), indexing="ij")
        at = ((r // 128) * (blocks // 4) + b // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + b % 4
        out[at.reshape(-1)] = scales.reshape(-1)
        return out

    if decoder == 0:  # bf16
        w["data"] = bf16_bits(g.standard_normal((n, k), dtype=np.float32) * 0.05).view(np.uint8).reshape(n, 2 * k)
    elif decoder == 1:  # f16
        w["data"] = (g.standard_normal((n, k), dtype=np.float32) * 0.05).astype(np.float16).view(np.uint8).reshape(n, 2 * k)
    elif decoder == 2:  # q8_0 blocks
        w["data"] = q8_0_weights(n, k, seed)
    elif decoder in (3, 4, 5, 6):  # nvfp4: UE4M3 scales of 16 values, 0x20 .. 0x47 (2^-3 .. 30)
        codes = g.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
        scales = g.integers(0x20, 0x48, size=(n, k // 16), dtype=np.uint8)
        if decoder == 3:
            w["data"], w["scales"] = codes, scales.reshape(-1)
        elif decoder == 4:
            w["data"], w["scales"] = codes, atoms(scales, k // 16)
        elif decoder == 5:
            w["data"] = np.concatenate([codes, scales], axis=1)
        else:  # GGML's blocks: value j of a 16-value sub-block in byte j % 8, low nibble below 8
            v = np.stack([codes & 15, codes >> 4], axis=-1).reshape(n, k // 64, 4, 16)  # codes in value order
            packed = (v[..., :8] | (v[..., 8:] << 4)).astype(np.uint8).reshape(n, k // 64, 32)
            w["data"] = np.concatenate([scales.reshape(n, k // 64, 4), packed], axis=-1).reshape(n, k // 64 * 36)
            w["plain"] = (codes, scales)  # the same values as nvfp4.split holds them
    elif decoder in (7, 8):  # mxfp8: E8M0 scales of 32 values
        codes = g.integers(0, 256, size=(n, k), dtype=np.uint8)
        codes[(codes & 0x7F) == 0x7F] = 0x38  # no NaN codes
        scales = g.integers(118, 126, size=(n, k // 32), dtype=np.uint8)
        w["data"], w["scales"] = codes, scales.reshape(-1) if decoder == 7 else atoms(scales, k // 32)
    elif decoder in (9, 10):  # mxfp4
        codes = g.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
        scales = g.integers(118, 126, size=(n, k // 32), dtype=np.uint8)
        w["data"], w["scales"] = codes, scales.reshape(-1) if decoder == 9 else atoms(scales, k // 32)
    elif decoder == 11:
        raise ValueError("affine weights come from affine_weight()")
    else:
        raise ValueError("no synthetic weight for this decoder")
    w["data"] = np.ascontiguousarray(w["data"])
    if tensor_scales:
        w["tensor_scale"] = g.uniform(0.5, 2.0, size=tensor_scales).astype(np.float32)
        w["rows_per_scale"] = n // tensor_scales
    return w


def affine_weight(n, k, seed, bits=4, group=64, scale="f16", zero_point=False, tensor_scales=0):
    """An MLX-style affine weight as the reference's affine.split decoder reads it (src/kernels/decode/operand.h:
    74-97): unsigned codes of `bits` bits packed little-endian along the row, a scale and a bias (or, with
    `zero_point`, a packed zero point) a group of `group` values; scales F16, BF16 or F32."""
    g = rng(seed)
    groups = k // group
    codes = g.integers(0, 1 << bits, size=(n, k), dtype=np.uint8)
    data = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8) if bits == 4 else codes
    sc = g.uniform(0.002, 0.01, size=(n, groups)).astype(np.float32)
    bias = (-sc * (1 << (bits - 1)) + g.uniform(-0.003, 0.003, size=(n, groups))).astype(np.float32)
    kind = {"f16": 1, "bf16": 2, "f32": 3}[scale]

    def pack(a):
        if kind == 3:
            return np.ascontiguousarray(a).view(np.uint8).reshape(n, -1)
        if kind == 2:
            return bf16_bits(a).view(np.uint8).reshape(n, -1)
        return a.astype(np.float16).view(np.uint8).reshape(n, -1)

    w = {"k": k, "data": np.ascontiguousarray(data), "scales": pack(sc), "group": group, "bits": bits,
         "scale_type": kind | (0x80 if zero_point else 0), "scale_row_bytes": groups * (4 if kind == 3 else 2)}
    if zero_point:
        zeros = g.integers(0, 1 << bits, size=(n, groups), dtype=np.uint8)
        if bits == 4:
            padded = np.zeros((n, (groups + 1) // 2 * 2), dtype=np.uint8)
            padded[:, :groups] = zeros
            zeros = (padded[:, 0::2] | (padded[:, 1::2] << 4)).astype(np.uint8)
        w["biases"] = np.ascontiguousarray(zeros)
    else:
        w["biases"] = pack(bias)
    if tensor_scales:
        w["tensor_scale"] = g.uniform(0.5, 2.0, size=tensor_scales).astype(np.float32)
        w["rows_per_scale"] = n // tensor_scales
    return w
