"""ctypes binding of the CPU oracle (oracle/oracle.c): TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module. The shipped package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

TYPE_Q4_0 = 2
TYPE_Q4_1 = 3
TYPE_Q5_0 = 6
TYPE_Q5_1 = 7
TYPE_Q8_0 = 8
TYPE_Q4_K = 12
TYPE_MXFP4 = 39
TYPE_IQ4_NL = 20
TYPE_Q5_K = 13
TYPE_Q6_K = 14
GLU_NONE, GLU_SWIGLU, GLU_SWIGLU_CLAMP, GLU_GEGLU = 0, 1, 2, 3
CB_3INST, CB_MCG, CB_MUL1 = 0, 1, 2
Q8_DEVICE, Q8_GGML_CPU = 0, 1


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


lib = _load()


class VecQDesc(C.Structure):
    _fields_ = [
        ("w", C.c_void_p), ("g", C.c_void_p), ("y", C.c_void_p), ("ids", C.c_void_p),
        ("dst", C.c_void_p),
        ("ncols_x", C.c_int), ("nrows", C.c_int), ("stride_row", C.c_int),
        ("stride_expert", C.c_int), ("y_token", C.c_int), ("y_slot", C.c_int),
        ("ids_stride", C.c_int), ("used", C.c_int), ("tokens", C.c_int),
        ("dst_token", C.c_int), ("dst_slot", C.c_int), ("glu", C.c_int), ("limit", C.c_float),
    ]


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _sig(name, res, *args):
    f = getattr(lib, name)
    f.restype = res
    f.argtypes = list(args)
    return f


_i64, _u64, _vp, _int = C.c_int64, C.c_uint64, C.c_void_p, C.c_int
_sig("orc_attention_quant", None, _int, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _i64, C.c_float,
     C.c_float, _int, _vp, _int)
_sig("orc_f16_to_f32", C.c_float, C.c_uint16)
_sig("orc_f32_to_f16", C.c_uint16, C.c_float)
_sig("orc_bf16_to_f32", C.c_float, C.c_uint16)
_sig("orc_f32_to_bf16", C.c_uint16, C.c_float)
_sig("orc_e4m3_to_f32", C.c_float, C.c_uint8)
_sig("orc_e8m0_to_f32", C.c_float, C.c_uint8)
_sig("orc_e2m1_to_f32", C.c_float, C.c_uint8)
_sig("orc_f32_to_e4m3", C.c_uint8, C.c_float)
_sig("orc_q8_1_quantize_row", None, _vp, _i64, _i64, _vp, _int)
_sig("orc_q8_1_decode_row", None, _vp, _i64, _vp)
_sig("orc_kv_quantize_row", None, _int, _vp, _i64, _vp)
_sig("orc_q4_k_scale_min", None, _vp, _int, _vp, _vp)
_sig("orc_decode_row", None, _int, _vp, _i64, _vp)
_sig("orc_block_sums", None, _int, _vp, _vp, _vp)
_sig("orc_block_product", C.c_double, _int, _vp, _vp)
_sig("orc_glu", C.c_double, _int, C.c_double, C.c_double, C.c_double)
_sig("orc_vecq", _int, _int, C.POINTER(VecQDesc), _int, _int)
_sig("orc_vecq_block_sums", None, _int, _vp, _vp, _int, _int, _int, _vp)
_sig("orc_mxfp8_scale_code", C.c_uint32, C.c_float)
_sig("orc_mxfp8_inverse_scale", C.c_float, C.c_uint32)
_sig("orc_scale_atom_offset", _u64, _u64, _u64, _u64)
_sig("orc_mxfp8_quantize", None, _vp, _i64, _i64, _i64, _vp, _vp)
_sig("orc_mxfp8_swizzle", None, _vp, _i64, _i64, _vp)
_sig("orc_mxfp8_dot", C.c_double, _vp, _vp, _i64, _vp, _vp, _i64, _i64)
_sig("orc_mxfp8_gemm", None, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _int)
_sig("orc_mxfp8_gemv", None, _vp, _vp, _i64, _i64, _vp, _i64, _vp)
_sig("orc_route", None, _vp, _i64, _i64, _i64, _int, C.c_float, _vp, _vp)
_sig("orc_expert_sort", _int, _vp, _i64, _i64, _vp, _vp)
_sig("orc_expert_reduce", None, _vp, _vp, _i64, _i64, _i64, _vp)
_sig("orc_exl3_codebook", C.c_uint16, _int, C.c_uint16)
_sig("orc_exl3_state", C.c_uint16, _vp, C.c_uint32, C.c_uint32)
_sig("orc_exl3_placement", None, _vp)
_sig("orc_exl3_rotated", None, _vp, _i64, _i64, _int, _int, _i64, _i64, _vp)
_sig("orc_exl3_rows", None, _vp, _vp, _vp, _i64, _i64, _int, _int, _i64, _i64, _vp)
_sig("orc_exl3_linear", None, _vp, _vp, _vp, _i64, _i64, _int, _int, _vp, _i64, _vp, _int)
_sig("orc_exl3_input", None, _vp, _i64, _vp, _i64, _vp)
_sig("orc_exl3_product", None, _vp, _vp, _i64, _i64, _int, _int, _vp, _i64, _vp, _int)
_sig("orc_max_threads", _int)


def max_threads():
    return int(lib.orc_max_threads())


def block_bytes(t):
    return {TYPE_Q4_0: 18, TYPE_Q4_1: 20, TYPE_Q5_0: 22, TYPE_Q5_1: 24, TYPE_Q8_0: 34, TYPE_Q4_K: 144, TYPE_MXFP4: 17, TYPE_IQ4_NL: 18, TYPE_Q5_K: 176, TYPE_Q6_K: 210}[t]


def block_elements(t):
    return 256 if t in (TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K) else 32


def padded_k(k):
    return (k + 511) // 512 * 512


def q8_1_quantize(x, flavor=Q8_DEVICE):
    """float32 [rows, k] -> uint8 [rows, padded_k/32*36]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = x.shape
    pk = padded_k(k)
    out = np.zeros((rows, pk // 32 * 36), dtype=np.uint8)
    for r in range(rows):
        lib.orc_q8_1_quantize_row(_p(x[r]), k, pk, _p(out[r]), flavor)
    return out


def kv_quantize(t, x):
    """float32 [rows, k] -> uint8 [rows, k/32*bytes] Q8_0 or Q4_0 blocks, GGML's reference
    quantizers (the KV cache store's arithmetic)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = x.shape
    out = np.zeros((rows, k // 32 * block_bytes(t)), dtype=np.uint8)
    for r in range(rows):
        lib.orc_kv_quantize_row(t, _p(x[r]), k, _p(out[r]))
    return out


def attention_quant(t, q, k, v, d, heads, kv_heads, rows, cells, scale, *, mask=None, sinks=None, softcap=0.0,
                    cell_stride=None, head_stride=None, q8_1_q=False, threads=1):
    """Attention over a Q8_0 / Q4_0 KV cache decoded exactly (the reference executor's kAttention in double).
    q float32 [heads, rows, d]; k, v uint8 with (cell, kv head)'s row at cell * cell_stride + head * head_stride
    (default: a cell's heads together); mask float16 [>= rows, cells]; returns float32 [rows, heads, d]."""
    row_bytes = d // 32 * block_bytes(t)
    head_stride = row_bytes if head_stride is None else head_stride
    cell_stride = row_bytes * kv_heads if cell_stride is None else cell_stride
    q = np.ascontiguousarray(q, dtype=np.float32)
    out = np.zeros((rows, heads, d), dtype=np.float32)
    mask_bits = None if mask is None else np.ascontiguousarray(mask).view(np.uint16)
    if mask_bits is not None:
        assert mask_bits.shape[1] == cells and mask_bits.shape[0] >= rows
    sk = None if sinks is None else np.ascontiguousarray(sinks, dtype=np.float32)
    lib.orc_attention_quant(t, _p(q), _p(k), _p(v), cell_stride, head_stride, _p(mask_bits) if mask_bits is not None else None,
                            _p(sk) if sk is not None else None, d, heads, kv_heads, rows, cells, scale, softcap,
                            int(q8_1_q), _p(out), threads)
    return out


def rope_neox(x, pos, n_dims, theta_scale, freq_scale=1.0, ext_factor=0.0, attn_factor=1.0, corr_dims=(0.0, 0.0),
              freq_factors=None):
    """float32 x [tokens, heads, head_dim] -> the forward NEOX RoPE's float32 values, as the reference's CPU executor
    forms them (src/kernels/reference/exec.cc:1343-1484: the mode's default case, offset 0, not the llama3 form): the
    angle's steps each rounded to F32 (theta_scale^pair from FP64, times the position, over the frequency factor,
    times the scale; YaRN's ramp between the correction dims), cosine and sine in FP64 times the magnitude, the
    rotation in FP64, the result rounded to F32. Channels from n_dims on pass through. numpy, not C: test
    infrastructure like the rest of this package."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    tokens, heads, head_dim = x.shape
    half = n_dims // 2
    f32 = np.float32
    pair = np.arange(half)
    power = np.power(np.float64(f32(theta_scale)), pair.astype(np.float64)).astype(np.float32)      # exec.cc:1449-1450
    out = x.copy()
    magnitude = f32(attn_factor)
    if ext_factor > 0.0:
        magnitude = f32(magnitude * f32(f32(1.0) + f32(f32(0.1) * f32(np.log(f32(f32(1.0) / f32(freq_scale)))))))
    for t in range(tokens):
        extrap = (f32(pos[t]) * power).astype(np.float32)
        if freq_factors is not None:
            extrap = (extrap / np.asarray(freq_factors, dtype=np.float32)[:half]).astype(np.float32)
        interp = (f32(freq_scale) * extrap).astype(np.float32)
        theta = interp
        if ext_factor > 0.0:
            y = ((pair.astype(np.float32) - f32(corr_dims[0])) / max(f32(0.001), f32(f32(corr_dims[1]) - f32(corr_dims[0])))).astype(np.float32)
            ramp = ((f32(1.0) - np.minimum(f32(1.0), np.maximum(f32(0.0), y))) * f32(ext_factor)).astype(np.float32)
            kept = (interp * (f32(1.0) - ramp)).astype(np.float32)
            mixed = (extrap * ramp).astype(np.float32)
            theta = (kept + mixed).astype(np.float32)
        c = np.cos(theta.astype(np.float64)) * np.float64(magnitude)
        sn = np.sin(theta.astype(np.float64)) * np.float64(magnitude)
        a = x[t, :, :half].astype(np.float64)
        b = x[t, :, half:n_dims].astype(np.float64)
        out[t, :, :half] = (a * c - b * sn).astype(np.float32)
        out[t, :, half:n_dims] = (a * sn + b * c).astype(np.float32)
    return out


def q8_1_decode(blocks, k):
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    y = np.zeros(k, dtype=np.float32)
    lib.orc_q8_1_decode_row(_p(blocks), k, _p(y))
    return y


def decode_rows(t, w, k):
    """uint8 [rows, k/qk*bs] -> float32 [rows, k]."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    out = np.zeros((w.shape[0], k), dtype=np.float32)
    for r in range(w.shape[0]):
        lib.orc_decode_row(t, _p(w[r]), k, _p(out[r]))
    return out


def vecq(t, w, q8, k, nrows, *, gate=None, ids=None, tokens=1, used=1, stride_row=None,
         stride_expert=0, y_token=None, y_slot=0, glu=GLU_NONE, limit=0.0, experts=0, threads=1):
    """The llmp.vecq product on the CPU. Returns float32 [tokens, used, nrows]."""
    qk = block_elements(t)
    w = np.ascontiguousarray(w, dtype=np.uint8)
    q8 = np.ascontiguousarray(q8, dtype=np.uint8)
    gate = None if gate is None else np.ascontiguousarray(gate, dtype=np.uint8)
    ids = None if ids is None else np.ascontiguousarray(ids, dtype=np.int32)
    dst = np.zeros((tokens, used, nrows), dtype=np.float32)
    d = VecQDesc()
    d.w, d.g, d.y, d.ids, d.dst = _p(w), _p(gate), _p(q8), _p(ids), _p(dst)
    d.ncols_x, d.nrows = k, nrows
    d.stride_row = k // qk if stride_row is None else stride_row
    d.stride_expert = stride_expert
    d.y_token = padded_k(k) // 32 if y_token is None else y_token
    d.y_slot = y_slot
    d.ids_stride = used
    d.used, d.tokens = used, tokens
    d.dst_token, d.dst_slot = used * nrows, nrows
    d.glu, d.limit = glu, limit
    rc = lib.orc_vecq(t, C.byref(d), experts, threads)
    if rc != 0:
        raise IndexError("expert id outside the table")
    return dst


def vecq_block_sums(t, w, q8, k, nrows):
    qk = block_elements(t)
    per = 16 if t in (TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K) else 1
    w = np.ascontiguousarray(w, dtype=np.uint8)
    q8 = np.ascontiguousarray(q8, dtype=np.uint8)
    out = np.zeros((nrows, k // qk, per), dtype=np.int32)
    lib.orc_vecq_block_sums(t, _p(w), _p(q8), k, nrows, k // qk, _p(out))
    return out


def glu(kind, gate, up, limit=0.0):
    return lib.orc_glu(kind, float(gate), float(up), float(limit))


def mxfp8_scale_bytes(rows, k):
    assert k % 128 == 0, "scale atoms hold four 32-value blocks: k must be a multiple of 128"
    return (rows + 127) // 128 * 128 * (k // 32)


def mxfp8_quantize(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = x.shape
    codes = np.zeros((rows, k), dtype=np.uint8)
    scales = np.zeros(mxfp8_scale_bytes(rows, k), dtype=np.uint8)
    lib.orc_mxfp8_quantize(_p(x), k, k, rows, _p(codes), _p(scales))
    return codes, scales


def mxfp8_swizzle(scales):
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    n, blocks = scales.shape
    out = np.zeros(mxfp8_scale_bytes(n, blocks * 32), dtype=np.uint8)
    lib.orc_mxfp8_swizzle(_p(scales), n, blocks, _p(out))
    return out


def mxfp8_dot(a_codes, a_scales, i, b_codes, b_scales, j):
    k = a_codes.shape[1]
    return lib.orc_mxfp8_dot(_p(a_codes), _p(a_scales), i, _p(b_codes), _p(b_scales), j, k)


def mxfp8_gemm(a_codes, a_scales, b_codes, b_scales, threads=1):
    m, k = a_codes.shape
    n = b_codes.shape[0]
    d = np.zeros((m, n), dtype=np.float32)
    lib.orc_mxfp8_gemm(_p(a_codes), _p(a_scales), _p(b_codes), _p(b_scales), m, n, k, _p(d), threads)
    return d


def mxfp8_gemv(codes, scales, x):
    n, k = codes.shape
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros((x.shape[0], n), dtype=np.float32)
    lib.orc_mxfp8_gemv(_p(codes), _p(np.ascontiguousarray(scales)), n, k, _p(x), x.shape[0], _p(y))
    return y


def nvfp4_values(codes, scales, rows, k, scale_row0=0):
    """The values of `rows` rows of NVFP4: E2M1 codes (uint8 [rows, k / 2], element 2i in byte i's low nibble) times
    the UE4M3 scale of their 16-element block, read from the 128-row by 4-scale atoms of
    src/kernels/ggml/moe_cutlass.h:42-46 of the reference (orc_scale_atom_offset) at row scale_row0 + r."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(rows, k // 2)
    e2m1 = np.array([lib.orc_e2m1_to_f32(c) for c in range(16)], dtype=np.float64)
    ue4m3 = np.array([lib.orc_ue4m3_to_f32(c) for c in range(256)], dtype=np.float64)
    values = np.empty((rows, k), dtype=np.float64)
    values[:, 0::2] = e2m1[codes & 15]
    values[:, 1::2] = e2m1[codes >> 4]
    blocks = k // 16
    at = np.array([[lib.orc_scale_atom_offset(scale_row0 + r, b, blocks) for b in range(blocks)] for r in range(rows)],
                  dtype=np.int64).reshape(rows, blocks)
    return values * np.repeat(ue4m3[np.asarray(scales, dtype=np.uint8)[at]], 16, axis=1)


def grouped_nvfp4_gemm(a_codes, a_scales, offsets, sf_rows, b_codes, b_scales, n, k):
    """llmp.moe.gemm's definition (src/kernels/ggml/moe_cutlass.h:12-27 of the reference): group e multiplies rows
    offsets[e] .. offsets[e + 1] of A (scales in a block of rows from sf_rows[e]) by expert e's n rows; b_codes[e]
    and b_scales[e] are that expert's codes and atoms. Float64 sums of the decoded values: [rows, n]."""
    rows = int(offsets[-1])
    out = np.zeros((rows, n), dtype=np.float64)
    for e in range(len(offsets) - 1):
        first, count = int(offsets[e]), int(offsets[e + 1] - offsets[e])
        if count == 0:
            continue
        a = nvfp4_values(np.asarray(a_codes)[first:first + count], a_scales, count, k, int(sf_rows[e]))
        b = nvfp4_values(b_codes[e], b_scales[e], n, k)
        out[first:first + count] = a @ b.T
    return out


def route(logits, used, normalize=True, scale=1.0):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tokens, experts = logits.shape
    ids = np.zeros((tokens, used), dtype=np.int32)
    w = np.zeros((tokens, used), dtype=np.float32)
    lib.orc_route(_p(logits), experts, used, tokens, int(normalize), scale, _p(ids), _p(w))
    return ids, w


def expert_sort(ids, experts):
    ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
    order = np.zeros(ids.size, dtype=np.int32)
    offsets = np.zeros(experts + 1, dtype=np.int32)
    if lib.orc_expert_sort(_p(ids), ids.size, experts, _p(order), _p(offsets)) != 0:
        raise IndexError("expert id outside the table")
    return order, offsets


def expert_reduce(x, w):
    """x float32 [tokens, used, width], w [tokens, used] -> [tokens, width]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    tokens, used, width = x.shape
    out = np.zeros((tokens, width), dtype=np.float32)
    lib.orc_expert_reduce(_p(x), _p(w), width, used, tokens, _p(out))
    return out


def exl3_rotated(trellis, k, n, bits, codebook, first=0, count=None):
    count = n if count is None else count
    out = np.zeros((k, count), dtype=np.uint16)
    lib.orc_exl3_rotated(_p(trellis), k, n, bits, codebook, first, count, _p(out))
    return out


def exl3_rows(trellis, suh, svh, k, n, bits, codebook, first=0, count=None):
    count = n if count is None else count
    out = np.zeros((count, k), dtype=np.float32)
    lib.orc_exl3_rows(_p(trellis), _p(suh), _p(svh), k, n, bits, codebook, first, count, _p(out))
    return out


def _half_bits(x):
    """F16 values as their bits: a float16 array is reinterpreted, never converted."""
    x = np.asarray(x)
    if x.dtype == np.float16:
        x = x.view(np.uint16)
    if x.dtype != np.uint16:
        raise TypeError(f"F16 bits expected, not {x.dtype}")
    return np.ascontiguousarray(x)


def exl3_linear(trellis, suh, svh, k, n, bits, codebook, x, threads=1):
    x = _half_bits(x)
    m = x.shape[0]
    y = np.zeros((m, n), dtype=np.float32)
    lib.orc_exl3_linear(_p(trellis), _p(suh), _p(svh), k, n, bits, codebook, _p(x), m, _p(y), threads)
    return y


def exl3_input(suh, k, x):
    x = _half_bits(x)
    xh = np.zeros_like(x)
    lib.orc_exl3_input(_p(suh), k, _p(x), x.shape[0], _p(xh))
    return xh


def exl3_product(trellis, svh, k, n, bits, codebook, xh, threads=1):
    xh = _half_bits(xh)
    m = xh.shape[0]
    y = np.zeros((m, n), dtype=np.float32)
    lib.orc_exl3_product(_p(trellis), _p(svh), k, n, bits, codebook, _p(xh), m, _p(y), threads)
    return y


# ---- decode products (src/kernels/decode/products.h of the reference)

DECODERS = ("bf16.dense", "f16.dense", "q8_0.blocks", "nvfp4.split", "nvfp4.atoms", "nvfp4.interleaved",
            "nvfp4.ggml_blocks", "mxfp8.split", "mxfp8.atoms", "mxfp4.split", "mxfp4.atoms", "affine.split")


class DecodeOperand(C.Structure):
    """src/kernels/decode/operand.h:74-97 of the reference, field for field."""
    _fields_ = [("data", C.c_void_p), ("scales", C.c_void_p), ("tensor_scale", C.c_void_p), ("biases", C.c_void_p),
                ("k", C.c_uint32), ("rows", C.c_uint32), ("rows_per_scale", C.c_uint32), ("pad", C.c_uint32),
                ("row_bytes", C.c_uint64), ("scale_row_bytes", C.c_uint32), ("group", C.c_uint16),
                ("bits", C.c_uint8), ("scale_type", C.c_uint8)]


_sig("orc_ue4m3_to_f32", C.c_float, C.c_uint8)
_sig("orc_decode_value", C.c_float, _int, C.POINTER(DecodeOperand), _u64, _u64)
_sig("orc_decode_vector", _int, _int, C.POINTER(DecodeOperand), _u64, _u64, _vp, _u64, _u64, _vp, _u64, _int)


def decode_operand(weight):
    """`weight`: a dict with data (uint8 [rows, row_bytes]), k, and where the decoder has them scales (uint8,
    flat) and tensor_scale (float32 [rows / rows_per_scale]). The arrays must outlive the operand."""
    op = DecodeOperand()
    data = weight["data"]
    op.data, op.scales, op.tensor_scale = _p(data), _p(weight.get("scales")), _p(weight.get("tensor_scale"))
    op.k, op.rows = weight["k"], data.shape[0]
    op.rows_per_scale = weight.get("rows_per_scale", data.shape[0])
    op.row_bytes = data.shape[1]
    if "group" in weight:  # the affine encoding
        op.biases = _p(weight.get("biases"))
        op.group, op.bits, op.scale_type = weight["group"], weight["bits"], weight["scale_type"]
        op.scale_row_bytes = weight["scale_row_bytes"]
    return op


def decode_rows_of(decoder, weight):
    """Every value of the weight, before the tensor scale: float32 [rows, k]."""
    op = decode_operand(weight)
    rows, k = weight["data"].shape[0], weight["k"]
    out = np.empty((rows, k), dtype=np.float32)
    for r in range(rows):
        for j in range(k):
            out[r, j] = lib.orc_decode_value(decoder, C.byref(op), r, j)
    return out


def decode_vector(decoder, weight, x, first=0, outputs=None, threads=1):
    """llmp.decode.vector on the CPU: float32 x [rows, k] -> [rows, outputs]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    op = decode_operand(weight)
    outputs = weight["data"].shape[0] - first if outputs is None else outputs
    y = np.zeros((x.shape[0], outputs), dtype=np.float32)
    rc = lib.orc_decode_vector(decoder, C.byref(op), first, outputs, _p(x), x.shape[0], x.shape[1], _p(y), outputs,
                               threads)
    if rc != 0:
        raise ValueError("no such decoder")
    return y


_sig("orc_decode_vector_glu", _int, _int, C.POINTER(DecodeOperand), _u64, _int, C.POINTER(DecodeOperand), _u64, _u64, _int,
     C.c_float, _vp, _u64, _u64, _vp, _u64, _int)


def decode_vector_glu(decoder, gate, up, x, glu, limit=0.0, gate_first=0, up_first=0, outputs=None, threads=1, up_decoder=None):
    """llmp.decode.vector_glu on the CPU; `glu` is the reference's ir::GluKind (0 SwiGLU, 1 GeGLU erf, 2 GeGLU
    tanh, 3 SwiGLU with a clamp)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    g, u = decode_operand(gate), decode_operand(up)
    outputs = gate["data"].shape[0] - gate_first if outputs is None else outputs
    y = np.zeros((x.shape[0], outputs), dtype=np.float32)
    rc = lib.orc_decode_vector_glu(decoder, C.byref(g), gate_first, decoder if up_decoder is None else up_decoder, C.byref(u), up_first, outputs, glu, limit, _p(x),
                                   x.shape[0], x.shape[1], _p(y), outputs, threads)
    if rc != 0:
        raise ValueError("no such product")
    return y


_sig("orc_decode_grouped", _int, _int, C.POINTER(DecodeOperand), _u64, C.c_uint32, C.c_uint32, _u64, _u64, _vp, _vp, _vp,
     _u64, _vp, _u64, _u64, _vp, _u64, _u64)


def decode_grouped(decoder, experts, k, n, offsets, pair_rows, x, y, pair_out=None, first=0, outputs=None):
    """llmp.decode.grouped on the CPU: `experts` a list of weights, `y` (float32 [y_rows, outputs]) updated in place."""
    ops_ = (DecodeOperand * len(experts))(*[decode_operand(w) for w in experts])
    x = np.ascontiguousarray(x, dtype=np.float32)
    outputs = n - first if outputs is None else outputs
    offsets = np.ascontiguousarray(offsets, dtype=np.int32)
    pair_rows = np.ascontiguousarray(pair_rows, dtype=np.int32)
    pair_out = None if pair_out is None else np.ascontiguousarray(pair_out, dtype=np.int32)
    rc = lib.orc_decode_grouped(decoder, ops_, len(experts), k, n, first, outputs, _p(offsets), _p(pair_rows), _p(pair_out),
                                len(pair_rows), _p(x), x.shape[0], x.shape[1], _p(y), y.shape[0], y.shape[1])
    if rc != 0:
        raise ValueError("no such decoder")
    return y


_sig("orc_decode_matrix", _int, _int, C.POINTER(DecodeOperand), _u64, _u64, _vp, _u64, _u64, _vp, _u64, _int)


def decode_matrix(decoder, weight, x, first=0, outputs=None, threads=1):
    """llmp.decode.matrix (the tensor-core path's rounding) on the CPU: float32 x [rows, k] -> [rows, outputs]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    op = decode_operand(weight)
    outputs = weight["data"].shape[0] - first if outputs is None else outputs
    y = np.zeros((x.shape[0], outputs), dtype=np.float32)
    rc = lib.orc_decode_matrix(decoder, C.byref(op), first, outputs, _p(x), x.shape[0], x.shape[1], _p(y), outputs, threads)
    if rc != 0:
        raise ValueError("no such decoder")
    return y
