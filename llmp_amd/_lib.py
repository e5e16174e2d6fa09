"""ctypes binding of lib/libllmp_hip.so (include/llmp_hip.h).

There is no fallback: if the library is missing, `load()` raises. torch is
imported first so that the process holds one HIP runtime.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "lib", "libllmp_hip.so")

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
X_F32, X_BF16, X_F16 = 0, 1, 2


class VecQDesc(C.Structure):
    """llmp_vecq_desc: src/kernels/ggml/vecq.h:22-41 of the reference."""
    _fields_ = [
        ("w", C.c_void_p), ("g", C.c_void_p), ("y", C.c_void_p), ("ids", C.c_void_p),
        ("dst", C.c_void_p),
        ("ncols_x", C.c_int), ("nrows", C.c_int), ("stride_row", C.c_int),
        ("stride_expert", C.c_int), ("y_token", C.c_int), ("y_slot", C.c_int),
        ("ids_stride", C.c_int), ("used", C.c_int), ("tokens", C.c_int),
        ("dst_token", C.c_int), ("dst_slot", C.c_int), ("glu", C.c_int), ("limit", C.c_float),
    ]


class Mxfp8Gemm(C.Structure):
    """llmp_mxfp8_gemm: mxfp8::Gemm of src/kernels/ggml/mxfp8_cutlass.h:56-70 of the reference."""
    _fields_ = [("m", C.c_int), ("n", C.c_int), ("k", C.c_int), ("a", C.c_void_p), ("a_scales", C.c_void_p),
                ("b", C.c_void_p), ("b_scales", C.c_void_p), ("d", C.c_void_p), ("bf16", C.c_uint8),
                ("scratch", C.c_void_p)]


class GroupedGemm(C.Structure):
    """llmp_grouped_gemm: moe::GroupedGemm of src/kernels/ggml/moe_cutlass.h:48-64 of the reference."""
    _fields_ = [("groups", C.c_int), ("n", C.c_int), ("k", C.c_int), ("offsets", C.c_void_p), ("sf_rows", C.c_void_p),
                ("a", C.c_void_p), ("a_scales", C.c_void_p), ("weights", C.c_void_p), ("expert_stride", C.c_uint64),
                ("codes_offset", C.c_uint64), ("scales_offset", C.c_uint64), ("d", C.c_void_p), ("scratch", C.c_void_p)]


class Exl3Weights(C.Structure):
    """llmp_exl3_weights: src/kernels/exl3/validate.h:84-96 of the reference, plus the codebook."""
    _fields_ = [("trellis", C.c_void_p), ("suh", C.c_void_p), ("svh", C.c_void_p), ("k", C.c_int), ("n", C.c_int),
                ("bits", C.c_int), ("codebook", C.c_int)]


class Exl3Linear(C.Structure):
    """llmp_exl3_linear: LinearOperands of src/kernels/exl3/validate.h:118-131 of the reference."""
    _fields_ = [("weights", Exl3Weights), ("x", C.c_void_p), ("a_had", C.c_void_p), ("y", C.c_void_p),
                ("f32", C.c_int), ("m", C.c_int)]


class Exl3MultiLinear(C.Structure):
    """llmp_exl3_multi_linear: MultiLinearOperands of src/kernels/exl3/validate.h:160-172 of the reference,
    without its pointer tables."""
    _fields_ = [("first", Exl3Weights), ("second", Exl3Weights), ("x", C.c_void_p), ("a_had", C.c_void_p),
                ("y", C.c_void_p), ("f32", C.c_int), ("m", C.c_int)]


class DecodeOperand(C.Structure):
    """llmp_decode_operand: Operand of src/kernels/decode/operand.h:74-97 of the reference."""
    _fields_ = [("data", C.c_void_p), ("scales", C.c_void_p), ("tensor_scale", C.c_void_p), ("biases", C.c_void_p),
                ("k", C.c_uint32), ("rows", C.c_uint32), ("rows_per_scale", C.c_uint32), ("pad", C.c_uint32),
                ("row_bytes", C.c_uint64), ("scale_row_bytes", C.c_uint32), ("group", C.c_uint16),
                ("bits", C.c_uint8), ("scale_type", C.c_uint8)]


class SetRowsStore(C.Structure):
    """llmp_set_rows_store: one member of llmp.set_rows.grouped_quant (src/kernels/ggml/kv_quant.h:172-178 of the
    reference)."""
    _fields_ = [("type", C.c_int), ("index_bytes", C.c_int), ("x", C.c_void_p), ("x_stride", C.c_int64),
                ("ids", C.c_void_p), ("destination", C.c_void_p), ("row_bytes", C.c_int64), ("k", C.c_int64),
                ("rows", C.c_int64), ("cells", C.c_int64)]


class MoeToken(C.Structure):
    """llmp_moe_token: one token's routed-expert FFN layer in one launch."""
    _fields_ = [("logits", C.c_void_p), ("x", C.c_void_p), ("gate_up", C.c_void_p), ("down", C.c_void_p), ("out", C.c_void_p),
                ("ids", C.c_void_p), ("weights", C.c_void_p), ("h", C.c_void_p), ("sync", C.c_void_p),
                ("gate_up_stride", C.c_int64), ("down_stride", C.c_int64), ("type", C.c_int32), ("x_type", C.c_int32),
                ("experts", C.c_int32), ("used", C.c_int32), ("hidden", C.c_int32), ("ffn", C.c_int32), ("glu", C.c_int32),
                ("normalize", C.c_int32), ("limit", C.c_float), ("route_scale", C.c_float)]


class AttnVecQuant(C.Structure):
    """llmp_attn_vec_quant: the operands of ggml.flash_attn_ext.vec_q8_0 / vec_q4_0 (src/kernels/ggml/kv_quant.h:146-160
    of the reference)."""
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("mask", C.c_void_p), ("sinks", C.c_void_p),
                ("out", C.c_void_p), ("q_row_stride", C.c_int64), ("q_head_stride", C.c_int64),
                ("k_cell_stride", C.c_int64), ("k_head_stride", C.c_int64), ("v_cell_stride", C.c_int64),
                ("v_head_stride", C.c_int64), ("mask_row_stride", C.c_int64), ("type", C.c_int32),
                ("head_dim", C.c_int32), ("heads", C.c_int32), ("kv_heads", C.c_int32), ("rows", C.c_int32),
                ("cells", C.c_int32), ("scale", C.c_float), ("softcap", C.c_float)]


class RopeStore(C.Structure):
    """llmp_rope_store: RopeStore of src/kernels/ggml/kv_quant_rope.cu:55-71 of the reference."""
    _fields_ = [("type", C.c_int), ("heads", C.c_int), ("head_dim", C.c_int), ("n_dims", C.c_int), ("x", C.c_void_p),
                ("x_head_stride", C.c_int64), ("x_token_stride", C.c_int64), ("pos", C.c_void_p),
                ("freq_factors", C.c_void_p), ("ids", C.c_void_p), ("destination", C.c_void_p),
                ("row_bytes", C.c_int64), ("tokens", C.c_int64), ("freq_scale", C.c_float), ("ext_factor", C.c_float),
                ("attn_factor", C.c_float), ("theta_scale", C.c_float), ("corr_dims", C.c_float * 2)]


class VecQSource(C.Structure):
    _fields_ = [("x", C.c_void_p), ("x_type", C.c_int), ("x_token", C.c_int64),
                ("x_slot", C.c_int64)]


_i64, _vp, _int = C.c_int64, C.c_void_p, C.c_int

# name -> (restype, argtypes): every symbol include/llmp_hip.h declares.
SYMBOLS = {
    "llmp_hip_last_error": (C.c_char_p, []),
    "llmp_hip_compute_units": (_int, []),
    "llmp_hip_stream_read_sink": (C.c_size_t, [_int]),
    "llmp_hip_stream_read": (_int, [_vp, C.c_size_t, _vp, _int, _vp]),
    "llmp_hip_q8_1_quantize": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp]),
    "llmp_hip_vecq": (_int, [_int, C.POINTER(VecQDesc), _int, _vp]),
    "llmp_hip_vecq_variants": (_int, []),
    "llmp_hip_vecq_variant_name": (C.c_char_p, [_int]),
    "llmp_hip_vecq_fused": (_int, [_int, C.POINTER(VecQDesc), C.POINTER(VecQSource), _int, _vp]),
    "llmp_hip_vecq_block_sums": (_int, [_int, C.POINTER(VecQDesc), _int, _vp, _vp]),
    "llmp_hip_vecq_sorted": (_int, [_int, C.POINTER(VecQDesc), _vp, _int, _int, _vp]),
    "llmp_hip_moe_router": (_int, [_vp, _int, _int, _int, _int, C.c_float, _vp, _vp, _vp]),
    "llmp_hip_moe_route_ints": (_i64, [_int, _int, _int]),
    "llmp_hip_moe_route": (_int, [_vp, _int, _int, _int, _int, _vp, _vp]),
    "llmp_hip_q8_1_quantize_rows": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "llmp_hip_moe_combine": (_int, [_vp, _vp, _vp, _int, _int, _int, _vp, _vp]),
    "llmp_hip_set_rows_quant": (_int, [_int, _vp, _i64, _vp, _int, _vp, _i64, _i64, _i64, _i64, _vp]),
    "llmp_hip_set_rows_quant_group": (_int, [_int, C.POINTER(SetRowsStore), _vp]),
    "llmp_hip_rope_set_rows_quant": (_int, [C.POINTER(RopeStore), _vp]),
    "llmp_hip_relayout_q4_k_tiles64": (_int, [_vp, _vp, C.c_int64, C.c_int64, _int, _vp]),
    "llmp_hip_relayout_q8_0_tiles64": (_int, [_vp, _vp, C.c_int64, C.c_int64, _int, _vp]),
    "llmp_hip_moe_token_scratch": (C.c_size_t, [C.POINTER(MoeToken)]),
    "llmp_hip_moe_token": (_int, [C.POINTER(MoeToken), _int, _int, _vp]),
    "llmp_hip_attn_vec_quant_scratch": (C.c_size_t, [C.POINTER(AttnVecQuant), _int]),
    "llmp_hip_attn_vec_quant": (_int, [C.POINTER(AttnVecQuant), _vp, C.c_size_t, _int, _vp]),
    "llmp_hip_mxfp8_quantize": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "llmp_hip_mxfp8_swizzle": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "llmp_hip_mxfp8_gemv": (_int, [_vp, _vp, _i64, _i64, _vp, _int, _vp, _vp]),
    "llmp_hip_mxfp8_gemm_available": (_int, []),
    "llmp_hip_mxfp8_gemm_scratch": (C.c_size_t, [C.POINTER(Mxfp8Gemm), _int]),
    "llmp_hip_mxfp8_gemm_run": (_int, [C.POINTER(Mxfp8Gemm), _int, _vp]),
    "llmp_hip_grouped_gemm_available": (_int, []),
    "llmp_hip_grouped_gemm_scratch": (C.c_size_t, [_int, _int]),
    "llmp_hip_grouped_gemm_run": (_int, [C.POINTER(GroupedGemm), _int, _vp]),
    "llmp_hip_exl3_reconstruct": (_int, [C.POINTER(Exl3Weights), _vp, _int, _int, _vp]),
    "llmp_hip_exl3_reconstruct_fused": (_int, [C.POINTER(Exl3Weights), _vp, _int, _int, _vp]),
    "llmp_hip_exl3_reconstructed_scratch": (C.c_size_t, [C.POINTER(Exl3Weights)]),
    "llmp_hip_exl3_linear_reconstructed": (_int, [C.POINTER(Exl3Linear), _vp, C.c_size_t, _int, _int, _vp]),
    "llmp_hip_exl3_hadamard": (_int, [_vp, _vp, _vp, _int, _int, _int, _int, _vp]),
    "llmp_hip_exl3_linear_scratch": (C.c_size_t, [C.POINTER(Exl3Linear)]),
    "llmp_hip_exl3_linear": (_int, [C.POINTER(Exl3Linear), _vp, C.c_size_t, _vp]),
    "llmp_hip_exl3_linear_static": (_int, [C.POINTER(Exl3Linear), _vp]),
    "llmp_hip_exl3_linear_static_prepare": (_int, [C.POINTER(Exl3Linear)]),
    "llmp_hip_decode_vector": (_int, [_int, C.POINTER(DecodeOperand), C.c_uint64, C.c_uint64, _vp, C.c_uint64,
                                      C.c_uint64, _vp, C.c_uint64, _vp]),
    "llmp_hip_decode_vector_glu": (_int, [_int, C.POINTER(DecodeOperand), C.c_uint64, _int, C.POINTER(DecodeOperand),
                                          C.c_uint64, C.c_uint64, _int, C.c_float, _vp, C.c_uint64, C.c_uint64, _vp,
                                          C.c_uint64, _vp]),
    "llmp_hip_decode_rows": (_int, [_int, C.POINTER(DecodeOperand), _vp, C.c_uint64, _vp, C.c_uint64, _vp, _vp]),
    "llmp_hip_decode_grouped": (_int, [_int, _vp, C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, _vp, _vp, _vp,
                                       C.c_uint64, _vp, C.c_uint64, C.c_uint64, _vp, C.c_uint64, C.c_uint64, C.c_uint64,
                                       _vp]),
    "llmp_hip_decode_matrix": (_int, [_int, C.POINTER(DecodeOperand), C.c_uint64, C.c_uint64, _vp, C.c_uint64,
                                      C.c_uint64, _vp, C.c_uint64, _int, _vp]),
    "llmp_hip_exl3_multi_linear_scratch": (C.c_size_t, [C.POINTER(Exl3MultiLinear)]),
    "llmp_hip_exl3_multi_linear": (_int, [C.POINTER(Exl3MultiLinear), _vp, C.c_size_t, _vp]),
}

_lib = None


class KernelFailure(RuntimeError):
    """A refusal (rejected: nothing was queued) or a fault (unknown: work may be queued):
    src/kernels/common/selected_operation.h:26-35 of the reference."""

    def __init__(self, code, detail):
        super().__init__(f"{'rejected' if code > 0 else 'unknown'} ({code}): {detail}")
        self.code = code
        self.rejected = code > 0
        self.detail = detail


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise ImportError(
            f"{SO_PATH} is not built: run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(make -C llmp_amd/csrc); there is no fallback path")
    import torch  # noqa: F401  (its HIP runtime first)
    lib = C.CDLL(SO_PATH)
    for name, (res, args) in SYMBOLS.items():
        f = getattr(lib, name)
        f.restype = res
        f.argtypes = args
    _lib = lib
    return lib


def check(code):
    if code != 0:
        raise KernelFailure(code, load().llmp_hip_last_error().decode())
