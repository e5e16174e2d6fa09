"""Operator wrappers over the C ABI. Device memory is held in torch tensors
(plumbing only): every call passes raw addresses and the current HIP stream to
lib/libllmp_hip.so and only queues work, as the reference's Run* operators do
(src/kernels/ggml/vecq.cu:1095-1175)."""
import ctypes as C

import torch

from . import _lib
from ._lib import (GLU_GEGLU, GLU_NONE, GLU_SWIGLU, GLU_SWIGLU_CLAMP, TYPE_Q4_K,  # noqa: F401
                   TYPE_Q8_0, X_BF16, X_F16, X_F32, KernelFailure, VecQDesc, VecQSource)

BLOCK_BYTES = {TYPE_Q8_0: 34, TYPE_Q4_K: 144}
BLOCK_ELEMENTS = {TYPE_Q8_0: 32, TYPE_Q4_K: 256}


def padded_k(k):
    """MATRIX_ROW_PADDING: src/kernels/ggml/llmp_ops.cc:2574-2576."""
    return (k + 511) // 512 * 512


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _x_type(x):
    return {torch.float32: X_F32, torch.bfloat16: X_BF16, torch.float16: X_F16}[x.dtype]


def quantize_q8_1(x, out=None):
    """llmp.q8_1: float32 [planes, rows, k] or [rows, k] -> uint8 Q8_1 blocks
    [..., padded_k / 32 * 36]."""
    lib = _lib.load()
    assert x.dtype == torch.float32 and x.is_cuda and x.stride(-1) == 1
    x3 = x if x.dim() == 3 else x.unsqueeze(0)
    planes, rows, k = x3.shape
    pk = padded_k(k)
    if out is None:
        out = torch.empty((planes, rows, pk // 32 * 36), dtype=torch.uint8, device=x.device)
    _lib.check(lib.llmp_hip_q8_1_quantize(_ptr(x3), _ptr(out), k, pk, x3.stride(1), rows, planes,
                                          x3.stride(0), _stream()))
    return out if x.dim() == 3 else out.view(rows, -1)


def _desc(t, w, k, nrows, *, gate, q8, ids, tokens, used, stride_row, stride_expert, y_token,
          y_slot, glu, limit, out):
    d = VecQDesc()
    d.w, d.g, d.y, d.ids, d.dst = (w.data_ptr(), gate.data_ptr() if gate is not None else None,
                                   q8.data_ptr() if q8 is not None else None,
                                   ids.data_ptr() if ids is not None else None, out.data_ptr())
    d.ncols_x, d.nrows = k, nrows
    d.stride_row = k // BLOCK_ELEMENTS[t] if stride_row is None else stride_row
    d.stride_expert = stride_expert
    d.y_token = padded_k(k) // 32 if y_token is None else y_token
    d.y_slot = y_slot
    d.ids_stride = used
    d.used, d.tokens = used, tokens
    d.dst_token, d.dst_slot = used * nrows, nrows
    d.glu, d.limit = glu, limit
    return d


def vecq(t, w, q8, k, nrows, *, gate=None, ids=None, tokens=1, used=1, stride_row=None,
         stride_expert=0, y_token=None, y_slot=0, glu=GLU_NONE, limit=0.0, variant=-1, out=None):
    """llmp.vecq over Q8_1 activations. Returns float32 [tokens, used, nrows]."""
    lib = _lib.load()
    if out is None:
        out = torch.empty((tokens, used, nrows), dtype=torch.float32, device=w.device)
    d = _desc(t, w, k, nrows, gate=gate, q8=q8, ids=ids, tokens=tokens, used=used,
              stride_row=stride_row, stride_expert=stride_expert, y_token=y_token, y_slot=y_slot,
              glu=glu, limit=limit, out=out)
    _lib.check(lib.llmp_hip_vecq(t, C.byref(d), variant, _stream()))
    return out


def vecq_fused(t, w, x, k, nrows, *, gate=None, ids=None, tokens=1, used=1, stride_row=None,
               stride_expert=0, x_token=None, x_slot=0, glu=GLU_NONE, limit=0.0, variant=-1,
               out=None):
    """llmp.vecq over unquantized activations (float32 or bfloat16), quantized to Q8_1 in LDS."""
    lib = _lib.load()
    if out is None:
        out = torch.empty((tokens, used, nrows), dtype=torch.float32, device=w.device)
    d = _desc(t, w, k, nrows, gate=gate, q8=None, ids=ids, tokens=tokens, used=used,
              stride_row=stride_row, stride_expert=stride_expert, y_token=0, y_slot=0, glu=glu,
              limit=limit, out=out)
    s = VecQSource()
    s.x, s.x_type = x.data_ptr(), _x_type(x)
    s.x_token = k if x_token is None else x_token
    s.x_slot = x_slot
    _lib.check(lib.llmp_hip_vecq_fused(t, C.byref(d), C.byref(s), variant, _stream()))
    return out


def vecq_block_sums(t, w, q8, k, nrows, variant=-1):
    """The kernel's int32 block sums of a dense one-token product: [nrows, blocks, per]."""
    lib = _lib.load()
    per = 1 if t == TYPE_Q8_0 else 16
    sums = torch.zeros((nrows, k // BLOCK_ELEMENTS[t], per), dtype=torch.int32, device=w.device)
    out = torch.empty((1, 1, nrows), dtype=torch.float32, device=w.device)
    d = _desc(t, w, k, nrows, gate=None, q8=q8, ids=None, tokens=1, used=1, stride_row=None,
              stride_expert=0, y_token=None, y_slot=0, glu=GLU_NONE, limit=0.0, out=out)
    _lib.check(lib.llmp_hip_vecq_block_sums(t, C.byref(d), variant, _ptr(sums), _stream()))
    return sums


def vecq_variants():
    lib = _lib.load()
    return [lib.llmp_hip_vecq_variant_name(i).decode() for i in range(lib.llmp_hip_vecq_variants())]
