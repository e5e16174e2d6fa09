"""Operator wrappers over the C ABI. Device memory is held in torch tensors
(plumbing only): every call passes raw addresses and the current HIP stream to
lib/libllmp_hip.so and only queues work, as the reference's Run* operators do
(src/kernels/ggml/vecq.cu:1095-1175)."""
import ctypes as C

import torch

from . import _lib
from ._lib import (GLU_GEGLU, GLU_NONE, GLU_SWIGLU, GLU_SWIGLU_CLAMP, TYPE_Q4_0, TYPE_Q4_1, TYPE_Q4_K,  # noqa: F401
                   TYPE_IQ4_NL, TYPE_MXFP4, TYPE_Q5_0, TYPE_Q5_1, TYPE_Q5_K, TYPE_Q6_K,
                   TYPE_Q8_0, X_BF16, X_F16, X_F32, DecodeOperand, Exl3Linear, Exl3MultiLinear, Exl3Weights, KernelFailure, Mxfp8Gemm, VecQDesc,
                   VecQSource)

BLOCK_BYTES = {TYPE_Q4_0: 18, TYPE_Q4_1: 20, TYPE_Q5_0: 22, TYPE_Q5_1: 24, TYPE_Q8_0: 34, TYPE_Q4_K: 144, TYPE_MXFP4: 17, TYPE_IQ4_NL: 18, TYPE_Q5_K: 176, TYPE_Q6_K: 210}
BLOCK_ELEMENTS = {TYPE_Q4_0: 32, TYPE_Q4_1: 32, TYPE_Q5_0: 32, TYPE_Q5_1: 32, TYPE_Q8_0: 32, TYPE_Q4_K: 256, TYPE_MXFP4: 32, TYPE_IQ4_NL: 32, TYPE_Q5_K: 256, TYPE_Q6_K: 256}


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
    per = 16 if t in (TYPE_Q4_K, TYPE_Q5_K, TYPE_Q6_K) else 1
    sums = torch.zeros((nrows, k // BLOCK_ELEMENTS[t], per), dtype=torch.int32, device=w.device)
    out = torch.empty((1, 1, nrows), dtype=torch.float32, device=w.device)
    d = _desc(t, w, k, nrows, gate=None, q8=q8, ids=None, tokens=1, used=1, stride_row=None,
              stride_expert=0, y_token=None, y_slot=0, glu=GLU_NONE, limit=0.0, out=out)
    _lib.check(lib.llmp_hip_vecq_block_sums(t, C.byref(d), variant, _ptr(sums), _stream()))
    return sums


def relayout_q4_k_tiles64(w, nrows, k, inverse=False):
    """The import-time relayout the variant "rows pass8 tiles64" reads: uint8 Q4_K rows (nrows x k / 256 super-blocks,
    packed) into 64-row tiles, a super-block's 64 rows together; inverse=True undoes it. Returns a new tensor."""
    lib = _lib.load()
    out = torch.empty_like(w)
    _lib.check(lib.llmp_hip_relayout_q4_k_tiles64(_ptr(w), _ptr(out), nrows, k // 256, int(inverse), _stream()))
    return out


def relayout_q8_0_tiles64(w, nrows, k, inverse=False):
    """The same for uint8 Q8_0 rows (nrows x k / 32 blocks, packed; k a multiple of 128): 64-row tiles, four blocks of a
    tile's rows a piece, codes and scales apart. Returns a new tensor."""
    lib = _lib.load()
    out = torch.empty_like(w)
    _lib.check(lib.llmp_hip_relayout_q8_0_tiles64(_ptr(w), _ptr(out), nrows, k // 32, int(inverse), _stream()))
    return out


def vecq_variants():
    lib = _lib.load()
    return [lib.llmp_hip_vecq_variant_name(i).decode() for i in range(lib.llmp_hip_vecq_variants())]


def vecq_sorted(t, w, q8, offsets, k, nrows, experts, *, gate=None, stride_row=None, stride_expert=0,
                glu=GLU_NONE, limit=0.0, variant=-1, out=None):
    """llmp.vecq over rows sorted by expert: q8 [rows, blocks*36] -> float32 [rows, nrows]."""
    lib = _lib.load()
    rows = q8.shape[0]
    if out is None:
        out = torch.empty((rows, nrows), dtype=torch.float32, device=w.device)
    d = _desc(t, w, k, nrows, gate=gate, q8=q8, ids=None, tokens=1, used=1, stride_row=stride_row,
              stride_expert=stride_expert, y_token=None, y_slot=0, glu=glu, limit=limit, out=out)
    d.dst_token = nrows
    _lib.check(lib.llmp_hip_vecq_sorted(t, C.byref(d), _ptr(offsets), experts, variant, _stream()))
    return out


def set_rows_quant(t, x, ids, destination, row_bytes=None):
    """llmp.set_rows.quant: float32 [rows, k] stored as rows ids[r] (int32 or int64) of a Q8_0 or
    Q4_0 destination (uint8 [cells, row_bytes])."""
    lib = _lib.load()
    rows, k = x.shape
    if row_bytes is None:
        row_bytes = destination.stride(0)
    index_bytes = 8 if ids.dtype == torch.int64 else 4
    _lib.check(lib.llmp_hip_set_rows_quant(t, _ptr(x), x.stride(0), _ptr(ids), index_bytes, _ptr(destination),
                                           row_bytes, k, rows, destination.shape[0], _stream()))
    return destination


def set_rows_quant_group(stores):
    """llmp.set_rows.grouped_quant: two to sixteen stores (t, x, ids, destination) in one launch."""
    lib = _lib.load()
    table = (_lib.SetRowsStore * len(stores))()
    for entry, (t, x, ids, destination) in zip(table, stores):
        entry.type, entry.index_bytes = t, 8 if ids.dtype == torch.int64 else 4
        entry.x, entry.x_stride, entry.ids = _ptr(x), x.stride(0), _ptr(ids)
        entry.destination, entry.row_bytes = _ptr(destination), destination.stride(0)
        entry.k, entry.rows, entry.cells = x.shape[1], x.shape[0], destination.shape[0]
    _lib.check(lib.llmp_hip_set_rows_quant_group(len(stores), table, _stream()))


def rope_set_rows_quant(t, x, pos, ids, destination, n_dims, theta_scale, *, freq_scale=1.0, ext_factor=0.0,
                        attn_factor=1.0, corr_dims=(0.0, 0.0), freq_factors=None):
    """llmp.rope.set_rows_quant: float32 x [tokens, heads, head_dim] rotated (NEOX) at int32 pos [tokens] and stored
    as rows ids[token] (int64) of a Q8_0 or Q4_0 destination (uint8 [cells, row_bytes])."""
    lib = _lib.load()
    tokens, heads, head_dim = x.shape
    s = _lib.RopeStore(type=t, heads=heads, head_dim=head_dim, n_dims=n_dims, x=_ptr(x), x_head_stride=x.stride(1),
                       x_token_stride=x.stride(0), pos=_ptr(pos),
                       freq_factors=_ptr(freq_factors) if freq_factors is not None else None, ids=_ptr(ids),
                       destination=_ptr(destination), row_bytes=destination.stride(0), tokens=tokens,
                       freq_scale=freq_scale, ext_factor=ext_factor, attn_factor=attn_factor, theta_scale=theta_scale)
    s.corr_dims[0], s.corr_dims[1] = corr_dims
    _lib.check(lib.llmp_hip_rope_set_rows_quant(C.byref(s), _stream()))
    return destination


def moe_router(logits, used, normalize=True, scale=1.0):
    """llmp.moe.router: float32 [tokens, experts] -> (ids int32 [tokens, used], weights float32)."""
    lib = _lib.load()
    tokens, experts = logits.shape
    ids = torch.empty((tokens, used), dtype=torch.int32, device=logits.device)
    weights = torch.empty((tokens, used), dtype=torch.float32, device=logits.device)
    _lib.check(lib.llmp_hip_moe_router(_ptr(logits), experts, used, tokens, int(normalize), scale, _ptr(ids),
                                       _ptr(weights), _stream()))
    return ids, weights


class Route:
    """Views of llmp.moe.route's buffer (src/kernels/ggml/moe_layout.h:46-70 of the reference)."""

    def __init__(self, buffer, experts, slots):
        self.buffer = buffer
        self.offsets = buffer[:experts + 1]
        self.scale_rows = buffer[experts + 1:2 * (experts + 1)]
        at = 2 * (experts + 1)
        self.position = buffer[at:at + slots]
        self.token = buffer[at + slots:at + 2 * slots]
        self.expert = buffer[at + 2 * slots:at + 3 * slots]


def moe_route(ids, experts):
    lib = _lib.load()
    tokens, used = ids.shape
    ints = lib.llmp_hip_moe_route_ints(experts, used, tokens)
    buffer = torch.empty(ints, dtype=torch.int32, device=ids.device)
    _lib.check(lib.llmp_hip_moe_route(_ptr(ids), ids.stride(0), experts, used, tokens, _ptr(buffer), _stream()))
    return Route(buffer, experts, tokens * used)


def quantize_q8_1_rows(x, rows=None, count=None):
    """llmp.q8_1 with a gather: output row r is input row rows[r]."""
    lib = _lib.load()
    assert x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1
    k = x.shape[1]
    count = (x.shape[0] if rows is None else rows.numel()) if count is None else count
    pk = padded_k(k)
    out = torch.empty((count, pk // 32 * 36), dtype=torch.uint8, device=x.device)
    _lib.check(lib.llmp_hip_q8_1_quantize_rows(_ptr(x), _ptr(rows), _ptr(out), k, pk, x.stride(0), count, _stream()))
    return out


def moe_combine(x, weights, position=None):
    """out[t] = sum_j x[row(t, j)] * weights[t, j] in slot order. x [rows, width]."""
    lib = _lib.load()
    tokens, used = weights.shape
    width = x.shape[-1]
    out = torch.empty((tokens, width), dtype=torch.float32, device=x.device)
    _lib.check(lib.llmp_hip_moe_combine(_ptr(x), _ptr(weights), _ptr(position), width, used, tokens, _ptr(out),
                                        _stream()))
    return out


def moe_ffn(t, logits, x, gate_up, down, hidden, ffn, experts, used, glu=GLU_SWIGLU, keep=None):
    """One routed-expert FFN layer (the decomposition of src/ir/decompose.cc:1080-1109 of the
    reference): route, gate/up with a GLU, down, weighted combine. gate_up is uint8
    [experts, 2 * ffn rows of hidden] (gate rows first), down uint8 [experts, hidden rows of ffn].
    Up to 128 (token, slot) pairs go through the routed mat-vec; more are sorted by expert.
    `keep`, a dict, receives the intermediates (h, hq, y and, when sorted, the route)."""
    tokens = x.shape[0]
    qk, bs = BLOCK_ELEMENTS[t], BLOCK_BYTES[t]
    ids, weights = moe_router(logits, used)
    gu_stride = 2 * ffn * (hidden // qk)
    gate = gate_up
    up = gate_up.view(-1)[ffn * (hidden // qk) * bs:]
    down_stride = hidden * (ffn // qk)
    if tokens * used <= 128:
        if keep is None and tokens * used <= 128:
            # Nobody asks for the intermediates and the pairs are few: each product quantizes
            # its activations itself (the same arithmetic, two launches fewer).
            h = vecq_fused(t, up, x, hidden, ffn, gate=gate, ids=ids, tokens=tokens, used=used,
                           stride_expert=gu_stride, glu=glu)
            y = vecq_fused(t, down, h, ffn, hidden, ids=ids, tokens=tokens, used=used, stride_expert=down_stride,
                           x_token=used * ffn, x_slot=ffn)
            return moe_combine(y.view(tokens * used, hidden), weights), ids, weights
        q8 = quantize_q8_1(x)
        h = vecq(t, up, q8, hidden, ffn, gate=gate, ids=ids, tokens=tokens, used=used, stride_expert=gu_stride,
                 glu=glu)
        hq = quantize_q8_1(h.view(tokens * used, ffn))
        blocks = padded_k(ffn) // 32
        y = vecq(t, down, hq, ffn, hidden, ids=ids, tokens=tokens, used=used, stride_expert=down_stride,
                 y_token=blocks * used, y_slot=blocks)
        if keep is not None:
            keep.update(h=h, hq=hq, y=y)
        return moe_combine(y.view(tokens * used, hidden), weights), ids, weights
    route = moe_route(ids, experts)
    q8 = quantize_q8_1_rows(x, route.token)
    h = vecq_sorted(t, up, q8, route.offsets, hidden, ffn, experts, gate=gate, stride_expert=gu_stride, glu=glu)
    hq = quantize_q8_1_rows(h)
    y = vecq_sorted(t, down, hq, route.offsets, ffn, hidden, experts, stride_expert=down_stride)
    if keep is not None:
        keep.update(h=h, hq=hq, y=y, route=route)
    return moe_combine(y, weights, route.position), ids, weights


def attn_vec_quant(t, q, k_cache, v_cache, mask, head_dim, heads, kv_heads, cells, scale, *, softcap=0.0, sinks=None,
                   cell_stride=None, head_stride=None, out=None, scratch=None):
    """ggml.flash_attn_ext.vec_q8_0 / vec_q4_0: q float32 [heads, rows, head_dim]; k_cache, v_cache uint8 holding
    the row of (cell, KV head) at cell * cell_stride + head * head_stride bytes (default: a cell's heads together);
    mask float16 [>= rows, cells]. Returns float32 [rows, heads, head_dim]."""
    lib = _lib.load()
    rows = q.shape[1]
    row_bytes = head_dim // 32 * BLOCK_BYTES[t]
    head_stride = row_bytes if head_stride is None else head_stride
    cell_stride = row_bytes * kv_heads if cell_stride is None else cell_stride
    if out is None:
        out = torch.empty((rows, heads, head_dim), dtype=torch.float32, device=q.device)
    op = _lib.AttnVecQuant()
    op.q, op.k, op.v, op.mask, op.out = q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), mask.data_ptr(), out.data_ptr()
    op.sinks = sinks.data_ptr() if sinks is not None else None
    op.q_row_stride, op.q_head_stride = q.stride(1), q.stride(0)
    op.k_cell_stride = op.v_cell_stride = cell_stride
    op.k_head_stride = op.v_head_stride = head_stride
    op.mask_row_stride = mask.stride(0)
    op.type, op.head_dim, op.heads, op.kv_heads, op.rows, op.cells = t, head_dim, heads, kv_heads, rows, cells
    op.scale, op.softcap = scale, softcap
    cus = lib.llmp_hip_compute_units()
    need = lib.llmp_hip_attn_vec_quant_scratch(C.byref(op), cus)
    if scratch is None:
        scratch = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    _lib.check(lib.llmp_hip_attn_vec_quant(C.byref(op), _ptr(scratch), scratch.numel(), cus, _stream()))
    return out


class MoeTokenState:
    """What llmp_hip_moe_token keeps between calls on a device: the meeting words (zero before their first use), the
    activated values' scratch, and the router's result."""

    def __init__(self, used, ffn, device):
        self.sync = torch.zeros(4 + 1024, dtype=torch.int32, device=device)
        self.h = torch.empty((used, ffn), dtype=torch.float32, device=device)
        self.ids = torch.empty(used, dtype=torch.int32, device=device)
        self.weights = torch.empty(used, dtype=torch.float32, device=device)


def moe_token(t, logits, x, gate_up, down, hidden, ffn, experts, used, state, *, glu=GLU_SWIGLU, limit=0.0, launches=2, out=None):
    """One token's routed-expert FFN layer in two launches, or one with the halves meeting inside it (llmp_hip_moe_token): logits float32 [experts], x float32 or
    bfloat16 [hidden]; gate_up, down as moe_ffn takes them. Returns float32 [hidden]; state.ids and state.weights hold
    the router's result."""
    lib = _lib.load()
    qk = BLOCK_ELEMENTS[t]
    if out is None:
        out = torch.empty(hidden, dtype=torch.float32, device=x.device)
    op = _lib.MoeToken()
    op.logits, op.x, op.gate_up, op.down, op.out = logits.data_ptr(), x.data_ptr(), gate_up.data_ptr(), down.data_ptr(), out.data_ptr()
    op.ids, op.weights, op.h, op.sync = state.ids.data_ptr(), state.weights.data_ptr(), state.h.data_ptr(), state.sync.data_ptr()
    op.gate_up_stride, op.down_stride = 2 * ffn * (hidden // qk), hidden * (ffn // qk)
    op.type, op.x_type, op.experts, op.used, op.hidden, op.ffn = t, _x_type(x), experts, used, hidden, ffn
    op.glu, op.normalize, op.limit, op.route_scale = glu, 1, limit, 1.0
    _lib.check(lib.llmp_hip_moe_token(C.byref(op), launches, lib.llmp_hip_compute_units(), _stream()))
    return out


def moe_gemm(a_codes, a_scales, offsets, sf_rows, weights, expert_stride, codes_offset, scales_offset, n, k, out=None):
    """llmp.moe.gemm (RunGroupedGemm, src/kernels/ggml/moe_cutlass.h:48-76 of the reference): routed rows sorted
    by expert, NVFP4 codes uint8 [rows, k / 2] with UE4M3 scales in atoms, times each expert's n rows of the
    same encoding inside `weights`; offsets and sf_rows int32 [groups + 1]. Returns bfloat16 [rows, n]."""
    lib = _lib.load()
    rows = a_codes.shape[0]
    if out is None:
        out = torch.empty((rows, n), dtype=torch.bfloat16, device=a_codes.device)
    g = _lib.GroupedGemm()
    g.groups, g.n, g.k = offsets.numel() - 1, n, k
    g.offsets, g.sf_rows, g.a, g.a_scales, g.weights = (offsets.data_ptr(), sf_rows.data_ptr(), a_codes.data_ptr(),
                                                        a_scales.data_ptr(), weights.data_ptr())
    g.expert_stride, g.codes_offset, g.scales_offset = expert_stride, codes_offset, scales_offset
    g.d, g.scratch = out.data_ptr(), None
    _lib.check(lib.llmp_hip_grouped_gemm_run(C.byref(g), lib.llmp_hip_compute_units(), _stream()))
    return out


def mxfp8_scale_bytes(rows, k):
    """SwizzledScaleBytes: src/kernels/ggml/mxfp8_cutlass.h:53-57 of the reference."""
    return (rows + 127) // 128 * 128 * (k // 32)


def stream_read(data, sink=None):
    """A launch that only reads `data` (a uint8 tensor of whole 16-byte chunks): the yardstick beside the streaming
    kernels' times. Returns the sink (reuse it across calls)."""
    lib = _lib.load()
    cus = lib.llmp_hip_compute_units()
    if sink is None:
        sink = torch.empty(lib.llmp_hip_stream_read_sink(cus), dtype=torch.uint8, device=data.device)
    _lib.check(lib.llmp_hip_stream_read(_ptr(data), data.numel() * data.element_size(), _ptr(sink), cus, _stream()))
    return sink


def mxfp8_quantize(x, out=None):
    """llmp.mxfp8.quantize: float32 / bfloat16 [rows, k] -> (codes uint8 [rows, k], scales uint8 atoms); `out`,
    a pair of such tensors, is filled in place."""
    lib = _lib.load()
    rows, k = x.shape
    if out is None:
        out = (torch.empty((rows, k), dtype=torch.uint8, device=x.device),
               torch.empty(mxfp8_scale_bytes(rows, k), dtype=torch.uint8, device=x.device))
    codes, scales = out
    _lib.check(lib.llmp_hip_mxfp8_quantize(_ptr(x), _x_type(x), x.stride(0), k, rows, _ptr(codes), _ptr(scales),
                                           _stream()))
    return codes, scales


def mxfp8_swizzle(scales):
    """llmp.mxfp8.swizzle: uint8 [n, k / 32] -> atoms."""
    lib = _lib.load()
    n, blocks = scales.shape
    out = torch.empty(mxfp8_scale_bytes(n, blocks * 32), dtype=torch.uint8, device=scales.device)
    _lib.check(lib.llmp_hip_mxfp8_swizzle(_ptr(scales), n, blocks * 32, _ptr(out), _stream()))
    return out


def mxfp8_gemv(codes, scales, x):
    """llmp.mxfp8.mul_mat_vec: codes [n, k], plain scales [n, k / 32], x float32 [tokens, k]."""
    lib = _lib.load()
    n, k = codes.shape
    tokens = x.shape[0]
    y = torch.empty((tokens, n), dtype=torch.float32, device=x.device)
    _lib.check(lib.llmp_hip_mxfp8_gemv(_ptr(codes), _ptr(scales), n, k, _ptr(x), tokens, _ptr(y), _stream()))
    return y


def mxfp8_gemm(a_codes, a_scales, b_codes, b_scales, bf16=True, out=None, compute_units=None):
    """llmp.mxfp8.gemm: D[m, n] = A[m, k] B[n, k]^T, scales in atoms. `compute_units`: the count the reference's run
    call passes (the device's by default); the launch has no more workgroups than that, each through its share of
    the tiles."""
    lib = _lib.load()
    m, k = a_codes.shape
    n = b_codes.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16 if bf16 else torch.float32, device=a_codes.device)
    g = Mxfp8Gemm()
    g.m, g.n, g.k = m, n, k
    g.a, g.a_scales, g.b, g.b_scales, g.d = (a_codes.data_ptr(), a_scales.data_ptr(), b_codes.data_ptr(),
                                             b_scales.data_ptr(), out.data_ptr())
    g.bf16 = int(bf16)
    g.scratch = None
    cus = lib.llmp_hip_compute_units() if compute_units is None else int(compute_units)
    _lib.check(lib.llmp_hip_mxfp8_gemm_run(C.byref(g), cus, _stream()))
    return out


EXL3_3INST, EXL3_MCG, EXL3_MUL1 = 0, 1, 2


def _exl3_weights(trellis, suh, svh, k, n, bits, codebook):
    w = Exl3Weights()
    w.trellis, w.suh, w.svh = trellis.data_ptr(), suh.data_ptr(), svh.data_ptr()
    w.k, w.n, w.bits, w.codebook = k, n, bits, codebook
    return w


def exl3_reconstruct(trellis, suh, svh, k, n, bits, codebook, column=0, columns=None, fused=False):
    """Columns [column, column + columns) as float16 [k, columns]: the rotated-basis weights, or (fused, the
    reference's ReconstructOperands::fused) the weights themselves, both transforms and side vectors applied."""
    lib = _lib.load()
    columns = n if columns is None else columns
    out = torch.empty((k, columns), dtype=torch.float16, device=trellis.device)
    w = _exl3_weights(trellis, suh, svh, k, n, bits, codebook)
    launch = lib.llmp_hip_exl3_reconstruct_fused if fused else lib.llmp_hip_exl3_reconstruct
    _lib.check(launch(C.byref(w), _ptr(out), column, columns, _stream()))
    return out


def exl3_hadamard(x, scale, input_scale=True):
    """128-point Hadamard transforms of x's rows, times 1 / sqrt(128), with the input or output scale."""
    lib = _lib.load()
    rows, columns = x.shape
    y = torch.empty_like(x)
    _lib.check(lib.llmp_hip_exl3_hadamard(_ptr(x), _ptr(y), _ptr(scale), rows, columns,
                                          int(x.dtype == torch.float32), int(input_scale), _stream()))
    return y


def exl3_linear(trellis, suh, svh, k, n, bits, codebook, x, f32=True, keep=None):
    """x float16 [m, k] through the EXL3 linear (sixteen rows a pass): [m, n] float32 or float16.
    `keep`, a dict, receives the transformed input a_had."""
    lib = _lib.load()
    m = x.shape[0]
    op = Exl3Linear()
    op.weights = _exl3_weights(trellis, suh, svh, k, n, bits, codebook)
    a_had = torch.empty((m, k), dtype=torch.float16, device=x.device)
    y = torch.empty((m, n), dtype=torch.float32 if f32 else torch.float16, device=x.device)
    op.x, op.a_had, op.y, op.f32, op.m = x.data_ptr(), a_had.data_ptr(), y.data_ptr(), int(f32), m
    need = lib.llmp_hip_exl3_linear_scratch(C.byref(op))
    scratch = torch.empty(max(need, 8), dtype=torch.uint8, device=x.device)
    _lib.check(lib.llmp_hip_exl3_linear(C.byref(op), _ptr(scratch), need, _stream()))
    if keep is not None:
        keep["a_had"] = a_had
    return y


def exl3_linear_reconstructed(trellis, suh, svh, k, n, bits, codebook, x, f32=True, fused=True, w=None):
    """The same linear through a reconstruction path (the reference's ReconstructedLinear, upstream's choice from 145
    rows; fused from 1,024): the weights reconstructed to float16 a slice at a time into the scratch `w`, a plain
    float16 product with float32 sums a slice. x float16 [m, k]: [m, n] float32 or float16."""
    lib = _lib.load()
    m = x.shape[0]
    op = Exl3Linear()
    op.weights = _exl3_weights(trellis, suh, svh, k, n, bits, codebook)
    a_had = torch.empty((m, k), dtype=torch.float16, device=x.device)
    y = torch.empty((m, n), dtype=torch.float32 if f32 else torch.float16, device=x.device)
    op.x, op.a_had, op.y, op.f32, op.m = x.data_ptr(), a_had.data_ptr(), y.data_ptr(), int(f32), m
    need = lib.llmp_hip_exl3_reconstructed_scratch(C.byref(op.weights))
    if w is None:
        w = torch.empty(need, dtype=torch.uint8, device=x.device)
    _lib.check(lib.llmp_hip_exl3_linear_reconstructed(C.byref(op), _ptr(w), w.numel() * w.element_size(), int(fused),
                                                      lib.llmp_hip_compute_units(), _stream()))
    return y


def exl3_linear_static(trellis, suh, svh, k, n, bits, codebook, x, a_had, y):
    """The same linear through llmp_hip_exl3_linear_static: the partial sums go to the library's static array
    on this device, the call allocates nothing. x float16 [m, k]; a_had float16 [m, k] and y float32 or
    float16 [m, n] are the caller's, filled in place."""
    lib = _lib.load()
    m = x.shape[0]
    op = Exl3Linear()
    op.weights = _exl3_weights(trellis, suh, svh, k, n, bits, codebook)
    op.x, op.a_had, op.y, op.f32, op.m = x.data_ptr(), a_had.data_ptr(), y.data_ptr(), int(y.dtype == torch.float32), m
    _lib.check(lib.llmp_hip_exl3_linear_static(C.byref(op), _stream()))
    return y


def exl3_linear_static_prepare(trellis, suh, svh, k, n, bits, codebook):
    """llmp_hip_exl3_linear_static_prepare: the set-up that is no launch (the static array's address on this device,
    the product kernels' dynamic LDS), to be done outside a stream capture."""
    lib = _lib.load()
    op = Exl3Linear()
    op.weights = _exl3_weights(trellis, suh, svh, k, n, bits, codebook)
    _lib.check(lib.llmp_hip_exl3_linear_static_prepare(C.byref(op)))


def exl3_multi_linear(first, second, x, f32=True, keep=None):
    """exl3.multi_linear: x float16 [m, k] (sixteen rows a pass) through a gate and an up linear of the same k, n and
    rate: [2, m, n]. `first` and `second` are (trellis, suh, svh, k, n, bits, codebook); `keep`, a dict,
    receives the two transformed inputs a_had [2, m, k]."""
    lib = _lib.load()
    m = x.shape[0]
    k, n = first[3], first[4]
    op = Exl3MultiLinear()
    op.first = _exl3_weights(*first)
    op.second = _exl3_weights(*second)
    a_had = torch.empty((2, m, k), dtype=torch.float16, device=x.device)
    y = torch.empty((2, m, n), dtype=torch.float32 if f32 else torch.float16, device=x.device)
    op.x, op.a_had, op.y, op.f32, op.m = x.data_ptr(), a_had.data_ptr(), y.data_ptr(), int(f32), m
    need = lib.llmp_hip_exl3_multi_linear_scratch(C.byref(op))
    scratch = torch.empty(max(need, 8), dtype=torch.uint8, device=x.device)
    _lib.check(lib.llmp_hip_exl3_multi_linear(C.byref(op), _ptr(scratch), need, _stream()))
    if keep is not None:
        keep["a_had"] = a_had
    return y


DECODERS = ("bf16.dense", "f16.dense", "q8_0.blocks", "nvfp4.split", "nvfp4.atoms", "nvfp4.interleaved",
            "nvfp4.ggml_blocks", "mxfp8.split", "mxfp8.atoms", "mxfp4.split", "mxfp4.atoms", "affine.split")


def _decode_operand(weight):
    data = weight["data"]
    op = DecodeOperand()
    op.data = data.data_ptr()
    op.scales = weight["scales"].data_ptr() if weight.get("scales") is not None else None
    op.tensor_scale = weight["tensor_scale"].data_ptr() if weight.get("tensor_scale") is not None else None
    op.k, op.rows, op.row_bytes = weight["k"], data.shape[0], data.stride(0)
    op.rows_per_scale = weight.get("rows_per_scale", data.shape[0])
    if "group" in weight:  # the affine encoding
        op.biases = weight["biases"].data_ptr() if weight.get("biases") is not None else None
        op.group, op.bits, op.scale_type = weight["group"], weight["bits"], weight["scale_type"]
        op.scale_row_bytes = weight["scale_row_bytes"]
    return op


def decode_vector_glu(decoder, gate, up, x, glu, limit=0.0, gate_first=0, up_first=0, outputs=None, up_decoder=None):
    """llmp.decode.vector_glu: glu(gate rows . x, up rows . x), float32 [rows, outputs]; `glu` is the
    reference's ir::GluKind (0 SwiGLU, 1 GeGLU erf, 2 GeGLU tanh, 3 SwiGLU with a clamp at `limit`)."""
    lib = _lib.load()
    g, u = _decode_operand(gate), _decode_operand(up)
    outputs = gate["data"].shape[0] - gate_first if outputs is None else outputs
    rows = x.shape[0]
    y = torch.empty((rows, outputs), dtype=torch.float32, device=x.device)
    _lib.check(lib.llmp_hip_decode_vector_glu(decoder, C.byref(g), gate_first, decoder if up_decoder is None else up_decoder,
                                              C.byref(u), up_first, outputs, glu, limit, _ptr(x), rows, x.stride(0),
                                              _ptr(y), y.stride(0), _stream()))
    return y


def decode_vector(decoder, weight, x, first=0, outputs=None, out=None):
    """llmp.decode.vector: float32 x [rows <= 16, k] times a weight in its stored encoding. `weight` is a
    dict of device tensors: data (uint8 [n, row_bytes]), k, and where the decoder has them scales (uint8)
    and tensor_scale (float32) with rows_per_scale. Returns float32 [rows, outputs]."""
    lib = _lib.load()
    data = weight["data"]
    op = _decode_operand(weight)
    outputs = data.shape[0] - first if outputs is None else outputs
    rows = x.shape[0]
    y = torch.empty((rows, outputs), dtype=torch.float32, device=x.device) if out is None else out
    _lib.check(lib.llmp_hip_decode_vector(decoder, C.byref(op), first, outputs, _ptr(x), rows, x.stride(0), _ptr(y),
                                          y.stride(0), _stream()))
    return y


def decode_rows(decoder, weight, ids, bad=None):
    """llmp.decode.rows: rows ids[i] (int32) of a weight in its stored encoding as float32 [count, k], times their
    tensor scales; an id outside the matrix gives a row of zeros and sets `bad` (an int32 tensor of one element)."""
    lib = _lib.load()
    op = _decode_operand(weight)
    out = torch.empty((ids.numel(), weight["k"]), dtype=torch.float32, device=ids.device)
    _lib.check(lib.llmp_hip_decode_rows(decoder, C.byref(op), _ptr(ids), ids.numel(), _ptr(out), out.stride(0),
                                        _ptr(bad) if bad is not None else None, _stream()))
    return out


def decode_grouped(decoder, experts, k, n, offsets, pair_rows, x, y, pair_out=None, first=0, outputs=None):
    """llmp.decode.grouped: an expert worklist's products. `experts` is a list of weights (dicts of device tensors,
    one matrix each); offsets (int32 [experts + 1]), pair_rows and pair_out (int32 [pairs]) are device tensors; `y`
    (float32 [y_rows, outputs]) is updated in place at the rows the pairs name."""
    import numpy as np
    lib = _lib.load()
    table = (DecodeOperand * len(experts))(*[_decode_operand(w) for w in experts])
    raw = np.frombuffer(bytes(table), dtype=np.uint8).copy()
    table_d = torch.from_numpy(raw).to(x.device)  # the operands, in device memory
    outputs = n - first if outputs is None else outputs
    _lib.check(lib.llmp_hip_decode_grouped(decoder, _ptr(table_d), len(experts), k, n, first, outputs, _ptr(offsets),
                                           _ptr(pair_rows), _ptr(pair_out) if pair_out is not None else None,
                                           pair_rows.numel(), _ptr(x), x.shape[0], x.stride(0), _ptr(y), y.shape[0],
                                           y.stride(0), 0, _stream()))
    torch.cuda.current_stream().synchronize()  # table_d must outlive the launch
    return y


def decode_matrix(decoder, weight, x, first=0, outputs=None, path=0, out=None):
    """llmp.decode.matrix: float32 x [rows, k] (any number of rows) times a weight in its stored encoding on the
    matrix cores, weights and inputs rounded to the decoder's matrix element. float32 [rows, outputs]."""
    lib = _lib.load()
    op = _decode_operand(weight)
    outputs = weight["data"].shape[0] - first if outputs is None else outputs
    rows = x.shape[0]
    y = torch.empty((rows, outputs), dtype=torch.float32, device=x.device) if out is None else out
    _lib.check(lib.llmp_hip_decode_matrix(decoder, C.byref(op), first, outputs, _ptr(x), rows, x.stride(0), _ptr(y),
                                          y.stride(0), path, _stream()))
    return y
