"""ggml.flash_attn_ext.vec_q8_0 / vec_q4_0 (llmp_hip_attn_vec_quant) against the oracle's attention over the same K
and V bytes decoded exactly, attention in F64: the reference's own cases and bound
(tests/unit/kv_quant_gpu_test.cc:826-950: decode and prefill shapes, D 64 and 256, no GQA and GQA 2, 7 and 8, with and
without a softcap, causal masks with biases; NMSE 5e-4), and, tighter, against the same attention over the queries as
the device multiplies them (through Q8_1): what is left is the order of F32 sums."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from llmp_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu

Q8_0, Q4_0 = ops.TYPE_Q8_0, ops.TYPE_Q4_0

# (head_dim, heads, kv_heads, rows, cells, softcap): the reference's twelve.
CASES = [(64, 14, 2, 1, 512, 0.0), (64, 2, 2, 1, 256, 0.0), (64, 2, 2, 1025, 1280, 0.0), (256, 4, 4, 3, 512, 30.0),
         (64, 14, 2, 2, 512, 0.0), (64, 14, 2, 33, 768, 0.0), (64, 4, 2, 1024, 1280, 0.0), (256, 8, 4, 1, 1024, 0.0),
         (256, 8, 4, 2, 512, 50.0), (256, 8, 4, 1, 512, 30.0), (256, 8, 4, 17, 512, 0.0), (256, 16, 2, 1, 2048, 0.0)]


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def operands(t, d, heads, kv_heads, rows, cells, seed):
    g = synth.rng(seed)
    keys = g.standard_normal((cells * kv_heads, d), dtype=np.float32)
    vals = g.standard_normal((cells * kv_heads, d), dtype=np.float32)
    k_cache = oracle.kv_quantize(t, keys).reshape(cells, -1)  # a cell's heads together
    v_cache = oracle.kv_quantize(t, vals).reshape(cells, -1)
    q = g.standard_normal((heads, rows, d), dtype=np.float32)
    # Causal over the filled cells, row r at position filled - rows + r, every fifth cell with a bias.
    mask_rows = rows + rows % 2
    filled = cells - 37
    mask = np.full((mask_rows, cells), -np.inf, dtype=np.float32)
    for r in range(mask_rows):
        position = min(filled - 1, filled - rows + r)
        mask[r, :position + 1] = 0.0
        mask[r, 1:position + 1:5] = -0.75
    return q, k_cache, v_cache, mask.astype(np.float16)


def nmse(got, want):
    return float(np.sum((got.astype(np.float64) - want) ** 2) / np.sum(want.astype(np.float64) ** 2))


@pytest.mark.parametrize("t", [Q8_0, Q4_0])
@pytest.mark.parametrize("case", CASES)
def test_attention_matches_the_oracle_at_decode_and_prefill_shapes(device, t, case):
    d, heads, kv_heads, rows, cells, softcap = case
    q, k_cache, v_cache, mask = operands(t, d, heads, kv_heads, rows, cells, 900 + d + heads + rows)
    scale = float(1.0 / np.sqrt(np.float32(d)))
    got = ops.attn_vec_quant(t, dev(q, device), dev(k_cache, device), dev(v_cache, device), dev(mask.view(np.int16), device).view(torch.float16),
                             d, heads, kv_heads, cells, scale, softcap=softcap).cpu().numpy()
    assert np.all(np.isfinite(got))
    # Sample the rows where the oracle would take long (every row of the device's output is checked for finiteness).
    pick = np.arange(rows) if rows <= 40 else np.unique(np.concatenate([np.arange(0, rows, 37), [rows - 2, rows - 1]]))
    threads = oracle.max_threads()
    exact = oracle.attention_quant(t, q[:, pick], k_cache, v_cache, d, heads, kv_heads, len(pick), cells, scale,
                                   mask=mask[pick], softcap=softcap, threads=threads)
    assert nmse(got[pick], exact) <= 5e-4  # the reference's bound
    same_q = oracle.attention_quant(t, q[:, pick], k_cache, v_cache, d, heads, kv_heads, len(pick), cells, scale,
                                    mask=mask[pick], softcap=softcap, q8_1_q=True, threads=threads)
    rms = np.sqrt(np.mean(same_q.astype(np.float64) ** 2))
    worst = np.max(np.abs(got[pick] - same_q) / np.maximum(np.abs(same_q), 1e-2 * rms))
    assert worst <= 2e-3, worst
    assert nmse(got[pick], same_q) <= 1e-8


def test_attention_sinks_pitched_cells_and_a_row_that_sees_nothing(device):
    t, d, heads, kv_heads, rows, cells = Q8_0, 64, 8, 2, 3, 256
    q, k_cache, v_cache, mask = operands(t, d, heads, kv_heads, rows, cells, 77)
    row_bytes = d // 32 * 34
    pitch = row_bytes * kv_heads + 2 * 34  # a gap of two blocks after every cell's rows
    kp = np.zeros((cells, pitch), dtype=np.uint8)
    vp = np.zeros((cells, pitch), dtype=np.uint8)
    kp[:, :row_bytes * kv_heads], vp[:, :row_bytes * kv_heads] = k_cache, v_cache
    mask[2, :] = -np.inf  # the third row sees nothing
    sinks = synth.rng(78).standard_normal(heads).astype(np.float32)
    mask_d = dev(mask.view(np.int16), device).view(torch.float16)
    for use_sinks in (False, True):
        got = ops.attn_vec_quant(t, dev(q, device), dev(kp, device), dev(vp, device), mask_d, d, heads, kv_heads, cells, 0.125,
                                 sinks=dev(sinks, device) if use_sinks else None, cell_stride=pitch, head_stride=row_bytes).cpu().numpy()
        want = oracle.attention_quant(t, q, kp, vp, d, heads, kv_heads, rows, cells, 0.125, mask=mask,
                                      sinks=sinks if use_sinks else None, cell_stride=pitch, head_stride=row_bytes, q8_1_q=True)
        assert nmse(got[:2], want[:2]) <= 1e-8
        if not use_sinks:
            assert np.all(got[2] == 0.0)
        else:
            assert np.all(np.abs(got[2]) <= 1e-30) and np.all(want[2] == 0.0)


def test_attention_refusals(device):
    lib = _lib.load()
    op = _lib.AttnVecQuant()
    op.q, op.k, op.v, op.mask, op.out = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000
    op.q_row_stride, op.q_head_stride = 64, 64
    op.k_cell_stride = op.v_cell_stride = 136
    op.k_head_stride = op.v_head_stride = 68
    op.mask_row_stride = 256
    op.type, op.head_dim, op.heads, op.kv_heads, op.rows, op.cells = Q8_0, 64, 4, 2, 1, 256
    op.scale, op.softcap = 0.125, 0.0
    assert lib.llmp_hip_attn_vec_quant_scratch(C.byref(op), 256) > 0

    def refused(what, **fields):
        saved = {k: getattr(op, k) for k in fields}
        for k, v in fields.items():
            setattr(op, k, v)
        assert lib.llmp_hip_attn_vec_quant_scratch(C.byref(op), 256) == 0
        assert lib.llmp_hip_attn_vec_quant(C.byref(op), 0x6000, 1 << 30, 256, None) == 1
        assert what in lib.llmp_hip_last_error(), lib.llmp_hip_last_error()
        for k, v in saved.items():
            setattr(op, k, v)

    refused(b"Q8_0 or both Q4_0", type=ops.TYPE_Q4_K)          # mixed or other encodings
    refused(b"head sizes", head_dim=128)                       # D 128 is not compiled
    refused(b"head sizes", type=Q4_0, head_dim=512)            # 512 for Q8_0 only
    refused(b"softcap", softcap=30.0)                          # a softcap at D 64
    refused(b"padded to 256", cells=300)                       # unpadded cells
    refused(b"query heads a KV head", heads=5)                 # not a whole group
    refused(b"at most 8", heads=18, kv_heads=2)
    refused(b"null operand", mask=None)
    refused(b"strides", k_cell_stride=100)
    assert lib.llmp_hip_attn_vec_quant(C.byref(op), 0x6000, 16, 256, None) == 1 and b"scratch" in lib.llmp_hip_last_error()
