"""llmp.set_rows.quant: F32 rows into a Q8_0 or Q4_0 cache at row indices, each block quantized
with GGML's reference arithmetic (src/kernels/ggml/kv_quant.cuh:27-69 of the reference): the
device's bytes are the oracle's."""
import numpy as np
import pytest
import torch

import oracle
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def corner_rows(k):
    """Rows that exercise the quantizers' branches: a zero block, equal magnitudes of both
    signs (the first decides Q4_0's scale), exact half steps, one huge value, tiny values."""
    g = synth.rng(71)
    x = g.standard_normal((6, k), dtype=np.float32)
    x[0, :32] = 0.0
    x[1, :32] = np.tile(np.array([-3.0, 3.0], dtype=np.float32), 16)
    x[2, :32] = np.tile(np.array([3.0, -3.0], dtype=np.float32), 16)
    x[3, :32] = (np.arange(32, dtype=np.float32) - 15.5) * 0.5
    x[4, 5] = 1.0e6
    x[5] *= 1.0e-30
    return x


@pytest.mark.parametrize("t", [ops.TYPE_Q8_0, ops.TYPE_Q4_0])
@pytest.mark.parametrize("index", [torch.int32, torch.int64])
def test_stored_rows_are_the_reference_quantizers_bytes(device, t, index):
    k, cells = 256, 40
    x = np.concatenate([corner_rows(k), synth.activations(9, k, 72) * 3.0])
    rows = x.shape[0]
    ids = synth.rng(73).permutation(cells)[:rows]
    row_bytes = k // 32 * ops.BLOCK_BYTES[t] + 6  # rows a few bytes apart from packed
    cache = torch.full((cells, row_bytes), 0xA5, dtype=torch.uint8, device=device)
    ops.set_rows_quant(t, dev(x, device), dev(ids, device).to(index), cache)
    got = cache.cpu().numpy()
    want = oracle.kv_quantize(t, x)
    for r in range(rows):
        assert np.array_equal(got[ids[r], : want.shape[1]], want[r]), r
        assert np.all(got[ids[r], want.shape[1]:] == 0xA5)  # nothing past the row's blocks
    untouched = np.setdiff1d(np.arange(cells), ids)
    assert np.all(got[untouched] == 0xA5)


def test_stored_q8_0_rows_feed_the_mat_vec(device):
    """A cache row decodes to the values a Q8_0 weight row of the same bytes gives: the store's
    blocks are the blocks llmp.vecq reads."""
    k, n = 512, 8
    x = synth.activations(n, k, 74)
    cache = torch.zeros((n, k // 32 * 34), dtype=torch.uint8, device=device)
    ops.set_rows_quant(ops.TYPE_Q8_0, dev(x, device), dev(np.arange(n, dtype=np.int32), device), cache)
    a = synth.activations(1, k, 75)
    q8 = oracle.q8_1_quantize(a)
    got = ops.vecq(ops.TYPE_Q8_0, cache, dev(q8, device), k, n).cpu().numpy()
    want = oracle.vecq(oracle.TYPE_Q8_0, cache.cpu().numpy(), q8, k, n)
    assert np.allclose(got, want, rtol=1e-4, atol=1e-5)


def test_refusals(device):
    x = torch.zeros((2, 64), dtype=torch.float32, device=device)
    ids = torch.zeros(2, dtype=torch.int32, device=device)
    cache = torch.zeros((4, 68), dtype=torch.uint8, device=device)
    with pytest.raises(ops.KernelFailure):
        ops.set_rows_quant(ops.TYPE_Q4_K, x, ids, cache)
    with pytest.raises(ops.KernelFailure):
        ops.set_rows_quant(ops.TYPE_Q8_0, x, ids, cache, row_bytes=40)  # rows would overlap
    with pytest.raises(ops.KernelFailure):
        ops.set_rows_quant(ops.TYPE_Q8_0, x[:, :48], ids, cache)  # not whole blocks


def test_grouped_stores_write_what_the_single_stores_write(device):
    """llmp.set_rows.grouped_quant (src/kernels/ggml/kv_quant.h:172-178 of the reference): a layer's K and V rows and
    another's, of different widths, types and index types, in one launch; every cache's bytes are the single
    store's (and so the oracle's)."""
    g = synth.rng(81)
    shapes = [(ops.TYPE_Q8_0, 256, 11, torch.int64), (ops.TYPE_Q4_0, 512, 7, torch.int32),
              (ops.TYPE_Q8_0, 64, 30, torch.int32), (ops.TYPE_Q4_0, 1024, 1, torch.int64)]
    stores, alone = [], []
    for t, k, rows, index in shapes:
        cells = rows + 9
        x = dev(synth.activations(rows, k, 82 + k) * 2.0, device)
        ids = dev(g.permutation(cells)[:rows], device).to(index)
        row_bytes = k // 32 * ops.BLOCK_BYTES[t]
        stores.append((t, x, ids, torch.full((cells, row_bytes), 0x5A, dtype=torch.uint8, device=device)))
        alone.append(ops.set_rows_quant(t, x, ids, torch.full((cells, row_bytes), 0x5A, dtype=torch.uint8, device=device)))
    ops.set_rows_quant_group(stores)
    for (t, x, ids, cache), single in zip(stores, alone):
        assert torch.equal(cache, single)
        want = oracle.kv_quantize(t, x.cpu().numpy())
        assert np.array_equal(cache.cpu().numpy()[ids.cpu().numpy()], want)


def test_grouped_store_refusals(device):
    x = torch.zeros((4, 64), dtype=torch.float32, device=device)
    ids = torch.arange(4, dtype=torch.int32, device=device)
    cache = torch.zeros((8, 68), dtype=torch.uint8, device=device)
    other = torch.zeros((8, 68), dtype=torch.uint8, device=device)
    with pytest.raises(ops.KernelFailure):  # two through sixteen
        ops.set_rows_quant_group([(ops.TYPE_Q8_0, x, ids, cache)])
    with pytest.raises(ops.KernelFailure):
        ops.set_rows_quant_group([(ops.TYPE_Q8_0, x, ids, cache)] * 17)
    with pytest.raises(ops.KernelFailure):  # the same destination twice
        ops.set_rows_quant_group([(ops.TYPE_Q8_0, x, ids, cache), (ops.TYPE_Q8_0, x, ids, cache)])
    with pytest.raises(ops.KernelFailure):  # a member that the single store refuses
        ops.set_rows_quant_group([(ops.TYPE_Q8_0, x, ids, cache), (ops.TYPE_Q4_K, x, ids, other)])
    assert torch.count_nonzero(cache) == 0 and torch.count_nonzero(other) == 0  # nothing was queued


@pytest.mark.parametrize("t", [ops.TYPE_Q8_0, ops.TYPE_Q4_0])
@pytest.mark.parametrize("yarn", [False, True])
@pytest.mark.parametrize("n_dims", [96, 64])  # halves of 48 (a block spans both) and of 32 (16-byte loads)
def test_rope_then_store_matches_the_oracles_rotation_and_quantizer(device, t, yarn, n_dims):
    """llmp.rope.set_rows_quant (src/kernels/ggml/kv_quant.h:180-192, kv_quant_rope.cu:29-120 of the reference)
    against oracle.rope_neox followed by the reference quantizers. The device rotates with F32 cosf / sinf / powf,
    the oracle as the reference's CPU executor does (FP64 cosine, sine and products): the stored bytes are the
    oracle's except for a few codes whose value lies at a rounding boundary (at most 1 in 500 bytes may differ here,
    and every stored value is within 0.6 quantization steps, Q4_0 1.1, of the oracle's rotated value)."""
    g = synth.rng(95)
    tokens, heads, head_dim, cells = 9, 4, 128, 20
    whole = synth.activations(tokens, heads * (head_dim + 32), 96).reshape(tokens, heads, head_dim + 32)
    x = whole[:, :, :head_dim]  # heads 160 floats apart
    pos = np.array([0, 1, 2, 17, 100, 511, 1024, 2047, 3000], dtype=np.int32)
    ids = g.permutation(cells)[:tokens].astype(np.int64)
    theta_scale = float(np.float32(10000.0 ** (-2.0 / n_dims)))
    ff = g.uniform(0.8, 2.0, size=n_dims // 2).astype(np.float32)
    kw = dict(freq_scale=0.5, ext_factor=1.0, attn_factor=1.2, corr_dims=(10.0, 30.0)) if yarn else {}
    rotated = oracle.rope_neox(x, pos, n_dims, theta_scale, freq_factors=ff, **kw)
    want = oracle.kv_quantize(t, rotated.reshape(tokens, heads * head_dim))
    xd = dev(whole, device)[:, :, :head_dim]
    cache = torch.full((cells, want.shape[1] + 4), 0xA5, dtype=torch.uint8, device=device)
    ops.rope_set_rows_quant(t, xd, dev(pos, device), dev(ids, device), cache, n_dims, theta_scale,
                            freq_factors=dev(ff, device), **kw)
    got = cache.cpu().numpy()
    assert np.all(got[np.setdiff1d(np.arange(cells), ids)] == 0xA5) and np.all(got[:, want.shape[1]:] == 0xA5)
    stored = got[ids][:, : want.shape[1]]
    assert np.count_nonzero(stored != want) <= stored.size // 500
    size = ops.BLOCK_BYTES[t]
    blocks = stored.reshape(tokens, -1, size)
    d = blocks[:, :, 0:2].copy().view(np.float16).astype(np.float32)[:, :, 0]
    if t == ops.TYPE_Q8_0:
        values = blocks[:, :, 2:].view(np.int8).astype(np.float32) * d[:, :, None]
    else:
        nib = blocks[:, :, 2:]
        values = (np.concatenate([nib & 15, nib >> 4], axis=2).astype(np.float32) - 8.0) * d[:, :, None]
    error = np.abs(values.reshape(tokens, -1) - rotated.reshape(tokens, -1))
    step = np.repeat(np.abs(d), 32, axis=1).reshape(tokens, -1)
    # Half a step, plus the F16 rounding of the scale times the largest code; Q4_0's top value is clamped a step down.
    assert np.all(error <= (0.6 if t == ops.TYPE_Q8_0 else 1.1) * step + 1e-6)
    # Position 0 and the channels past n_dims are the plain store's bytes.
    plain = oracle.kv_quantize(t, x.reshape(tokens, heads * head_dim))
    if not yarn:
        assert np.array_equal(stored[0], plain[0])


def test_rope_store_refusals(device):
    x = torch.zeros((2, 2, 64), dtype=torch.float32, device=device)
    pos = torch.zeros(2, dtype=torch.int32, device=device)
    ids = torch.arange(2, dtype=torch.int64, device=device)
    cache = torch.zeros((4, 2 * 2 * 34), dtype=torch.uint8, device=device)
    for bad in (dict(n_dims=65), dict(n_dims=33), dict(theta_scale=0.0)):
        args = dict(n_dims=64, theta_scale=0.9)
        args.update(bad)
        with pytest.raises(ops.KernelFailure):
            ops.rope_set_rows_quant(ops.TYPE_Q8_0, x, pos, ids, cache, args["n_dims"], args["theta_scale"])
    with pytest.raises(ops.KernelFailure):
        ops.rope_set_rows_quant(ops.TYPE_Q4_K, x, pos, ids, cache, 64, 0.9)
    with pytest.raises(ops.KernelFailure):  # rows would overlap
        ops.rope_set_rows_quant(ops.TYPE_Q8_0, x, pos, ids, torch.zeros((4, 100), dtype=torch.uint8, device=device), 64, 0.9)
    assert torch.count_nonzero(cache) == 0
