"""Parity of llmp.decode.vector, vector_glu and rows (HIP, through the C ABI) against the CPU oracle: every decoder,
1 to 16 input rows, row windows, strides, tensor scales, undefined block scales. Float outputs to
a maximum relative error of 1e-3 (the accumulation order is the only difference: both sides
decode every value exactly)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu

DECODERS = list(range(11))


def to_device(weight, device):
    out = dict(weight)
    for key in ("data", "scales", "tensor_scale"):
        if weight.get(key) is not None:
            out[key] = torch.from_numpy(np.ascontiguousarray(weight[key])).to(device)
    return out


@pytest.mark.parametrize("decoder", DECODERS)
@pytest.mark.parametrize("rows", [1, 3, 4, 9, 16])
def test_every_decoder_matches_oracle(device, decoder, rows):
    n, k = 133, 1024  # an odd number of output rows: the last wave's second row is a copy
    w = synth.decode_weight(decoder, n, k, 700 + decoder)
    x = synth.activations(rows, k, 710 + rows)
    want = oracle.decode_vector(decoder, w, x, threads=oracle.max_threads())
    got = ops.decode_vector(decoder, to_device(w, device), torch.from_numpy(x).to(device)).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, (oracle.DECODERS[decoder], worst)
    # An input row's outputs do not depend on the rows beside it (src/kernels/decode/products.h:33-35).
    alone = ops.decode_vector(decoder, to_device(w, device), torch.from_numpy(x[rows - 1:]).to(device)).cpu().numpy()
    assert np.array_equal(alone[0].view(np.uint32), got[rows - 1].view(np.uint32))


@pytest.mark.parametrize("decoder", [0, 3, 6, 8])
def test_windows_strides_and_tensor_scales(device, decoder):
    n, k, rows = 256, 512, 2
    w = synth.decode_weight(decoder, n, k, 720 + decoder, tensor_scales=4)
    x = synth.activations(rows, k, 721)
    wide = np.zeros((rows, k + 8), dtype=np.float32)
    wide[:, :k] = x
    xd = torch.from_numpy(wide).to(device)[:, :k]  # rows k + 8 floats apart
    want = oracle.decode_vector(decoder, w, x, first=60, outputs=77)
    got = ops.decode_vector(decoder, to_device(w, device), xd, first=60, outputs=77).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst
    # The tensor scale multiplies each output once: rows 64.. take the second scale.
    plain = dict(w)
    plain["tensor_scale"] = None
    bare = ops.decode_vector(decoder, to_device(plain, device), xd, first=60, outputs=77).cpu().numpy()
    scale = w["tensor_scale"][(60 + np.arange(77)) // w["rows_per_scale"]]
    assert np.array_equal((bare * scale).view(np.uint32), got.view(np.uint32))


def test_every_code_and_undefined_scales(device):
    """All 256 E4M3 codes and all 16 E2M1 codes against the oracle's values exactly (one nonzero input
    a row picks one weight value out); block scales the format leaves undefined are NaN
    (tests/unit/reference_decode_test.cc:407-484 of the reference)."""
    k = 256
    # mxfp8.split: row r holds code r at position r % k, scale 2^0; x is all ones.
    codes = np.zeros((256, k), dtype=np.uint8)
    codes[np.arange(256), np.arange(256) % k] = np.arange(256, dtype=np.uint8)
    w = {"k": k, "data": codes, "scales": np.full(256 * (k // 32), 127, dtype=np.uint8)}
    x = np.ones((1, k), dtype=np.float32)
    got = ops.decode_vector(7, to_device(w, device), torch.from_numpy(x).to(device)).cpu().numpy()[0]
    want = np.array([oracle.lib.orc_e4m3_to_f32(c) for c in range(256)], dtype=np.float32)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    keep = ~np.isnan(want)
    assert np.array_equal(got[keep], want[keep])
    # nvfp4.split: row r holds code r % 16 in nibble r of its first bytes, scale 0x38 (1.0).
    codes = np.zeros((32, k // 2), dtype=np.uint8)
    for r in range(32):
        codes[r, r // 2] = (r % 16) << (4 * (r % 2))
    scales = np.full((32, k // 16), 0x38, dtype=np.uint8)
    w = {"k": k, "data": codes, "scales": scales.reshape(-1)}
    got = ops.decode_vector(3, to_device(w, device), torch.from_numpy(x).to(device)).cpu().numpy()[0]
    want = np.array([oracle.lib.orc_e2m1_to_f32(r % 16) for r in range(32)], dtype=np.float32)
    assert np.array_equal(got, want)
    # Undefined scales: UE4M3 from 0x7F up, E8M0 0xFF.
    for decoder, bad in ((3, 0x7F), (3, 0x80), (3, 0xFF), (6, 0xB8), (9, 0xFF), (7, 0xFF)):
        w = synth.decode_weight(decoder, 4, k, 730 + decoder)
        if decoder == 6:
            w["data"][2, 1] = bad  # row 2's second sub-block scale
        else:
            w["scales"] = w["scales"].copy()
            blocks = k // (16 if decoder == 3 else 32)
            w["scales"][2 * blocks + 1] = bad
        got = ops.decode_vector(decoder, to_device(w, device), torch.from_numpy(synth.activations(1, k, 731)).to(device))
        got = got.cpu().numpy()[0]
        assert np.isnan(got[2]) and np.all(np.isfinite(got[[0, 1, 3]])), (decoder, bad, got)


def test_long_rows_take_fewer_input_rows_a_launch(device):
    n, k, rows = 12, 8192, 7  # two input rows a launch at this length
    w = synth.decode_weight(9, n, k, 740)
    x = synth.activations(rows, k, 741)
    want = oracle.decode_vector(9, w, x, threads=oracle.max_threads())
    got = ops.decode_vector(9, to_device(w, device), torch.from_numpy(x).to(device)).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst


def test_refusals(device):
    w = to_device(synth.decode_weight(3, 8, 256, 750), device)
    x = torch.zeros((17, 256), dtype=torch.float32, device=device)
    with pytest.raises(ops.KernelFailure) as e:
        ops.decode_vector(3, w, x)
    assert e.value.rejected
    with pytest.raises(ops.KernelFailure):  # an affine operand without its group, width and scale type
        ops.decode_vector(11, w, x[:1])
    with pytest.raises(ops.KernelFailure):  # rows [6, 10) of 8
        ops.decode_vector(3, w, x[:1], first=6, outputs=4)
    with pytest.raises(ops.KernelFailure):  # scale atoms take k in whole 64 values
        ops.decode_vector(4, to_device(synth.decode_weight(3, 8, 32, 751), device), x[:1, :32])


@pytest.mark.parametrize("decoder", [0, 2, 6, 8, 9])
@pytest.mark.parametrize("glu", [0, 1, 2, 3])
@pytest.mark.parametrize("rows", [1, 5])
def test_vector_glu_matches_oracle(device, decoder, glu, rows):
    """RunVectorGlu (src/kernels/decode/products.h:120-139 of the reference): the four GLUs of
    src/kernels/decode/templates.cuh:73-90 over a gate and an up weight with their own tensor scales."""
    n, k = 96, 512
    gate = synth.decode_weight(decoder, n, k, 760 + decoder, tensor_scales=2)
    up = synth.decode_weight(decoder, n, k, 770 + decoder, tensor_scales=3)
    x = synth.activations(rows, k, 780 + rows) * 0.25
    limit = 1.5 if glu == 3 else 0.0
    want = oracle.decode_vector_glu(decoder, gate, up, x, glu, limit, gate_first=8, up_first=3, outputs=70)
    got = ops.decode_vector_glu(decoder, to_device(gate, device), to_device(up, device), torch.from_numpy(x).to(device),
                                glu, limit, gate_first=8, up_first=3, outputs=70).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, (oracle.DECODERS[decoder], glu, worst)
    # The two sums are the plain products': SwiGLU of llmp.decode.vector's outputs, to float rounding.
    g = ops.decode_vector(decoder, to_device(gate, device), torch.from_numpy(x).to(device), first=8, outputs=70)
    u = ops.decode_vector(decoder, to_device(up, device), torch.from_numpy(x).to(device), first=3, outputs=70)
    if glu == 0:
        silu = g / (1.0 + torch.exp(-g)) * u
        np.testing.assert_allclose(got, silu.cpu().numpy(), rtol=2e-6, atol=1e-9)


def test_vector_glu_of_one_stacked_weight_and_refusals(device):
    n, k = 64, 256
    w = synth.decode_weight(3, 2 * n, k, 790)  # gate rows, then up rows, in one weight
    x = synth.activations(2, k, 791) * 0.25
    want = oracle.decode_vector_glu(3, w, w, x, 0, gate_first=0, up_first=n, outputs=n)
    wd = to_device(w, device)
    xd = torch.from_numpy(x).to(device)
    got = ops.decode_vector_glu(3, wd, wd, xd, 0, gate_first=0, up_first=n, outputs=n).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst
    with pytest.raises(ops.KernelFailure):  # an unknown GLU
        ops.decode_vector_glu(3, wd, wd, xd, 4, outputs=n)
    with pytest.raises(ops.KernelFailure):  # up rows [100, 164) of 128
        ops.decode_vector_glu(3, wd, wd, xd, 0, up_first=100, outputs=n)
    with pytest.raises(ops.KernelFailure):  # a gate and an up of two decoders that are no pair the reference builds
        ops.decode_vector_glu(3, wd, to_device(synth.decode_weight(9, n, k, 792), device), xd, 0, outputs=n, up_decoder=9)


@pytest.mark.parametrize("gate_decoder,up_decoder", [(7, 0), (3, 2), (3, 0), (9, 0), (9, 2), (11, 0)])
@pytest.mark.parametrize("rows", [1, 6])
def test_vector_glu_of_two_decoders(device, gate_decoder, up_decoder, rows):
    """The six mixed pairs the reference instantiates (src/kernels/decode/implementations.cc:73-81): a block-scaled or
    affine gate with a BF16 or Q8_0 up, each weight decoded by its own decoder, against the oracle."""
    n, k = 80, 512
    gate = synth.affine_weight(n, k, 806, bits=4, group=64, tensor_scales=2) if gate_decoder == 11 else \
        synth.decode_weight(gate_decoder, n, k, 795 + gate_decoder, tensor_scales=2)
    up = synth.decode_weight(up_decoder, n, k, 796 + up_decoder)
    x = synth.activations(rows, k, 797 + rows) * 0.25
    for glu in (0, 2):
        want = oracle.decode_vector_glu(gate_decoder, gate, up, x, glu, gate_first=5, up_first=2, outputs=64, up_decoder=up_decoder)
        on = lambda w: {key: (torch.from_numpy(np.ascontiguousarray(v)).to(device) if isinstance(v, np.ndarray) else v) for key, v in w.items()}
        got = ops.decode_vector_glu(gate_decoder, on(gate), on(up), torch.from_numpy(x).to(device), glu,
                                    gate_first=5, up_first=2, outputs=64, up_decoder=up_decoder).cpu().numpy()
        ok, worst = rel_close(got, want, 1e-3)
        assert ok, (gate_decoder, up_decoder, glu, worst)


@pytest.mark.parametrize("decoder", DECODERS)
def test_rows_gather_is_the_decoded_rows_bit_for_bit(device, decoder):
    """RunRows (src/kernels/decode/products.h:172-183 of the reference): rows by index as F32, times their tensor
    scale; an id outside the matrix writes zeros and raises the flag."""
    n, k = 40, 512
    w = synth.decode_weight(decoder, n, k, 800 + decoder, tensor_scales=4)
    dense = oracle.decode_rows_of(decoder, w) * w["tensor_scale"][np.arange(n) // w["rows_per_scale"]][:, None]
    ids = np.array([3, 39, 0, 17, 17, 8, 25], dtype=np.int32)
    bad = torch.zeros(1, dtype=torch.int32, device=device)
    got = ops.decode_rows(decoder, to_device(w, device), torch.from_numpy(ids).to(device), bad=bad).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), dense[ids].astype(np.float32).view(np.uint32))
    assert int(bad.item()) == 0
    ids = np.array([5, -1, 40, 12], dtype=np.int32)
    got = ops.decode_rows(decoder, to_device(w, device), torch.from_numpy(ids).to(device), bad=bad).cpu().numpy()
    assert int(bad.item()) == 1
    assert np.all(got[1] == 0) and np.all(got[2] == 0)
    assert np.array_equal(got[[0, 3]].view(np.uint32), dense[[5, 12]].astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("scale", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("zero_point", [False, True])
def test_affine_decoder(device, bits, scale, zero_point):
    """affine.split (src/kernels/decode/decoders.cuh:241-345 of the reference): rows gathered bit for bit, the
    vector product and its GLU form to 1e-3."""
    n, k, group = 66, 1024, 64 if bits == 4 else 128
    w = synth.affine_weight(n, k, 810 + bits, bits=bits, group=group, scale=scale, zero_point=zero_point, tensor_scales=2)
    wd = {key: (torch.from_numpy(np.ascontiguousarray(v)).to(device) if isinstance(v, np.ndarray) else v) for key, v in w.items()}
    dense = oracle.decode_rows_of(11, w) * w["tensor_scale"][np.arange(n) // w["rows_per_scale"]][:, None]
    ids = torch.arange(n, dtype=torch.int32, device=device)
    got = ops.decode_rows(11, wd, ids).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), dense.astype(np.float32).view(np.uint32))
    x = synth.activations(3, k, 811)
    xd = torch.from_numpy(x).to(device)
    ok, worst = rel_close(ops.decode_vector(11, wd, xd).cpu().numpy(), oracle.decode_vector(11, w, x), 1e-3)
    assert ok, worst
    want = oracle.decode_vector_glu(11, w, w, x * 0.25, 2, gate_first=0, up_first=33, outputs=33)
    got = ops.decode_vector_glu(11, wd, wd, xd * 0.25, 2, gate_first=0, up_first=33, outputs=33).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, worst


@pytest.mark.parametrize("decoder", [0, 3, 6, 8, 11])
def test_grouped_products_match_oracle(device, decoder):
    """RunGrouped (src/kernels/decode/products.h:141-170 of the reference): an expert worklist with empty experts,
    experts of one to nine pairs, output rows by pair or by pair_out, and what the device skips: an operand of
    another K, pairs naming rows outside x or y (their output rows stay as they were)."""
    experts, n, k = 7, 48, 512
    make = (lambda seed: synth.affine_weight(n, k, seed, bits=4, group=64)) if decoder == 11 else \
           (lambda seed: synth.decode_weight(decoder, n, k, seed, tensor_scales=2))
    weights = [make(820 + e) for e in range(experts)]
    weights[5] = (synth.affine_weight(n, 256, 830, bits=4, group=64) if decoder == 11
                  else synth.decode_weight(decoder, n, 256, 830))  # another K: skipped
    counts = [3, 0, 9, 1, 4, 2, 5]
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    pairs = int(offsets[-1])
    g = synth.rng(831)
    x = synth.activations(10, k, 832)
    pair_rows = g.integers(0, 10, size=pairs).astype(np.int32)
    pair_rows[4] = 10   # past x_rows: skipped
    pair_out = g.permutation(pairs + 3)[:pairs].astype(np.int32)
    pair_out[7] = pairs + 3  # past y_rows: skipped
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    dev_weights = [{key: (to_dev(v) if isinstance(v, np.ndarray) else v) for key, v in w.items() if key != "plain"}
                   for w in weights]
    for out in (None, pair_out):
        rows_y = pairs if out is None else pairs + 3
        want = np.full((rows_y, n), 7.0, dtype=np.float32)
        oracle.decode_grouped(decoder, weights, k, n, offsets, pair_rows, x, want, pair_out=out)
        y = torch.full((rows_y, n), 7.0, dtype=torch.float32, device=device)
        ops.decode_grouped(decoder, dev_weights, k, n, to_dev(offsets), to_dev(pair_rows), to_dev(x), y,
                           pair_out=None if out is None else to_dev(out))
        got = y.cpu().numpy()
        untouched = want == 7.0
        assert np.array_equal(got == 7.0, untouched)
        ok, worst = rel_close(got[~untouched], want[~untouched], 1e-3)
        assert ok, worst
    # A window of output rows.
    want = np.zeros((pairs, 20), dtype=np.float32)
    oracle.decode_grouped(decoder, weights, k, n, offsets, pair_rows, x, want, first=9, outputs=20)
    y = torch.zeros((pairs, 20), dtype=torch.float32, device=device)
    ops.decode_grouped(decoder, dev_weights, k, n, to_dev(offsets), to_dev(pair_rows), to_dev(x), y, first=9, outputs=20)
    ok, worst = rel_close(y.cpu().numpy(), want, 1e-3)
    assert ok, worst


@pytest.mark.parametrize("decoder", list(range(11)) + [11])
@pytest.mark.parametrize("rows", [1, 17, 130])
def test_matrix_products_match_oracle(device, decoder, rows):
    """RunMatrix's tensor-core path (src/kernels/decode/products.h:27-33, 111-118 of the reference): weights and inputs
    rounded to the decoder's matrix element, F32 sums; partial tiles of outputs, input rows and K."""
    n, k = 150, 608 if decoder in (0, 1, 3, 5, 11) else 640  # 608 = 9.5 chunks of 64 where the decoder's K allows
    w = synth.affine_weight(n, k, 840, bits=8, group=32, scale="bf16") if decoder == 11 else \
        synth.decode_weight(decoder, n, k, 840 + decoder, tensor_scales=3)
    x = synth.activations(rows, k, 841 + rows)
    wd = {key: (torch.from_numpy(np.ascontiguousarray(v)).to(device) if isinstance(v, np.ndarray) else v)
          for key, v in w.items() if key != "plain"}
    want = oracle.decode_matrix(decoder, w, x, first=7, outputs=139, threads=oracle.max_threads())
    got = ops.decode_matrix(decoder, wd, torch.from_numpy(x).to(device), first=7, outputs=139).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, (oracle.DECODERS[decoder], worst)
    # Against the vector product (F32 inputs): the rounding of the inputs to BF16 or F16 is all that differs.
    if rows == 1:
        plain = ops.decode_vector(decoder, wd, torch.from_numpy(x).to(device), first=7, outputs=139).cpu().numpy()
        assert np.abs(got - plain).max() <= 2e-2 * np.abs(plain).max()


@pytest.mark.parametrize("decoder", list(range(12)))
def test_matrix_large_tiles_match_oracle(device, decoder):
    """Enough outputs and input rows for the tiles of 256 outputs by 128 input rows, with partial tiles of
    both and of K (src/kernels/decode/products.h:111-118 of the reference)."""
    n, rows = 2100, 3700
    k = 160 if decoder in (0, 1, 3, 5, 11) else 256 if decoder in (8, 10) else 192  # 2.5, 4 or 3 chunks of 64
    w = synth.affine_weight(n, k, 860, bits=4, group=32, scale="f16") if decoder == 11 else \
        synth.decode_weight(decoder, n, k, 860 + decoder, tensor_scales=5)
    x = synth.activations(rows, k, 861)
    wd = {key: (torch.from_numpy(np.ascontiguousarray(v)).to(device) if isinstance(v, np.ndarray) else v)
          for key, v in w.items() if key != "plain"}
    want = oracle.decode_matrix(decoder, w, x, first=7, outputs=2060, threads=oracle.max_threads())
    got = ops.decode_matrix(decoder, wd, torch.from_numpy(x).to(device), first=7, outputs=2060).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, (oracle.DECODERS[decoder], worst)


@pytest.mark.parametrize("decoder", list(range(12)))
def test_matrix_tall_tiles_match_oracle(device, decoder):
    """Enough outputs and input rows for a tile of 256 outputs by 256 input rows on every compute unit (17 by 16
    tiles), with partial tiles of both and of K."""
    n, rows = 4140, 3900
    k = 160 if decoder in (0, 1, 3, 5, 11) else 256 if decoder in (8, 10) else 192
    w = synth.affine_weight(n, k, 880, bits=4, group=32, scale="f16") if decoder == 11 else \
        synth.decode_weight(decoder, n, k, 880 + decoder, tensor_scales=5)
    x = synth.activations(rows, k, 881)
    wd = {key: (torch.from_numpy(np.ascontiguousarray(v)).to(device) if isinstance(v, np.ndarray) else v)
          for key, v in w.items() if key != "plain"}
    want = oracle.decode_matrix(decoder, w, x, first=7, outputs=4100, threads=oracle.max_threads())
    got = ops.decode_matrix(decoder, wd, torch.from_numpy(x).to(device), first=7, outputs=4100).cpu().numpy()
    ok, worst = rel_close(got, want, 1e-3)
    assert ok, (oracle.DECODERS[decoder], worst)


def test_matrix_refusals(device):
    w = to_device(synth.decode_weight(3, 8, 256, 850), device)
    x = torch.zeros((4, 256), dtype=torch.float32, device=device)
    with pytest.raises(ops.KernelFailure):  # the FMA path is for devices without matrix cores
        ops.decode_matrix(3, w, x, path=1)
    with pytest.raises(ops.KernelFailure):
        ops.decode_matrix(3, w, x, first=6, outputs=4)
