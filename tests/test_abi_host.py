"""The C-ABI library without a GPU: it loads, exports every symbol include/llmp_hip.h declares,
and its host-side checks refuse bad launches before anything is queued (no GPU call is reached:
tests/unit/dsv4_fast_test.cc:391-399 of the reference checks the same on its device)."""
import ctypes as C
import os
import re

import pytest

from llmp_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="llmp_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llmp_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), name
        assert name in _lib.SYMBOLS, f"{name} has no ctypes signature"
    assert sorted(_lib.SYMBOLS) == names


def test_library_exports_the_provider_and_launch_context():
    """include/llmp_hip_launch.h: bound from C++ (include/llmp_hip_launch.hpp), so exported names are what is checked."""
    lib = _lib.load()
    names = declared_symbols("llmp_hip_launch.h")
    assert len(names) >= 35
    for name in names:
        assert hasattr(lib, name), name


def test_library_exports_the_memory_provider():
    """include/llmp_hip_memory.h: bound from C++ (include/llmp_hip_memory.hpp), so exported names are what is checked."""
    lib = _lib.load()
    names = declared_symbols("llmp_hip_memory.h")
    assert len(names) >= 21
    for name in names:
        assert hasattr(lib, name), name


def test_variant_table_is_named():
    lib = _lib.load()
    n = lib.llmp_hip_vecq_variants()
    assert n >= 4
    names = [lib.llmp_hip_vecq_variant_name(i).decode() for i in range(n)]
    assert len(set(names)) == n and lib.llmp_hip_vecq_variant_name(-1) == b"default"


def desc(**kw):
    d = _lib.VecQDesc()
    base = dict(w=0x1000, g=None, y=0x2000, ids=None, dst=0x3000, ncols_x=512, nrows=8, stride_row=2, stride_expert=0,
                y_token=16, y_slot=0, ids_stride=0, used=1, tokens=1, dst_token=8, dst_slot=0, glu=0, limit=0.0)
    base.update(kw)
    for k, v in base.items():
        setattr(d, k, v)
    return d


@pytest.mark.parametrize("t,kw,why", [
    (12, dict(ncols_x=500), "whole"),
    (12, dict(tokens=17), "tokens"),
    (12, dict(tokens=0), "tokens"),
    (12, dict(glu=3), "gate"),
    (12, dict(g=0x4000, glu=0), "gate"),
    (12, dict(g=0x4000, glu=3, limit=1.0), "GeGLU"),
    (12, dict(ids=0x5000, used=16, tokens=16), "pairs"),
    (12, dict(w=None), "null"),
    (12, dict(w=0x1008), "aligned"),
    (12, dict(dst=0x3002), "aligned"),
    (12, dict(stride_row=1), "overlap"),
    (8, dict(ncols_x=48), "whole"),
    (8, dict(w=0x1001, stride_row=16), "aligned"),
    (4, dict(), "type"),
    (39, dict(ncols_x=768, stride_row=24), "MXFP4"),
    (39, dict(ncols_x=512, stride_row=24), "MXFP4"),
    (39, dict(w=0x1004, stride_row=16), "MXFP4"),
    (2, dict(ncols_x=288, stride_row=9), "Q4_0"),
    (20, dict(ncols_x=288, stride_row=9), "IQ4_NL"),
    (13, dict(w=0x1008), "Q5_K"),
    (14, dict(ncols_x=3840, stride_row=15, nrows=3), "Q6_K"),
    (13, dict(ncols_x=288), "whole"),
    (12, dict(used=300), "slots"),
])
def test_vecq_refusals_queue_nothing(t, kw, why):
    lib = _lib.load()
    code = lib.llmp_hip_vecq(t, C.byref(desc(**kw)), -1, None)
    assert code > 0
    assert why in lib.llmp_hip_last_error().decode()


def test_other_entry_points_refuse_bad_operands():
    lib = _lib.load()
    assert lib.llmp_hip_vecq(12, None, -1, None) > 0
    assert lib.llmp_hip_vecq(12, C.byref(desc()), 99, None) > 0
    # The flat form takes Q8_0 rows of whole 256 values at 16-byte boundaries only; the matrix-core form Q8_0 rows
    # of whole 128 values, an even number of blocks apart.
    assert lib.llmp_hip_vecq(8, C.byref(desc(ncols_x=480, stride_row=15)), 6, None) > 0
    assert lib.llmp_hip_vecq(8, C.byref(desc(stride_row=17)), 6, None) > 0
    assert lib.llmp_hip_vecq(8, C.byref(desc(ncols_x=480, stride_row=16, tokens=4)), 9, None) > 0
    assert lib.llmp_hip_vecq(8, C.byref(desc(stride_row=17, tokens=4)), 9, None) > 0
    assert lib.llmp_hip_vecq(4, C.byref(desc(tokens=4)), 9, None) > 0
    assert lib.llmp_hip_vecq_fused(12, C.byref(desc()), None, -1, None) > 0
    assert lib.llmp_hip_vecq_block_sums(12, C.byref(desc()), -1, None, None) > 0
    assert lib.llmp_hip_q8_1_quantize(None, None, 32, 512, 32, 1, 1, 32, None) > 0
    assert lib.llmp_hip_q8_1_quantize(0x1000, 0x2000, 600, 512, 600, 1, 1, 600, None) > 0
    assert lib.llmp_hip_moe_router(0x1000, 2000, 8, 1, 1, 1.0, 0x2000, 0x3000, None) > 0
    assert lib.llmp_hip_moe_router(0x1000, 128, 0, 1, 1, 1.0, 0x2000, 0x3000, None) > 0
    assert lib.llmp_hip_moe_combine(0x1000, 0x2000, None, 6, 8, 1, 0x3000, None) > 0
    assert lib.llmp_hip_moe_route(None, 8, 128, 8, 1, 0x1000, None) > 0
    assert lib.llmp_hip_vecq_sorted(8, C.byref(desc(ncols_x=480, stride_row=15)), 0x1000, 4, -1, None) > 0
    assert lib.llmp_hip_moe_route_ints(128, 8, 512) == 2 * 129 + 3 * 4096 + 8 * 128


def test_exl3_linears_refuse_bad_operands():
    lib = _lib.load()

    def weights(k=128, n=128, bits=4, trellis=0x1000):
        w = _lib.Exl3Weights()
        w.trellis, w.suh, w.svh, w.k, w.n, w.bits, w.codebook = trellis, 0x2000, 0x3000, k, n, bits, 0
        return w

    one = _lib.Exl3Linear()
    one.weights, one.x, one.a_had, one.y, one.f32, one.m = weights(), 0x4000, 0x5000, 0x6000, 1, 65537
    assert lib.llmp_hip_exl3_linear(C.byref(one), 0x7000, 1 << 30, None) > 0 and b"rows" in lib.llmp_hip_last_error()
    two = _lib.Exl3MultiLinear()
    two.first, two.second = weights(), weights(bits=3)
    two.x, two.a_had, two.y, two.f32, two.m = 0x4000, 0x5000, 0x6000, 1, 2
    assert lib.llmp_hip_exl3_multi_linear(C.byref(two), 0x7000, 1 << 30, None) > 0
    assert b"share" in lib.llmp_hip_last_error()
    two.second = weights(n=256)
    assert lib.llmp_hip_exl3_multi_linear(C.byref(two), 0x7000, 1 << 30, None) > 0
    two.second = weights()
    assert lib.llmp_hip_exl3_multi_linear(C.byref(two), 0x7000, 8, None) > 0 and b"scratch" in lib.llmp_hip_last_error()
    assert lib.llmp_hip_exl3_multi_linear_scratch(C.byref(two)) == 2 * lib.llmp_hip_exl3_linear_scratch(C.byref(one)) // 16 * 2


def test_default_descriptors_are_refused_before_any_plan():
    """A default-constructed descriptor (k = 0) through the block sums and the sorted rows: refused by the
    descriptor's checks, for every type, before a plan divides by the row's units."""
    lib = _lib.load()
    empty = _lib.VecQDesc()
    for t in (2, 3, 6, 7, 8, 12, 13, 14, 20, 39):
        assert lib.llmp_hip_vecq_block_sums(t, C.byref(empty), -1, 0x1000, None) > 0
        assert lib.llmp_hip_vecq_sorted(t, C.byref(empty), 0x1000, 4, -1, None) > 0
        nearly = desc(ncols_x=0)
        assert lib.llmp_hip_vecq_block_sums(t, C.byref(nearly), -1, 0x1000, None) > 0
        assert lib.llmp_hip_vecq_sorted(t, C.byref(nearly), 0x1000, 4, -1, None) > 0
        assert b"whole" in lib.llmp_hip_last_error()


def test_exl3_refuses_overlapping_operands():
    """src/kernels/exl3/validate.cc:32-62 and 120-126 of the reference: a written range that meets another
    operand is refused before anything is queued."""
    lib = _lib.load()

    def weights(trellis=0x100000, suh=0x200000, svh=0x210000):
        w = _lib.Exl3Weights()
        w.trellis, w.suh, w.svh, w.k, w.n, w.bits, w.codebook = trellis, suh, svh, 128, 128, 4, 0
        return w

    def linear(**kw):
        op = _lib.Exl3Linear()
        base = dict(x=0x300000, a_had=0x310000, y=0x320000, f32=1, m=2)
        base.update(kw)
        op.weights = weights()
        for k, v in base.items():
            setattr(op, k, v)
        return op

    scratch = 0x400000
    cases = [(dict(y=0x300000), b"y overlaps x"), (dict(a_had=0x300000), b"a_had overlaps x"),
             (dict(a_had=0x320000), b"a_had overlaps y"), (dict(y=0x100000 + 64), b"y overlaps the trellis"),
             (dict(y=0x200000), b"y overlaps suh"), (dict(a_had=0x210000), b"a_had overlaps svh"),
             (dict(y=scratch + 8), b"y overlaps the scratch"), (dict(x=scratch), b"the scratch overlaps x")]
    for kw, why in cases:
        op = linear(**kw)
        assert lib.llmp_hip_exl3_linear(C.byref(op), scratch, 1 << 20, None) > 0, kw
        assert why in lib.llmp_hip_last_error(), (kw, lib.llmp_hip_last_error())
    two = _lib.Exl3MultiLinear()
    two.first, two.second = weights(), weights(trellis=0x500000)
    two.x, two.a_had, two.y, two.f32, two.m = 0x300000, 0x310000, 0x310000 + 2 * 2 * 128 * 2 - 8, 1, 2
    assert lib.llmp_hip_exl3_multi_linear(C.byref(two), scratch, 1 << 20, None) > 0
    assert b"a_had overlaps y" in lib.llmp_hip_last_error()
    two.y = 0x500000 + 32
    assert lib.llmp_hip_exl3_multi_linear(C.byref(two), scratch, 1 << 20, None) > 0
    assert b"y overlaps the trellis" in lib.llmp_hip_last_error()
    w = weights()
    assert lib.llmp_hip_exl3_reconstruct(C.byref(w), 0x100000 + 4096, 0, 16, None) > 0
    assert b"w overlaps the trellis" in lib.llmp_hip_last_error()
    # The transform: in place for F16 only; otherwise x, y and the scale apart.
    assert lib.llmp_hip_exl3_hadamard(0x1000, 0x1000, 0x8000, 2, 128, 1, 0, None) > 0
    assert lib.llmp_hip_exl3_hadamard(0x1000, 0x1100, 0x8000, 2, 128, 0, 0, None) > 0 and b"y overlaps x" in lib.llmp_hip_last_error()
    assert lib.llmp_hip_exl3_hadamard(0x1000, 0x8000 + 64, 0x8000, 2, 128, 0, 0, None) > 0
    assert b"y overlaps the scale" in lib.llmp_hip_last_error()


def test_set_rows_quant_refuses_a_destination_over_its_operands():
    lib = _lib.load()
    store = lambda **kw: lib.llmp_hip_set_rows_quant(kw.get("t", 8), kw.get("x", 0x10000), 64, kw.get("ids", 0x20000), 4,
                                                     kw.get("dst", 0x30000), 68, 64, 4, kw.get("cells", 16), None)
    assert store(cells=0) > 0 and b"no cells" in lib.llmp_hip_last_error()
    assert store(dst=0x10000 + 512) > 0 and b"overlaps" in lib.llmp_hip_last_error()
    assert store(dst=0x20000 - 68 * 16 + 2) > 0 and b"overlaps" in lib.llmp_hip_last_error()
    assert store(t=12) > 0 and b"Q8_0 or Q4_0" in lib.llmp_hip_last_error()


def test_decode_vector_refuses_bad_operands():
    lib = _lib.load()

    def operand(**kw):
        w = _lib.DecodeOperand()
        base = dict(data=0x1000, scales=0x2000, tensor_scale=None, biases=None, k=256, rows=64, rows_per_scale=64,
                    row_bytes=128)
        base.update(kw)
        for name, value in base.items():
            setattr(w, name, value)
        return w

    def run(decoder, w, first=0, outputs=8, x=0x4000, rows=1, x_stride=256, y=0x5000, y_stride=64):
        return lib.llmp_hip_decode_vector(decoder, C.byref(w), first, outputs, x, rows, x_stride, y, y_stride, None)

    assert run(12, operand()) > 0 and b"no kernel" in lib.llmp_hip_last_error()
    assert run(11, operand()) > 0 and b"affine" in lib.llmp_hip_last_error()           # no group, width or scale type
    assert run(3, operand(), rows=17) > 0 and b"1 to 16" in lib.llmp_hip_last_error()
    assert run(3, operand(), first=60, outputs=8) > 0
    assert run(3, operand(scales=None)) > 0 and b"scales" in lib.llmp_hip_last_error()
    assert run(4, operand(k=32, row_bytes=16)) > 0 and b"multiple" in lib.llmp_hip_last_error()
    assert run(7, operand(data=0x1008, row_bytes=256)) > 0 and b"aligned" in lib.llmp_hip_last_error()
    assert run(3, operand(), x=0x4004) > 0
    assert run(3, operand(), x_stride=258) > 0
    assert run(9, operand(k=32768, row_bytes=16384), x_stride=32768) > 0 and b"staging" in lib.llmp_hip_last_error()
    gate, up = operand(), operand(k=512, row_bytes=256)
    glu = lambda gd, ud, kind: lib.llmp_hip_decode_vector_glu(gd, C.byref(gate), 0, ud, C.byref(up), 0, 8, kind, 0.0,
                                                              0x4000, 1, 512, 0x5000, 64, None)
    assert glu(3, 3, 0) > 0 and b"differ" in lib.llmp_hip_last_error()            # K 256 against 512
    assert glu(3, 9, 0) > 0 and b"no instantiation" in lib.llmp_hip_last_error()  # mixed decoders
    up = operand()
    assert glu(3, 3, 7) > 0 and b"GLU" in lib.llmp_hip_last_error()
    rows = lambda **kw: lib.llmp_hip_decode_rows(kw.get("decoder", 3), C.byref(operand()), kw.get("ids", 0x6000),
                                                 kw.get("count", 4), kw.get("out", 0x7000), kw.get("stride", 256), None, None)
    assert rows(decoder=12) > 0 and rows(ids=None) > 0 and rows(count=0) > 0 and rows(out=0x7004) > 0 and rows(stride=250) > 0


def test_decode_grouped_refuses_bad_operands():
    lib = _lib.load()

    def run(decoder=3, experts=0x1000, count=4, k=256, n=64, first=0, outputs=64, offsets=0x2000, rows=0x3000,
            pairs=8, x=0x4000, x_stride=256, y=0x5000, y_stride=64):
        return lib.llmp_hip_decode_grouped(decoder, experts, count, k, n, first, outputs, offsets, rows, None, pairs, x,
                                           16, x_stride, y, 8, y_stride, 0, None)

    assert run(decoder=12) > 0 and b"no kernel" in lib.llmp_hip_last_error()
    assert run(experts=None) > 0 and run(count=0) > 0 and run(pairs=0) > 0
    assert run(decoder=4, k=32) > 0 and b"multiple" in lib.llmp_hip_last_error()
    assert run(first=60, outputs=8) > 0 and b"outputs" in lib.llmp_hip_last_error()
    assert run(x=0x4004) > 0 and run(x_stride=250) > 0
    assert run(k=32768, x_stride=32768) > 0 and b"staging" in lib.llmp_hip_last_error()


def test_decode_matrix_refuses_bad_operands():
    lib = _lib.load()
    w = _lib.DecodeOperand()
    w.data, w.scales, w.k, w.rows, w.rows_per_scale, w.row_bytes = 0x1000, 0x2000, 256, 64, 64, 128
    run = lambda **kw: lib.llmp_hip_decode_matrix(kw.get("decoder", 3), C.byref(w), kw.get("first", 0), kw.get("outputs", 8),
                                                  kw.get("x", 0x4000), kw.get("rows", 100), kw.get("x_stride", 256), 0x5000,
                                                  64, kw.get("path", 0), None)
    assert run(path=1) > 0 and b"FMA" in lib.llmp_hip_last_error()
    assert run(rows=0) > 0 and run(decoder=12) > 0 and run(first=60) > 0 and run(x=0x4004) > 0 and run(x_stride=100) > 0


def test_grouped_store_refusals_queue_nothing():
    lib = _lib.load()
    table = (_lib.SetRowsStore * 2)()
    for i, entry in enumerate(table):
        entry.type, entry.index_bytes, entry.x, entry.x_stride, entry.ids = 8, 4, 0x10000, 64, 0x20000
        entry.destination, entry.row_bytes, entry.k, entry.rows, entry.cells = 0x30000 + 0x1000 * i, 68, 64, 4, 8
    assert lib.llmp_hip_set_rows_quant_group(1, table, None) > 0 and b"two through sixteen" in lib.llmp_hip_last_error()
    assert lib.llmp_hip_set_rows_quant_group(2, None, None) > 0
    table[1].destination = 0x30000 + 100  # inside the first store's 8 x 68 bytes
    assert lib.llmp_hip_set_rows_quant_group(2, table, None) > 0 and b"overlaps" in lib.llmp_hip_last_error()
    table[1].destination = 0x10000  # on the first store's values
    assert lib.llmp_hip_set_rows_quant_group(2, table, None) > 0 and b"overlaps" in lib.llmp_hip_last_error()
    table[1].destination, table[1].k = 0x40000, 48
    assert lib.llmp_hip_set_rows_quant_group(2, table, None) > 0 and b"whole 32-value blocks" in lib.llmp_hip_last_error()


def test_rope_store_refusals_queue_nothing():
    lib = _lib.load()
    s = _lib.RopeStore(type=8, heads=2, head_dim=64, n_dims=64, x=0x10000, x_head_stride=64, x_token_stride=128,
                       pos=0x20000, freq_factors=None, ids=0x30000, destination=0x40000, row_bytes=136, tokens=3,
                       freq_scale=1.0, ext_factor=0.0, attn_factor=1.0, theta_scale=0.9)
    for field, value, why in (("n_dims", 66, b"rotated dims"), ("head_dim", 48, b"whole 32-value blocks"),
                              ("row_bytes", 100, b"overlap"), ("type", 12, b"Q8_0 or Q4_0"), ("pos", None, b"null"),
                              ("theta_scale", 0.0, b"positive")):
        old = getattr(s, field)
        setattr(s, field, value)
        assert lib.llmp_hip_rope_set_rows_quant(C.byref(s), None) > 0 and why in lib.llmp_hip_last_error(), field
        setattr(s, field, old)
    assert lib.llmp_hip_rope_set_rows_quant(None, None) > 0
