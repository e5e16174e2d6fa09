"""llmp_hip_exl3_linear_static, the entry point that allocates nothing (its partial sums live in a static device
array of the library): its output is bit for bit llmp_hip_exl3_linear's, on two calls in a row over the same
array, the second smaller, and a linear whose partial sums exceed the array is refused."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from conftest import rel_close
from llmp_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def halves(a, device):
    return dev(np.ascontiguousarray(a).view(np.int16), device).view(torch.float16)


def test_static_scratch_linear_equals_the_linear_on_two_calls_in_a_row(device):
    bits, codebook = 4, ops.EXL3_3INST
    cases = []
    for k, n, m, f32, seed in ((2048, 1024, 16, True, 91), (512, 256, 3, False, 92)):  # the second smaller
        trellis, suh, svh = synth.exl3_weights(k, n, bits, seed)
        x = synth.rng(seed + 10).standard_normal((m, k)).astype(np.float16)
        weights = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
        a_had = torch.zeros((m, k), dtype=torch.float16, device=device)
        y = torch.full((m, n), 7.0, dtype=torch.float32 if f32 else torch.float16, device=device)
        cases.append((weights, halves(x, device), a_had, y, f32, (trellis, suh, svh, x)))
    # The set-up that is no launch (the array's address, the kernels' LDS attribute) first: what it takes from the
    # runtime, a code object's load included, is taken here and not by the calls that are counted below.
    for weights, *_ in cases:
        ops.exl3_linear_static_prepare(*weights)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]  # hipMemGetInfo: sees what the library or the runtime would take too
    # Two calls in a row on one stream, sharing the device's static array; nothing is allocated between them.
    for weights, x, a_had, y, _, _ in cases:
        ops.exl3_linear_static(*weights, x, a_had, y)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    for weights, x, a_had, y, f32, host in cases:
        keep = {}
        want = ops.exl3_linear(*weights, x, f32=f32, keep=keep)
        word = torch.int32 if f32 else torch.int16
        assert torch.equal(y.view(word), want.view(word))
        assert torch.equal(a_had.view(torch.int16), keep["a_had"].view(torch.int16))
    # And against the oracle, stage two over the device's transformed input (accumulation order only).
    weights, x, a_had, y, _, (trellis, suh, svh, xh) = cases[0]
    want = oracle.exl3_product(trellis, svh.view(np.uint16), weights[3], weights[4], bits, codebook,
                               a_had.cpu().numpy().view(np.uint16), threads=oracle.max_threads())
    ok, worst = rel_close(y.cpu().numpy(), want, 1e-3)
    assert ok, worst
    # The second call again after the first: the array's leftovers from a larger call change nothing.
    weights, x, a_had, y, f32, _ = cases[1]
    first = y.clone()
    ops.exl3_linear_static(*cases[0][0], cases[0][1], cases[0][2], cases[0][3])
    ops.exl3_linear_static(*weights, x, a_had, y)
    torch.cuda.synchronize()
    assert torch.equal(first.view(torch.int16), y.view(torch.int16))


def test_static_scratch_linear_captured_in_a_graph_replays_bit_for_bit(device):
    """Prepared outside the capture, captured through the launch context's thread-local capture, replayed twice with
    a different x each time and eager work between: every replay is bit for bit the eager linear."""
    bits, codebook, k, n, m = 4, ops.EXL3_3INST, 1024, 512, 2
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 95)
    weights = (dev(trellis, device), halves(suh, device), halves(svh, device), k, n, bits, codebook)
    ops.exl3_linear_static_prepare(*weights)
    x = torch.zeros((m, k), dtype=torch.float16, device=device)
    a_had = torch.zeros((m, k), dtype=torch.float16, device=device)
    y = torch.zeros((m, n), dtype=torch.float32, device=device)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side, capture_error_mode="thread_local"):
        ops.exl3_linear_static(*weights, x, a_had, y)
    for seed in (96, 97):
        fresh = halves(synth.rng(seed).standard_normal((m, k)).astype(np.float16), device)
        x.copy_(fresh)
        want = ops.exl3_linear(*weights, fresh, f32=True)  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int32), want.view(torch.int32))


def test_static_scratch_linear_refuses_what_exceeds_its_array(device):
    lib = _lib.load()
    op = _lib.Exl3Linear()
    w = _lib.Exl3Weights()
    w.trellis, w.suh, w.svh, w.k, w.n, w.bits, w.codebook = 0x100000, 0x8000000, 0x9000000, 4096, 262144, 4, 0
    op.weights, op.x, op.a_had, op.y, op.f32, op.m = w, 0xA000000, 0xB000000, 0xC000000, 1, 16
    assert lib.llmp_hip_exl3_linear_scratch(C.byref(op)) > (4 << 20)
    assert lib.llmp_hip_exl3_linear_static(C.byref(op), None) == 1
    assert b"exceed the static area" in lib.llmp_hip_last_error()
    op.m = 65537  # and the linear's own refusals still hold
    w.n = 128
    op.weights = w
    assert lib.llmp_hip_exl3_linear_static(C.byref(op), None) == 1 and b"rows" in lib.llmp_hip_last_error()
