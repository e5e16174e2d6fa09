"""Every operation only queues kernels on the caller's stream, so a step can be captured in a
HIP graph and replayed (the reference's launch contexts capture their steps,
src/kernels/ggml/launch.h:34-48; its tests replay and compare, tests/unit/dsv4_fast_test.cc:
376-389): each replay, with eager work and synchronizations in between, must give the eager
result bit for bit."""
import numpy as np
import pytest
import torch

from llmp_amd import ops, synth

pytestmark = pytest.mark.gpu


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def replayed_equals_eager(device, step, inputs):
    """`step()` returns a tensor computed from `inputs` (device tensors it reads). Captured once,
    replayed three times over changed inputs, compared with eager runs over the same inputs."""
    originals = [t.clone() for t in inputs]
    eager_first = step().clone()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        step()  # warm the launch paths outside the capture
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        out = step()
    for round_ in range(3):
        # Change the inputs in place (the graph reads the same addresses), run other work eagerly.
        for t, original in zip(inputs, originals):
            if t.dtype in (torch.float32, torch.float16, torch.bfloat16):
                t.copy_(original * (1.0 + 0.25 * round_))
        torch.cuda.synchronize()
        want = step().clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.uint8), want.view(torch.uint8)), round_
    for t, original in zip(inputs, originals):
        t.copy_(original)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.uint8), eager_first.view(torch.uint8))


def test_quantize_and_gate_up_product(device):
    k, n, tokens = 3840, 96, 1
    gate, up = dev(synth.q4_k_weights(n, k, 1), device), dev(synth.q4_k_weights(n, k, 2), device)
    x = dev(synth.activations(tokens, k, 3), device)
    step = lambda: ops.vecq(ops.TYPE_Q4_K, up, ops.quantize_q8_1(x), k, n, gate=gate, glu=ops.GLU_GEGLU)
    replayed_equals_eager(device, step, [x])


def test_matrix_core_products(device):
    k, n, tokens = 2048, 80, 8
    w4, w8 = dev(synth.q4_k_weights(n, k, 4), device), dev(synth.q8_0_weights(n, k, 5), device)
    x = dev(synth.activations(tokens, k, 6), device)
    replayed_equals_eager(device, lambda: ops.vecq(ops.TYPE_Q4_K, w4, ops.quantize_q8_1(x), k, n, tokens=tokens), [x])
    replayed_equals_eager(device, lambda: ops.vecq(ops.TYPE_Q8_0, w8, ops.quantize_q8_1(x), k, n, tokens=tokens), [x])


@pytest.mark.parametrize("tokens", [2, 40])
def test_routed_layer(device, tokens):
    """2 tokens: the products quantize inside; 40: routed rows sorted by expert first."""
    hidden, ffn, experts, used = 1024, 256, 16, 4
    gate_up = dev(synth.q4_k_weights(experts * 2 * ffn, hidden, 7).reshape(experts, -1), device)
    down = dev(synth.q4_k_weights(experts * hidden, ffn, 8).reshape(experts, -1), device)
    logits = dev(synth.rng(9).standard_normal((tokens, experts), dtype=np.float32), device)
    x = dev(synth.activations(tokens, hidden, 10), device)
    step = lambda: ops.moe_ffn(ops.TYPE_Q4_K, logits, x, gate_up, down, hidden, ffn, experts, used)[0]
    replayed_equals_eager(device, step, [x])


def test_mxfp8_quantize_and_gemm(device):
    m, n, k = 256, 192, 512
    g = torch.Generator().manual_seed(11)
    a = torch.randn((m, k), generator=g).to(device)
    wc, ws = ops.mxfp8_quantize((torch.randn((n, k), generator=g) * 0.02).to(device))

    def step():
        ac, as_ = ops.mxfp8_quantize(a)
        return ops.mxfp8_gemm(ac, as_, wc, ws)

    replayed_equals_eager(device, step, [a])


@pytest.mark.parametrize("m", [1, 16])
def test_exl3_linear(device, m):
    k, n, bits = 256, 384, 4
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 12)
    t = dev(trellis, device)
    su = dev(suh.view(np.int16), device).view(torch.float16)
    sv = dev(svh.view(np.int16), device).view(torch.float16)
    x = dev(synth.rng(13).standard_normal((m, k)).astype(np.float16).view(np.int16), device).view(torch.float16)
    replayed_equals_eager(device, lambda: ops.exl3_linear(t, su, sv, k, n, bits, ops.EXL3_3INST, x), [x])
