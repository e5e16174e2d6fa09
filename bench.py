"""Benchmark of the quantized mat-vec hot path on one MI355X.

A step is the decode-time gate/up product of one token: llmp.q8_1 (the activation's
quantization to Q8_1) followed by llmp.vecq, the fused Q4_K gate/up GEGLU mat-vec (hidden
3840, two 15360-row matrices), over one of several distinct weight copies, rotated so that
neither L2 nor the 256 MB Infinity Cache holds them. --fused makes it the single launch that
quantizes the bf16 activation inside the kernel.
Prints one JSON line; see --help."""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
K, N = 3840, 15360
ROW_BYTES = K // 256 * 144
WEIGHT_BYTES = 2 * N * ROW_BYTES  # gate + up: 66,355,200
ROTATE_BYTES = 384 << 20


def algorithmic_bytes(tokens):
    # weights + bf16 activations in + fp32 outputs
    return WEIGHT_BYTES + tokens * (K * 2 + N * 4)


def cpu_baseline(gate, up, x, budget_s=12.0):
    """The oracle's mat-vec over the same inputs on the host cores (OpenMP over rows)."""
    import oracle
    threads = oracle.max_threads()
    q8 = oracle.q8_1_quantize(x)
    run = lambda: oracle.vecq(oracle.TYPE_Q4_K, up, q8, K, N, gate=gate, tokens=1,
                              glu=oracle.GLU_GEGLU, threads=threads)
    run()
    passes, t0 = 0, time.perf_counter()
    while True:
        run()
        passes += 1
        elapsed = time.perf_counter() - t0
        if elapsed >= budget_s:
            break
    return {"value": round(WEIGHT_BYTES * passes / elapsed / 1e9, 3), "unit": "GB/s", "cores": threads,
            "kind": "port",
            "sample": f"{passes} full passes of the same gate/up matrices (q8_1 once, double accumulation), "
                      f"{elapsed:.1f} s"}


def event_us(body, count, warm=5):
    """Microseconds a call of body(i), by HIP events on the launching stream."""
    import torch
    for i in range(warm):
        body(i)
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record()
    for i in range(count):
        body(warm + i)
    end.record()
    torch.cuda.synchronize()
    return begin.elapsed_time(end) / count * 1e3


def graph_us(body, count, warm=3):
    """Microseconds a call of body(i) when `count` calls replay as one HIP graph (how the
    reference replays captured steps, src/kernels/ggml/launch.h:34-48): the launches of an
    operation made of several small kernels then cost what the GPU takes, not the host."""
    import torch
    for i in range(warm):
        body(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(count):
            body(i)
    graph.replay()
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record()
    graph.replay()
    end.record()
    torch.cuda.synchronize()
    return begin.elapsed_time(end) / count * 1e3


def other_configs(device, args):
    """Short measurements of the other benchmark configurations (not the headline line): each
    over distinct weight copies where the weights are what is streamed."""
    import numpy as np
    import torch

    from llmp_amd import ops, synth

    out = {}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)

    # Config 1: Q8_0 mat-vec 4096 x 4096, one F32 token through llmp.q8_1.
    n = k = 4096
    w = dev(synth.q8_0_weights(n, k, 201))
    copies = [w] + [w.clone() for _ in range(-(-ROTATE_BYTES // w.numel()) - 1)]
    x = dev(synth.activations(1, k, 202))
    q8 = ops.quantize_q8_1(x)
    y = torch.empty((1, 1, n), dtype=torch.float32, device=device)
    us = graph_us(lambda i: ops.vecq(ops.TYPE_Q8_0, copies[i % len(copies)], q8, k, n, out=y), 4 * len(copies))
    bytes_ = n * (k // 32) * 34 + k * 4 + n * 4
    out["q8_0_matvec_4096x4096_b1"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1),
                                       "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del copies, w

    # Config 2 at batch 4 and 8.
    gate, up = dev(synth.q4_k_weights(N, K, 101)), dev(synth.q4_k_weights(N, K, 102))
    count = -(-ROTATE_BYTES // WEIGHT_BYTES)
    gates = [gate] + [gate.clone() for _ in range(count - 1)]
    ups = [up] + [up.clone() for _ in range(count - 1)]
    for tokens in (4, 8):
        q8 = ops.quantize_q8_1(dev(synth.activations(tokens, K, 203)))
        y = torch.empty((tokens, 1, N), dtype=torch.float32, device=device)
        us = graph_us(lambda i: ops.vecq(ops.TYPE_Q4_K, ups[i % count], q8, K, N, gate=gates[i % count], tokens=tokens,
                                         glu=ops.GLU_GEGLU, out=y), 4 * count)
        out[f"q4_k_gate_up_geglu_b{tokens}"] = {"us": round(us, 2),
                                                "GB/s": round(algorithmic_bytes(tokens) / us / 1e3, 1)}
    del gates, ups, gate, up
    torch.cuda.empty_cache()

    # The same layer's down projection (15360 -> 3840, Q4_K, one token): rows of 60 super-blocks.
    kd, nd = N, K
    wdn = dev(synth.q4_k_weights(nd, kd, 104))
    downs = [wdn] + [wdn.clone() for _ in range(-(-ROTATE_BYTES // wdn.numel()) - 1)]
    q8 = ops.quantize_q8_1(dev(synth.activations(1, kd, 105)))
    y = torch.empty((1, 1, nd), dtype=torch.float32, device=device)
    us = graph_us(lambda i: ops.vecq(ops.TYPE_Q4_K, downs[i % len(downs)], q8, kd, nd, out=y), 4 * len(downs))
    bytes_ = wdn.numel() + kd * 4 + nd * 4
    out["q4_k_down_15360x3840_b1"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1),
                                      "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del downs, wdn
    torch.cuda.empty_cache()

    # An MXFP4 gate/up pair (4096 -> 2 x 14336, SwiGLU, one token): the same streaming form, 17-byte blocks.
    km, nm = 4096, 14336
    gate = dev(synth.mxfp4_weights(nm, km, 106))
    count = -(-ROTATE_BYTES // (2 * gate.numel()))
    gates = [gate] + [gate.clone() for _ in range(count - 1)]
    ups = [gate.clone() for _ in range(count)]
    q8 = ops.quantize_q8_1(dev(synth.activations(1, km, 107)))
    y = torch.empty((1, 1, nm), dtype=torch.float32, device=device)
    us = graph_us(lambda i: ops.vecq(ops.TYPE_MXFP4, ups[i % count], q8, km, nm, gate=gates[i % count],
                                     glu=ops.GLU_SWIGLU, out=y), 4 * count)
    bytes_ = 2 * gate.numel() + km * 4 + nm * 4
    out["mxfp4_gate_up_swiglu_4096x2x14336_b1"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1),
                                                   "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4)}
    del gates, ups, gate
    torch.cuda.empty_cache()

    # Config 3: MXFP8 GEMM 2048 x 12288 x 4096, bf16 out, and its activation quantizer.
    m, n, k = 2048, 12288, 4096
    g = torch.Generator().manual_seed(3)
    a = torch.randn((m, k), generator=g).to(device).to(torch.bfloat16)
    wt = (torch.randn((n, k), generator=g) * 0.02).to(device)
    ac, asc = ops.mxfp8_quantize(a)
    wc, wsc = ops.mxfp8_quantize(wt)
    d = torch.empty((m, n), dtype=torch.bfloat16, device=device)
    us = event_us(lambda i: ops.mxfp8_gemm(ac, asc, wc, wsc, out=d), 30)
    flops = 2.0 * m * n * k
    out["mxfp8_gemm_2048x12288x4096"] = {"us": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1),
                                         "frac_dense_fp8_mfma_peak": round(flops / us / 1e6 / 5033.0, 4)}
    out["mxfp8_quantize_2048x4096_bf16"] = {"us": round(event_us(lambda i: ops.mxfp8_quantize(a), 30), 1)}
    del a, wt, ac, asc, wc, wsc, d
    torch.cuda.empty_cache()

    # Config 4: routed-expert FFN layer, 128 experts top-8, hidden 2048, FFN 768, Q4_K.
    hidden, ffn, experts, used = 2048, 768, 128, 8
    gate_up = dev(synth.q4_k_weights(experts * 2 * ffn, hidden, 204).reshape(experts, -1))
    down = dev(synth.q4_k_weights(experts * hidden, ffn, 205).reshape(experts, -1))
    expert_bytes = gate_up.numel() // experts + down.numel() // experts
    for tokens in (1, 16, 512):
        logits = dev(synth.rng(206).standard_normal((tokens, experts), dtype=np.float32))
        xs = dev(synth.activations(tokens, hidden, 207))
        _, ids, _ = ops.moe_ffn(ops.TYPE_Q4_K, logits, xs, gate_up, down, hidden, ffn, experts, used)
        distinct = int(torch.unique(ids).numel())
        layer = lambda i: ops.moe_ffn(ops.TYPE_Q4_K, logits, xs, gate_up, down, hidden, ffn, experts, used)
        us = graph_us(layer, 10 if tokens == 512 else 20)
        eager = event_us(layer, 20 if tokens == 512 else 50)
        entry = {"us": round(us, 1), "us_launched_from_python": round(eager, 1), "distinct_experts": distinct,
                 "GB/s_of_touched_expert_bytes": round(distinct * expert_bytes / us / 1e3, 1),
                 "note": "whole layer replayed as a HIP graph: router, [q8_1,] gate/up+GLU, [q8_1,] down, combine "
                         "(up to 64 pairs the products quantize their activations themselves; above 128 "
                         "pairs the rows are sorted by expert first); weights not rotated"}
        if tokens == 512:
            entry["TFLOP/s"] = round(tokens * used * 3 * 2.0 * hidden * ffn / us / 1e6, 2)
        out[f"moe_q4_k_ffn_t{tokens}"] = entry
    del gate_up, down
    torch.cuda.empty_cache()

    # Config 5: EXL3 linear 4096 x 14336 at 4 bits, 3INST codebook.
    k, n, bits = 4096, 14336, 4
    trellis, suh, svh = synth.exl3_weights(k, n, bits, 208)
    t0 = dev(trellis)
    trellises = [t0] + [t0.clone() for _ in range(-(-ROTATE_BYTES // t0.numel()) - 1)]
    suh_d = dev(suh.view(np.int16)).view(torch.float16)
    svh_d = dev(svh.view(np.int16)).view(torch.float16)
    for m in (1, 16):
        xs = dev(synth.rng(209).standard_normal((m, k)).astype(np.float16).view(np.int16)).view(torch.float16)
        us = graph_us(lambda i: ops.exl3_linear(trellises[i % len(trellises)], suh_d, svh_d, k, n, bits,
                                                ops.EXL3_3INST, xs), 2 * len(trellises))
        bytes_ = t0.numel() + 2 * k + 2 * n + m * (k * 2 + n * 4)
        out[f"exl3_linear_4096x14336_4bpw_m{m}"] = {"us": round(us, 1), "GB/s": round(bytes_ / us / 1e3, 1),
                                                    "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4),
                                                    "note": "input transform, product, output transform, replayed as a HIP graph"}
    # The same shape's gate and up through exl3.multi_linear (both linears in the same launches).
    xs = dev(synth.rng(209).standard_normal((1, k)).astype(np.float16).view(np.int16)).view(torch.float16)
    half = len(trellises) // 2
    side = lambda i: (trellises[i % len(trellises)], suh_d, svh_d, k, n, bits, ops.EXL3_3INST)
    us = graph_us(lambda i: ops.exl3_multi_linear(side(i), side(i + half), xs), len(trellises))
    bytes_ = 2 * (t0.numel() + 2 * k + 2 * n) + k * 2 + 2 * (k * 2 + n * 4)
    out["exl3_multi_linear_4096x2x14336_4bpw_m1"] = {"us": round(us, 1), "GB/s": round(bytes_ / us / 1e3, 1),
                                                     "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4)}
    return out


def block_formats(device):
    """One gate/up pair (4096 -> 2 x 14336, SwiGLU, one token over ready Q8_1 blocks) in each block type the
    streaming mat-vec reads, llmp.decode.vector over five stored encodings, and the KV cache store's two types:
    `python bench.py --formats`."""
    import numpy as np
    import torch

    from llmp_amd import ops, synth

    out = {}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    k, n = 4096, 14336
    q8 = ops.quantize_q8_1(dev(synth.activations(1, k, 301)))
    y = torch.empty((1, 1, n), dtype=torch.float32, device=device)
    names = {ops.TYPE_Q4_0: "q4_0", ops.TYPE_Q4_1: "q4_1", ops.TYPE_Q5_0: "q5_0", ops.TYPE_Q5_1: "q5_1",
             ops.TYPE_Q8_0: "q8_0", ops.TYPE_Q4_K: "q4_k", ops.TYPE_MXFP4: "mxfp4", ops.TYPE_IQ4_NL: "iq4_nl", ops.TYPE_Q5_K: "q5_k", ops.TYPE_Q6_K: "q6_k"}
    for t, name in names.items():
        if t == ops.TYPE_Q4_K:
            make = lambda seed: synth.q4_k_weights(n, k, seed)
        elif t == ops.TYPE_Q8_0:
            make = lambda seed: synth.q8_0_weights(n, k, seed)
        elif t == ops.TYPE_MXFP4:
            make = lambda seed: synth.mxfp4_weights(n, k, seed)
        elif t == ops.TYPE_Q5_K:
            make = lambda seed: synth.q5_k_weights(n, k, seed)
        elif t == ops.TYPE_Q6_K:
            make = lambda seed: synth.q6_k_weights(n, k, seed)
        else:
            make = lambda seed, t=t: synth.legacy_weights(t, n, k, seed)
        gate, up = dev(make(302)), dev(make(303))
        count = -(-ROTATE_BYTES // (2 * gate.numel()))
        gates = [gate] + [gate.clone() for _ in range(count - 1)]
        ups = [up] + [up.clone() for _ in range(count - 1)]
        us = graph_us(lambda i: ops.vecq(t, ups[i % count], q8, k, n, gate=gates[i % count], glu=ops.GLU_SWIGLU, out=y),
                      4 * count)
        bytes_ = 2 * gate.numel() + q8.numel() + n * 4
        out[f"{name}_gate_up_swiglu_4096x2x14336_b1"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1),
                                                         "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4)}
        del gates, ups, gate, up
        torch.cuda.empty_cache()
    # llmp.decode.vector: one F32 input row times a 14336 x 4096 weight in its stored encoding.
    x = dev(synth.activations(1, k, 306))
    yd = torch.empty((1, n), dtype=torch.float32, device=device)
    for decoder in (0, 3, 6, 7, 9):
        w = synth.decode_weight(decoder, n, k, 307)
        base = {key: (dev(v) if isinstance(v, np.ndarray) else v) for key, v in w.items() if key != "plain"}
        bytes_w = base["data"].numel() + (base["scales"].numel() if base.get("scales") is not None else 0)
        count = max(2, -(-ROTATE_BYTES // bytes_w))
        ws = [base] + [{**base, "data": base["data"].clone()} for _ in range(count - 1)]
        us = graph_us(lambda i: ops.decode_vector(decoder, ws[i % count], x, out=yd), 2 * count)
        bytes_ = bytes_w + k * 4 + n * 4
        out[f"decode_vector_{ops.DECODERS[decoder].replace('.', '_')}_4096x14336_rows1"] = {
            "us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1), "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4)}
        del ws, base
        torch.cuda.empty_cache()
    # llmp.decode.matrix: 512 and 2048 F32 input rows times the same NVFP4 and BF16 weights on the matrix cores.
    for decoder in (0, 3):
        w = synth.decode_weight(decoder, n, k, 307)
        base = {key: (dev(v) if isinstance(v, np.ndarray) else v) for key, v in w.items() if key != "plain"}
        for rows in (512, 2048):
            xm = dev(synth.activations(rows, k, 308))
            ym = torch.empty((rows, n), dtype=torch.float32, device=device)
            us = event_us(lambda i: ops.decode_matrix(decoder, base, xm, out=ym), 20)
            out[f"decode_matrix_{ops.DECODERS[decoder].replace('.', '_')}_4096x14336_rows{rows}"] = {
                "us": round(us, 1), "TFLOP/s": round(2.0 * rows * n * k / us / 1e6, 1),
                "frac_bf16_peak": round(2.0 * rows * n * k / us / 1e6 / 2500.0, 4)}
        del base
        torch.cuda.empty_cache()
    # llmp.set_rows.quant: 512 rows of 8192 floats (a layer's K or V rows of a 512-token chunk) into a cache.
    rows, width, cells = 512, 8192, 4096
    x = dev(synth.activations(rows, width, 304))
    ids = dev(synth.rng(305).permutation(cells)[:rows].astype(np.int64))
    for t, name, size in ((ops.TYPE_Q8_0, "q8_0", 34), (ops.TYPE_Q4_0, "q4_0", 18)):
        cache = torch.zeros((cells, width // 32 * size), dtype=torch.uint8, device=device)
        us = graph_us(lambda i: ops.set_rows_quant(t, x, ids, cache), 40)
        bytes_ = rows * width * 4 + rows * (width // 32 * size)
        out[f"set_rows_quant_{name}_512x8192"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1)}
    # llmp.set_rows.grouped_quant: the K and the V rows (Q8_0 and Q4_0) in one launch.
    caches = [torch.zeros((cells, width // 32 * size), dtype=torch.uint8, device=device) for size in (34, 18)]
    x2 = dev(synth.activations(rows, width, 306))
    us = graph_us(lambda i: ops.set_rows_quant_group([(ops.TYPE_Q8_0, x, ids, caches[0]), (ops.TYPE_Q4_0, x2, ids, caches[1])]), 40)
    bytes_ = 2 * rows * width * 4 + rows * (width // 32 * 52)
    out["set_rows_grouped_quant_q8_0_q4_0_512x8192"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1)}
    # llmp.rope.set_rows_quant: 512 tokens of 64 heads of 128 values rotated (NEOX) and stored as Q8_0.
    heads, head_dim = 64, 128
    xr = x.reshape(rows, heads, head_dim)
    pos = dev(np.arange(rows, dtype=np.int32) + 1000)
    theta_scale = float(np.float32(10000.0 ** (-2.0 / head_dim)))
    us = graph_us(lambda i: ops.rope_set_rows_quant(ops.TYPE_Q8_0, xr, pos, ids, caches[0], head_dim, theta_scale), 40)
    bytes_ = rows * width * 4 + rows * (width // 32 * 34)
    out["rope_set_rows_quant_q8_0_512x64x128"] = {"us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1)}
    return out


# HBM bytes per launch of the dominant kernel at batch 1 through the default variant, from two
# rocprofv3 --pmc runs of this file (FETCH_SIZE 32,478.4 KiB and WRITE_SIZE 60.1 KiB per dispatch,
# scaled by 1.9988 and 1.0: what the same counters read for --calibrate-copy's copy of 64,800 KiB).
# Counters cannot be read from inside a run, so other shapes and variants report null.
PROFILED_TRAFFIC_BYTES = int(round((32478.4 * 1.9988 + 60.1) * 1024))


def measured_traffic(args):
    if args.tokens == 1 and args.variant == -1 and not args.fused:
        return PROFILED_TRAFFIC_BYTES
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--tokens", type=int, default=1)
    ap.add_argument("--variant", type=int, default=-1)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations' short measurements")
    ap.add_argument("--formats", action="store_true",
                    help="instead of the benchmark line: one JSON line with every block type's gate/up mat-vec and "
                         "the KV cache store")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain device copies of the weights' size (for scaling hardware counters)")
    ap.add_argument("--fused", action="store_true",
                    help="a step is one launch that quantizes the activations in the kernel, instead of "
                         "llmp.q8_1 followed by llmp.vecq over its Q8_1 blocks (the reference's two operations)")
    ap.add_argument("--eager", action="store_true", help="launch each step from Python instead of a graph")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus above 1 is not built")

    import numpy as np
    import torch

    from llmp_amd import ops, synth

    device = torch.device("cuda:0")
    if args.formats:
        print(json.dumps({"block_formats": block_formats(device), "data": "synthetic", "launch": "hip graph",
                          "weight_copies_rotated_bytes": ROTATE_BYTES}))
        return
    gate = synth.q4_k_weights(N, K, 101)
    up = synth.q4_k_weights(N, K, 102)
    x = synth.bf16_to_f32(synth.bf16_bits(synth.activations(args.tokens, K, 103)))
    copies = max(2, -(-ROTATE_BYTES // WEIGHT_BYTES))
    gd0, ud0 = torch.from_numpy(gate).to(device), torch.from_numpy(up).to(device)
    gates = [gd0] + [gd0.clone() for _ in range(copies - 1)]
    ups = [ud0] + [ud0.clone() for _ in range(copies - 1)]
    xd = torch.from_numpy(x).to(device).to(torch.bfloat16)
    out = torch.empty((args.tokens, 1, N), dtype=torch.float32, device=device)

    x32 = torch.from_numpy(x).to(device)
    q8 = ops.quantize_q8_1(x32)

    def step(i):
        c = i % copies
        if not args.fused:
            ops.quantize_q8_1(x32, out=q8.view(1, args.tokens, -1))
            ops.vecq(ops.TYPE_Q4_K, ups[c], q8, K, N, gate=gates[c], tokens=args.tokens, glu=ops.GLU_GEGLU,
                     variant=args.variant, out=out)
            return
        ops.vecq_fused(ops.TYPE_Q4_K, ups[c], xd, K, N, gate=gates[c], tokens=args.tokens,
                       glu=ops.GLU_GEGLU, variant=args.variant, out=out)

    def kernel_only(i):
        c = i % copies
        ops.vecq(ops.TYPE_Q4_K, ups[c], q8, K, N, gate=gates[c], tokens=args.tokens, glu=ops.GLU_GEGLU,
                 variant=args.variant, out=out)

    # Decode steps are replayed as captured graphs (the reference's launch contexts capture
    # them too, src/kernels/ggml/launch.h:34-48): one graph of W steps, one of K steps.
    side = torch.cuda.Stream()

    def timed_region(body, count, first):
        """Milliseconds of `count` calls of body(i), by HIP events on the launching stream."""
        graph = None
        if not args.eager:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(count):
                    body(first + i)
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        begin.record()
        if graph is None:
            for i in range(count):
                body(first + i)
        else:
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end), (time.perf_counter() - t0) * 1e3

    if args.calibrate_copy:
        # A copy of known size: WEIGHT_BYTES read, WEIGHT_BYTES written.
        whole = torch.cat([gates[0].view(-1), ups[0].view(-1)])
        target = torch.empty_like(whole)
        for _ in range(20):
            target.copy_(whole)
        torch.cuda.synchronize()
        del whole, target
    step(0)
    torch.cuda.synchronize()
    timed_region(step, args.warmup, 0)
    total_ms, wall_ms = timed_region(step, args.steps, args.warmup)
    # The dominant kernel alone (the mat-vec over ready Q8_1 blocks), the same rotation.
    timed_region(kernel_only if not args.fused else step, args.warmup, 0)
    kernel_ms, _ = timed_region(kernel_only if not args.fused else step, args.steps, args.warmup)
    kernel_us = kernel_ms / args.steps * 1e3
    ms = total_ms / args.steps
    value = WEIGHT_BYTES / (ms * 1e-3) / 1e9
    achieved = algorithmic_bytes(args.tokens) / (kernel_us * 1e-6) / 1e9
    line = {
        "metric": "Q-matvec weight GB/s at batch 1 (Q4_K fused gate/up GEGLU mat-vec)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot (Q4_K x Q8_1), fp32 accumulate", "data": "synthetic",
        "config": {"workload": f"GGML Q4_K fused gate/up GEGLU MMVQ, K={K}, N=2x{N}, batch {args.tokens}, "
                               + ("bf16 activations quantized to q8_1 in-kernel" if args.fused else "fp32 activations through llmp.q8_1")
                               + ", fp32 out",
                   "weight_copies_rotated": copies, "variant": args.variant, "launch": "eager" if args.eager else "hip graph",
                   "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(args),
                     "kernel": "VecQFlatQ4K (llmp.vecq, Q4_K, GLU)",
                     "algorithmic_bytes_per_launch": algorithmic_bytes(args.tokens),
                     "avg_launch_us": round(kernel_us, 3), "host_wall_ms_per_step": round(wall_ms / args.steps, 6)},
    }
    if not args.no_extras:
        del gates, ups
        torch.cuda.empty_cache()
        line["other_configs"] = other_configs(device, args)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(gate, up, x)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
