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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--tokens", type=int, default=1)
    ap.add_argument("--variant", type=int, default=-1)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--fused", action="store_true",
                    help="a step is one launch that quantizes the activations in the kernel, instead of "
                         "llmp.q8_1 followed by llmp.vecq over its Q8_1 blocks (the reference's two operations)")
    ap.add_argument("--eager", action="store_true", help="launch each step from Python instead of a graph")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus above 1 is not built (see DESIGN.md, sharding)")

    import numpy as np
    import torch

    from llmp_amd import ops, synth

    device = torch.device("cuda:0")
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
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "VecQFlatQ4K (llmp.vecq, Q4_K, GLU)",
                     "algorithmic_bytes_per_launch": algorithmic_bytes(args.tokens),
                     "avg_launch_us": round(kernel_us, 3), "host_wall_ms_per_step": round(wall_ms / args.steps, 6)},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(gate, up, x)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
