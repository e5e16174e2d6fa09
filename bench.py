"""Benchmark of the quantized mat-vec hot path on one MI355X.

A step is the decode-time gate/up product of one token: the activation's quantization to Q8_1
(llmp.q8_1) and the fused Q4_K gate/up GEGLU mat-vec over its blocks (llmp.vecq; hidden 3840, two
15360-row matrices), over one of several distinct weight copies, rotated so that neither L2 nor
the 256 MB Infinity Cache holds them. By default the step is one launch, which quantizes the bf16
activation inside the kernel under its first tile's loads (the same bits out); --two-launches
makes it the reference's two operations, llmp.q8_1 followed by llmp.vecq, which the default run
times beside it (`two_launch_step`).
Prints one JSON line; see --help. `other_configs` holds the other four benchmark configurations (Q8_0 mat-vec,
MXFP8 GEMM, the routed-expert layer at 1, 16 and 512 tokens, the EXL3 linear at 1 and 16 rows), each with the
roofline of its dominant kernel and the CPU oracle timed beside it; `--only <key>` runs one of them alone."""
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
    # Untimed replays first: after idle time (the host preparing operands) the device's clocks take milliseconds of
    # work to settle (the MXFP8 GEMM's first launches take 104 us, those after 10 ms of launches 91).
    for _ in range(SETTLE_REPLAYS):
        graph.replay()
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record()
    graph.replay()
    end.record()
    torch.cuda.synchronize()
    return begin.elapsed_time(end) / count * 1e3


SETTLE_REPLAYS = 20


MFMA_FP8_PEAK_TFLOPS = 5000.0  # dense FP8 (and int8), the published figure

# HBM bytes per launch of each configuration's roofline kernel(s), from rocprofv3 --pmc runs of this file
# (`--only <name> --no-cpu --eager --calibrate-copy`: FETCH_SIZE and WRITE_SIZE in KiB per dispatch, scaled by what
# the same counters read for --calibrate-copy's copy of known size: FETCH_SIZE reads half the bytes fetched, factor
# 2.0014, WRITE_SIZE all of them, factor 1.0010). Counters cannot be read from inside a run: a configuration that has
# not been profiled reports null.
def _traffic(fetch_kib, write_kib):
    return int(round((fetch_kib * 2.0014 + write_kib * 1.0010) * 1024))


PROFILED_TRAFFIC = {
    "q4_k_gate_up_geglu_b1": int(round((32478.4 * 1.9988 + 60.1) * 1024)),
    "q4_k_gate_up_geglu_b1_one_launch": int(round((32505.0 * 1.9988 + 60.1) * 1024)),
    "q8_0_matvec_4096x4096_b1": _traffic(8768.0, 16.0),
    # A weight row a lane asks for 144 bytes a row a load, ragged against the 64-byte units HBM is fetched in; the
    # unit two neighbouring super-blocks share is often fetched for each: 1.3 to 1.4 times the algorithmic bytes.
    "q4_k_gate_up_geglu_b4": _traffic(43611.5, 240.0),
    "q4_k_gate_up_geglu_b8": _traffic(43637.9, 480.0),
    # The same kernel over weights relaid out into 64-row tiles: a wave's 9216 bytes are consecutive.
    "q4_k_gate_up_geglu_b4_tiles64": _traffic(32567.8, 240.0),
    "q4_k_gate_up_geglu_b8_tiles64": _traffic(32649.7, 480.0),
    "q8_0_gate_up_swiglu_4096x2x14336_b8": _traffic(78810.1, 448.0),
    "q8_0_gate_up_swiglu_4096x2x14336_b8_tiles64": _traffic(61149.7, 448.0),
    "q4_k_down_15360x3840_b1": _traffic(16320.6, 30.0),
    # Tiles of 16 rows: 576-byte runs of a row, and every workgroup's own copy of the tokens where L2 misses.
    "q4_k_down_15360x3840_b4": _traffic(16805.5, 60.0),
    "q4_k_down_15360x3840_b8": _traffic(17157.2, 120.0),
    # The GEMM's tiles re-read the operands (each activation tile by 64 workgroups, each weight tile by 8) through
    # L2s of 4 MB an XCD: 191 MB fetched for 59 MB of operands, 50 MB written.
    "mxfp8_gemm_2048x12288x4096": _traffic(93182.8, 49173.6),
    "moe_q4_k_ffn_t1": _traffic(7028.8, 24.0),        # the gate/up launch
    "moe_q4_k_ffn_t16": _traffic(76769.0, 469.8),     # the gate/up launch
    "moe_q4_k_ffn_t512": _traffic(182457.3, 12338.4),  # the gate/up launch: the experts' tokens once a segment of rows
    "attn_vec_q8_0_d256_h16_kv8_cells8192_rows1": _traffic(17562.0 + 279.5, 528.0 + 16.0),  # the splits + their combination
    "attn_vec_q4_0_d256_h16_kv8_cells8192_rows1": _traffic(9369.5 + 279.5, 528.0 + 16.0),
    "attn_vec_q8_0_d256_h16_kv8_cells32768_rows1": _traffic(73938.5 + 537.5, 1056.0 + 16.0),
    "attn_vec_q4_0_d256_h16_kv8_cells32768_rows1": _traffic(40693.4 + 537.5, 1056.0 + 16.0),
    "exl3_linear_4096x14336_4bpw_m1": _traffic(14475.9 + 143.5, 232.0 + 56.0),  # product + output transform
    "exl3_linear_4096x14336_4bpw_m16": _traffic(14906.0 + 114.5 + 1921.5, 3584.0 + 128.0 + 896.0),
    "exl3_multi_linear_4096x2x14336_4bpw_m1": _traffic(28815.7 + 255.5, 464.0 + 112.0),
}


def cpu_leg(run, units_per_pass, unit, budget_s, sample, threads, scale=1.0):
    """The oracle timed on the host cores: `run()` repeated for about budget_s seconds."""
    run()
    passes, t0 = 0, time.perf_counter()
    while True:
        run()
        passes += 1
        elapsed = time.perf_counter() - t0
        if elapsed >= budget_s:
            break
    return {"value": round(units_per_pass * passes / elapsed * scale, 4), "unit": unit, "cores": threads, "kind": "port",
            "sample": f"{passes} passes of {sample}, {elapsed:.1f} s"}


def hbm_roofline(name, kernel, bytes_, us):
    achieved = bytes_ / us / 1e3
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": PROFILED_TRAFFIC.get(name), "kernel": kernel,
            "algorithmic_bytes_per_launch": int(bytes_), "avg_launch_us": round(us, 3)}


def read_only_launch(device, bytes_, kernel_us, eager=False):
    """The yardstick beside a streaming kernel's time: a launch that only reads as many bytes (llmp_hip_stream_read,
    eight 16-byte loads in flight a lane) over copies rotated like the weights, timed the same way."""
    import torch

    from llmp_amd import ops

    size = (int(bytes_) + 15) // 16 * 16
    copies = [torch.randint(0, 255, (size,), dtype=torch.uint8, device=device) for _ in range(-(-ROTATE_BYTES // size) + 1)]
    sink = ops.stream_read(copies[0])
    body = lambda i: ops.stream_read(copies[i % len(copies)], sink)
    us = event_us(body, 8 * len(copies)) if eager else graph_us(body, 8 * len(copies))
    del copies
    torch.cuda.empty_cache()
    return {"us": round(us, 3), "GB/s": round(size / us / 1e3, 1), "frac_hbm_peak": round(size / us / 1e3 / HBM_PEAK_GBPS, 4),
            "kernel_over_read_only": round(kernel_us / us, 3)}


def other_configs(device, args, only=None):
    """The other benchmark configurations (not the headline line), each with the roofline of its dominant
    kernel and the oracle timed on the host cores over a bounded sample of the same workload. Weights are
    what is streamed: every launch reads a copy that neither L2 nor the 256 MB Infinity Cache holds."""
    import numpy as np
    import torch

    import oracle
    from llmp_amd import ops, synth

    out = {}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    want = lambda name: only is None or only == name
    threads = oracle.max_threads()
    cpu = not args.no_cpu
    timed = (lambda body, count: event_us(body, count)) if args.eager else graph_us

    # Config 1: Q8_0 mat-vec 4096 x 4096, one F32 token through llmp.q8_1.
    if want("q8_0_matvec_4096x4096_b1"):
        n = k = 4096
        w_host = synth.q8_0_weights(n, k, 201)
        w = dev(w_host)
        copies = [w] + [w.clone() for _ in range(-(-ROTATE_BYTES // w.numel()) - 1)]
        x_host = synth.activations(1, k, 202)
        x = dev(x_host)
        q8 = ops.quantize_q8_1(x)
        y = torch.empty((1, 1, n), dtype=torch.float32, device=device)

        def step(i):
            ops.quantize_q8_1(x, out=q8)
            ops.vecq(ops.TYPE_Q8_0, copies[i % len(copies)], q8, k, n, out=y)

        step_us = timed(step, 4 * len(copies))
        one_launch_us = timed(lambda i: ops.vecq_fused(ops.TYPE_Q8_0, copies[i % len(copies)], x, k, n, out=y), 4 * len(copies))
        us = timed(lambda i: ops.vecq(ops.TYPE_Q8_0, copies[i % len(copies)], q8, k, n, out=y), 4 * len(copies))
        bytes_ = n * (k // 32) * 34 + k * 4 + n * 4
        entry = {"workload": "GGML Q8_0 mat-vec, N=4096, K=4096, batch 1, fp32 activations through llmp.q8_1",
                 "step_us": round(step_us, 2), "weight_GB/s_of_the_step": round(w.numel() / step_us / 1e3, 1),
                 "step_us_as_one_launch": round(one_launch_us, 2),
                 "roofline": hbm_roofline("q8_0_matvec_4096x4096_b1", "VecQFlat<FormatQ8> (llmp.vecq, Q8_0)", bytes_, us),
                 "read_only_launch": read_only_launch(device, bytes_, us, args.eager)}
        if cpu:
            q8_host = oracle.q8_1_quantize(x_host)
            entry["cpu_baseline"] = cpu_leg(lambda: oracle.vecq(oracle.TYPE_Q8_0, w_host, q8_host, k, n, threads=threads),
                                            w.numel() / 1e9, "GB/s", 3.0, "the whole 4096 x 4096 mat-vec (q8_1 once)", threads)
        out["q8_0_matvec_4096x4096_b1"] = entry
        del copies, w

    # Config 2 at batch 4 and 8.
    if any(want(f"q4_k_gate_up_geglu_b{t}{suffix}") for t in (4, 8) for suffix in ("", "_tiles64")):
        gate_host, up_host = synth.q4_k_weights(N, K, 101), synth.q4_k_weights(N, K, 102)
        gate, up = dev(gate_host), dev(up_host)
        count = -(-ROTATE_BYTES // WEIGHT_BYTES)
        gates = [gate] + [gate.clone() for _ in range(count - 1)]
        ups = [up] + [up.clone() for _ in range(count - 1)]
        for tokens in (4, 8):
            name = f"q4_k_gate_up_geglu_b{tokens}"
            if not want(name) and not want(name + "_tiles64"):
                continue
            x_host = synth.bf16_to_f32(synth.bf16_bits(synth.activations(tokens, K, 203)))
            q8 = ops.quantize_q8_1(dev(x_host))
            y = torch.empty((tokens, 1, N), dtype=torch.float32, device=device)
            if want(name):
                us = timed(lambda i: ops.vecq(ops.TYPE_Q4_K, ups[i % count], q8, K, N, gate=gates[i % count], tokens=tokens,
                                              glu=ops.GLU_GEGLU, out=y), 4 * count)
                entry = {"workload": f"config 2 at batch {tokens}",
                         "roofline": hbm_roofline(name, "VecQRows<glu, %d tokens> (llmp.vecq, Q4_K, a weight row a lane on "
                                                  "v_mfma_i32_4x4x4_16B_i8)" % (4 if tokens <= 4 else 8), algorithmic_bytes(tokens), us)}
                if cpu:
                    q8_host = oracle.q8_1_quantize(x_host)
                    entry["cpu_baseline"] = cpu_leg(
                        lambda: oracle.vecq(oracle.TYPE_Q4_K, up_host, q8_host, K, N, gate=gate_host, tokens=tokens,
                                            glu=oracle.GLU_GEGLU, threads=threads),
                        WEIGHT_BYTES / 1e9, "GB/s", 2.0, f"the whole gate/up pair at {tokens} tokens", threads)
                out[name] = entry
            # The same over weights relaid out at import into 64-row tiles (lossless; the kernel's reads become whole
            # 64-byte units): beside the reference's layout, not in place of it.
            tiled_name = name + "_tiles64"
            tiled_variant = ops.vecq_variants().index("rows pass8 tiles64")
            if want(tiled_name):
                if "gates_tiled" not in locals():
                    gates_tiled = [ops.relayout_q4_k_tiles64(g_, N, K) for g_ in gates]
                    ups_tiled = [ops.relayout_q4_k_tiles64(u_, N, K) for u_ in ups]
                us_tiled = timed(lambda i: ops.vecq(ops.TYPE_Q4_K, ups_tiled[i % count], q8, K, N, gate=gates_tiled[i % count],
                                                    tokens=tokens, glu=ops.GLU_GEGLU, variant=tiled_variant, out=y), 4 * count)
                out[tiled_name] = {"workload": f"config 2 at batch {tokens}, weights relaid out at import (llmp_hip_relayout_q4_k_tiles64)",
                                   "roofline": hbm_roofline(tiled_name, "VecQRows<glu, %d tokens> over 64-row tiles" % (4 if tokens <= 4 else 8),
                                                            algorithmic_bytes(tokens), us_tiled)}
        del gates, ups, gate, up
        if "gates_tiled" in locals():
            del gates_tiled, ups_tiled
        torch.cuda.empty_cache()

    # Q8_0 at 8 tokens (config 1's block type on a Llama-like gate/up pair, 4096 -> 2 x 14336, SwiGLU): the default form
    # over the file's layout and the row-a-lane form over weights relaid out at import.
    if want("q8_0_gate_up_swiglu_4096x2x14336_b8") or want("q8_0_gate_up_swiglu_4096x2x14336_b8_tiles64"):
        k8, n8, tokens = 4096, 14336, 8
        pair_bytes = 2 * n8 * (k8 // 32) * 34
        count = -(-ROTATE_BYTES // pair_bytes)
        gates8 = [dev(synth.q8_0_weights(n8, k8, 231))]
        ups8 = [dev(synth.q8_0_weights(n8, k8, 232))]
        gates8 += [gates8[0].clone() for _ in range(count - 1)]
        ups8 += [ups8[0].clone() for _ in range(count - 1)]
        q8 = ops.quantize_q8_1(dev(synth.activations(tokens, k8, 233)))
        y = torch.empty((tokens, 1, n8), dtype=torch.float32, device=device)
        bytes_ = pair_bytes + tokens * (k8 // 32) * 36 + tokens * n8 * 4
        if want("q8_0_gate_up_swiglu_4096x2x14336_b8"):
            us = timed(lambda i: ops.vecq(ops.TYPE_Q8_0, ups8[i % count], q8, k8, n8, gate=gates8[i % count], tokens=tokens,
                                          glu=ops.GLU_SWIGLU, out=y), 2 * count)
            out["q8_0_gate_up_swiglu_4096x2x14336_b8"] = {
                "workload": "Q8_0 gate/up pair 4096 -> 2 x 14336 with SwiGLU at 8 tokens, the file's layout; not one of the benchmark's five configurations",
                "roofline": hbm_roofline("q8_0_gate_up_swiglu_4096x2x14336_b8", "VecQRows<glu, 8 tokens, Q8_0 in the file's layout> (a weight row a lane on v_mfma_i32_4x4x4_16B_i8)", bytes_, us)}
        if want("q8_0_gate_up_swiglu_4096x2x14336_b8_tiles64"):
            tiled_variant = ops.vecq_variants().index("rows pass8 tiles64")
            gates8t = [ops.relayout_q8_0_tiles64(g_, n8, k8) for g_ in gates8]
            ups8t = [ops.relayout_q8_0_tiles64(u_, n8, k8) for u_ in ups8]
            us = timed(lambda i: ops.vecq(ops.TYPE_Q8_0, ups8t[i % count], q8, k8, n8, gate=gates8t[i % count], tokens=tokens,
                                          glu=ops.GLU_SWIGLU, variant=tiled_variant, out=y), 2 * count)
            out["q8_0_gate_up_swiglu_4096x2x14336_b8_tiles64"] = {
                "workload": "the same over weights relaid out at import (llmp_hip_relayout_q8_0_tiles64)",
                "roofline": hbm_roofline("q8_0_gate_up_swiglu_4096x2x14336_b8_tiles64",
                                         "VecQRows<glu, 8 tokens, Q8_0> over 64-row tiles (a weight row a lane on v_mfma_i32_4x4x4_16B_i8)", bytes_, us)}
            del gates8t, ups8t
        del gates8, ups8
        torch.cuda.empty_cache()

    # The same layer's down projection (15360 -> 3840, Q4_K): rows of 60 super-blocks, 60 tiles of 64 rows. One token, and
    # four and eight (the row-a-lane form in tiles of 16 rows, eight tokens staged in two spans of the row).
    down_keys = ("q4_k_down_15360x3840_b1", "q4_k_down_15360x3840_b4", "q4_k_down_15360x3840_b8")
    if any(want(key) for key in down_keys):
        kd, nd = N, K
        wdn = dev(synth.q4_k_weights(nd, kd, 104))
        downs = [wdn] + [wdn.clone() for _ in range(-(-ROTATE_BYTES // wdn.numel()) - 1)]
        for key, tokens, kernel in zip(down_keys, (1, 4, 8), ("VecQFlat<FormatQ4K>", "VecQRows<4 tokens, Q4_K in tiles of 16 rows>",
                                                               "VecQRows<8 tokens, Q4_K in tiles of 16 rows, spans>")):
            if not want(key):
                continue
            q8 = ops.quantize_q8_1(dev(synth.activations(tokens, kd, 105)))
            y = torch.empty((tokens, 1, nd), dtype=torch.float32, device=device)
            us = timed(lambda i: ops.vecq(ops.TYPE_Q4_K, downs[i % len(downs)], q8, kd, nd, tokens=tokens, out=y), 4 * len(downs))
            bytes_ = wdn.numel() + (kd * 4 + nd * 4 if tokens == 1 else tokens * (kd // 32) * 36 + tokens * nd * 4)
            out[key] = {"roofline": hbm_roofline(key, kernel, bytes_, us)}
            if tokens > 1:
                out[key]["workload"] = f"config 2's down projection at {tokens} tokens; not one of the benchmark's five configurations"
        del downs, wdn
        torch.cuda.empty_cache()

    # Config 3: MXFP8 GEMM 2048 x 12288 x 4096, bf16 out, and its activation quantizer.
    if want("mxfp8_gemm_2048x12288x4096"):
        m, n, k = 2048, 12288, 4096
        g = torch.Generator().manual_seed(3)
        a_host = torch.randn((m, k), generator=g).to(torch.bfloat16)
        w_host = torch.randn((n, k), generator=g) * 0.02
        a = a_host.to(device)
        wt = w_host.to(device)
        ac, asc = ops.mxfp8_quantize(a)
        wc, wsc = ops.mxfp8_quantize(wt)
        d = torch.empty((m, n), dtype=torch.bfloat16, device=device)
        us = event_us(lambda i: ops.mxfp8_gemm(ac, asc, wc, wsc, out=d), 30, warm=100)
        quant_us = graph_us(lambda i: ops.mxfp8_quantize(a, out=(ac, asc)), 30)
        flops = 2.0 * m * n * k
        achieved = flops / us / 1e6
        quant_bytes = m * k * 2 + m * k + m * k // 32
        entry = {"workload": "MXFP8 block-scaled GEMM, M=2048, K=4096, N=12288, E4M3 codes with E8M0 scales per 32, fp32 "
                             "accumulate, bf16 out; activations quantized per token by llmp.mxfp8.quantize",
                 "step_us": round(us + quant_us, 1), "TFLOP/s_of_the_step": round(flops / (us + quant_us) / 1e6, 1),
                 "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(achieved / MFMA_FP8_PEAK_TFLOPS, 4), "traffic": PROFILED_TRAFFIC.get("mxfp8_gemm_2048x12288x4096"),
                              "kernel": "GemmKernel192 (v_mfma_scale_f32_16x16x128_f8f6f4)", "algorithmic_flops_per_launch": int(flops),
                              "avg_launch_us": round(us, 2)},
                 "quantize": {"us": round(quant_us, 2), "bytes": quant_bytes, "GB/s": round(quant_bytes / quant_us / 1e3, 1),
                              "frac_hbm_peak": round(quant_bytes / quant_us / 1e3 / HBM_PEAK_GBPS, 4)}}
        if cpu:
            rows = 16  # a bounded sample: the first rows of A against the whole of B
            a_f32 = a_host[:rows].float().numpy()
            acodes, ascales = oracle.mxfp8_quantize(a_f32)
            bcodes, bscales = oracle.mxfp8_quantize(w_host.numpy())
            entry["cpu_baseline"] = cpu_leg(lambda: oracle.mxfp8_gemm(acodes, ascales, bcodes, bscales, threads=threads),
                                            2.0 * rows * n * k / 1e12, "TFLOP/s", 4.0,
                                            f"the first {rows} of the 2048 rows of A against all 12288 rows of B", threads)
        out["mxfp8_gemm_2048x12288x4096"] = entry
        del a, wt, ac, asc, wc, wsc, d
        torch.cuda.empty_cache()

    # Config 4: routed-expert FFN layer, 128 experts top-8, hidden 2048, FFN 768, Q4_K. Sixteen copies of the
    # experts' weights are rotated: a token's eight experts (21 MB) come from a different copy each launch, so
    # more than 320 MB pass between two reads of the same bytes.
    moe_names = [f"moe_q4_k_ffn_t{t}" for t in (1, 16, 512)]
    if any(want(nm) for nm in moe_names):
        hidden, ffn, experts, used = 2048, 768, 128, 8
        gu_host = synth.q4_k_weights(experts * 2 * ffn, hidden, 204).reshape(experts, -1)
        dn_host = synth.q4_k_weights(experts * hidden, ffn, 205).reshape(experts, -1)
        gate_up, down = dev(gu_host), dev(dn_host)
        sets = 16
        gus = [gate_up] + [gate_up.clone() for _ in range(sets - 1)]
        dns = [down] + [down.clone() for _ in range(sets - 1)]
        gu_bytes, dn_bytes = gate_up.numel() // experts, down.numel() // experts
        qk = 256
        for tokens in (1, 16, 512):
            name = f"moe_q4_k_ffn_t{tokens}"
            if not want(name):
                continue
            logits_host = synth.rng(206).standard_normal((tokens, experts), dtype=np.float32)
            x_host = synth.activations(tokens, hidden, 207)
            logits, xs = dev(logits_host), dev(x_host)
            _, ids, _ = ops.moe_ffn(ops.TYPE_Q4_K, logits, xs, gate_up, down, hidden, ffn, experts, used)
            distinct = int(torch.unique(ids).numel())
            layer = lambda i: ops.moe_ffn(ops.TYPE_Q4_K, logits, xs, gus[i % sets], dns[i % sets], hidden, ffn, experts, used)
            us = timed(layer, 2 * sets)
            chain_us = None
            if tokens == 1:
                # One token: the layer in one launch (llmp_hip_moe_token), bit for bit the four operations' result.
                chain_us = us
                state = ops.MoeTokenState(used, ffn, device)
                y1 = torch.empty(hidden, dtype=torch.float32, device=device)
                us = timed(lambda i: ops.moe_token(ops.TYPE_Q4_K, logits.view(-1), xs.view(-1), gus[i % sets], dns[i % sets], hidden, ffn,
                                                   experts, used, state, launches=2, out=y1), 2 * sets)
                one_us = timed(lambda i: ops.moe_token(ops.TYPE_Q4_K, logits.view(-1), xs.view(-1), gus[i % sets], dns[i % sets], hidden,
                                                       ffn, experts, used, state, launches=1, out=y1), 2 * sets)
                assert int(state.sync[2]) == 0, "a workgroup gave up waiting at the layer's meeting"
            # The dominant kernel alone: the gate/up product with its GLU over ready inputs.
            pairs = tokens * used
            h = torch.empty((pairs, ffn), dtype=torch.float32, device=device)
            gu_stride = 2 * ffn * (hidden // qk)
            up_of = lambda g: g.view(-1)[ffn * (hidden // qk) * 144:]
            if pairs <= 128:
                product = lambda i: ops.vecq_fused(ops.TYPE_Q4_K, up_of(gus[i % sets]), xs, hidden, ffn, gate=gus[i % sets], ids=ids,
                                                   tokens=tokens, used=used, stride_expert=gu_stride, glu=ops.GLU_SWIGLU,
                                                   out=h.view(tokens, used, ffn))
                kernel = "VecQFlat<FormatQ4K, glu, in-kernel q8_1> routed (gate/up; four tokens a pass from two tokens on)"
            else:
                route = ops.moe_route(ids, experts)
                q8 = ops.quantize_q8_1_rows(xs, route.token)
                product = lambda i: ops.vecq_sorted(ops.TYPE_Q4_K, up_of(gus[i % sets]), q8, route.offsets, hidden, ffn, experts,
                                                    gate=gus[i % sets], stride_expert=gu_stride, glu=ops.GLU_SWIGLU, out=h)
                kernel = "VecQMma<glu> over rows sorted by expert (gate/up)"
            product_us = timed(product, 2 * sets)
            product_bytes = distinct * gu_bytes + tokens * hidden * 4 + pairs * ffn * 4
            layer_bytes = distinct * (gu_bytes + dn_bytes) + tokens * hidden * 4 * 2
            entry = {"workload": f"MoE expert-grouped Q4_K FFN layer, 128 experts top-8, hidden 2048, expert FFN 768, {tokens} "
                                 "token(s): router, [q8_1,] gate/up + SwiGLU, [q8_1,] down, ordered weighted combine (one token: llmp_hip_moe_token)",
                     "layer_us": round(us, 1), "distinct_experts": distinct, "expert_weight_sets_rotated": sets,
                     "layer_algorithmic_bytes": layer_bytes, "layer_GB/s": round(layer_bytes / us / 1e3, 1),
                     "layer_frac_hbm_peak": round(layer_bytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                     "roofline": hbm_roofline(name, kernel, product_bytes, product_us)}
            if chain_us is not None:
                entry["layer_launches"] = "two (llmp_hip_moe_token: router + gate/up + SwiGLU; down + combine)"
                entry["layer_us_as_one_launch_meeting_inside"] = round(one_us, 1)
                entry["layer_us_as_four_operations"] = round(chain_us, 1)
            if tokens == 512:
                flops = tokens * used * 3 * 2.0 * hidden * ffn
                entry["layer_TFLOP/s"] = round(flops / us / 1e6, 2)
                entry["layer_frac_int8_mfma_peak"] = round(flops / us / 1e6 / MFMA_FP8_PEAK_TFLOPS, 4)
            if cpu:
                def cpu_layer():
                    ids_c, w_c = oracle.route(logits_host, used)
                    up_c = gu_host.reshape(-1)[ffn * (hidden // qk) * 144:]
                    h_c = oracle.vecq(oracle.TYPE_Q4_K, up_c, oracle.q8_1_quantize(x_host), hidden, ffn, gate=gu_host, ids=ids_c,
                                      tokens=tokens, used=used, stride_expert=gu_stride, glu=oracle.GLU_SWIGLU, experts=experts,
                                      threads=threads)
                    hq = oracle.q8_1_quantize(h_c.reshape(pairs, ffn))
                    blocks = oracle.padded_k(ffn) // 32
                    y_c = oracle.vecq(oracle.TYPE_Q4_K, dn_host, hq, ffn, hidden, ids=ids_c, tokens=tokens, used=used,
                                      stride_expert=hidden * (ffn // qk), y_token=blocks * used, y_slot=blocks, experts=experts,
                                      threads=threads)
                    return oracle.expert_reduce(y_c, w_c)
                entry["cpu_baseline"] = cpu_leg(cpu_layer, layer_bytes / 1e9, "GB/s", 2.0, f"the whole layer at {tokens} token(s)", threads)
            out[name] = entry
        del gus, dns, gate_up, down
        torch.cuda.empty_cache()

    # llmp.moe.gemm (the reference's NVFP4 grouped expert product) on config 4's shape: 512 tokens' 4096 rows sorted by
    # expert over 128 experts, each expert's 768 x 2048 (gate or up) and 2048 x 768 (down) weights. Not one of the
    # benchmark's five configurations: timed so that its cost is known.
    if want("moe_gemm_nvfp4_128_experts_t512"):
        experts, used, tokens = 128, 8, 512
        g = synth.rng(230)
        logits_host = g.standard_normal((tokens, experts), dtype=np.float32)
        _, ids, _ = (None, ops.moe_router(dev(logits_host), used)[0], None)
        counts = torch.bincount(ids.view(-1).to(torch.int64), minlength=experts).cpu().numpy()
        offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
        sf_rows = np.concatenate([[0], np.cumsum((counts + 127) // 128 * 128)]).astype(np.int32)
        rows = int(offsets[-1])
        entry = {"workload": "llmp.moe.gemm: NVFP4 (E2M1 codes, UE4M3 scales a 16) rows sorted by expert, 128 experts, "
                             f"{rows} rows, bf16 out; not one of the benchmark's five configurations", "shapes": {}}
        for n, k in ((768, 2048), (2048, 768)):
            a_codes = dev(g.integers(0, 256, size=(rows, k // 2), dtype=np.uint8))
            a_scales = dev(g.integers(0x20, 0x50, size=int(sf_rows[-1]) * (k // 16), dtype=np.uint8))
            codes_bytes, scales_bytes = n * (k // 2), (n + 127) // 128 * 128 * (k // 16)
            scales_offset = (codes_bytes + 255) // 256 * 256
            expert_stride = (scales_offset + scales_bytes + 255) // 256 * 256
            weights = g.integers(0, 256, size=(experts, expert_stride), dtype=np.uint8)
            weights[:, scales_offset:] = g.integers(0x20, 0x50, size=(experts, expert_stride - scales_offset), dtype=np.uint8)
            wd = dev(weights)
            wds = [wd] + [wd.clone() for _ in range(3)]
            d = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
            od, sd = dev(offsets), dev(sf_rows)
            us = timed(lambda i: ops.moe_gemm(a_codes, a_scales, od, sd, wds[i % 4], expert_stride, 0, scales_offset, n, k, out=d), 8)
            flops = 2.0 * rows * n * k
            entry["shapes"][f"n{n}_k{k}"] = {"us": round(us, 1), "TFLOP/s": round(flops / us / 1e6, 1),
                                             "frac_bf16_mfma_peak": round(flops / us / 1e6 / 2500.0, 4),
                                             "weight_GB/s": round(experts * (codes_bytes + scales_bytes) / us / 1e3, 1)}
        out["moe_gemm_nvfp4_128_experts_t512"] = entry
        torch.cuda.empty_cache()

    # The attention that reads the quantized KV cache (ggml.flash_attn_ext.vec_q8_0, beside the path: not one of
    # the benchmark's five configurations), at config 2's model's decode shape: 16 heads over 8 KV heads of 256, one query row, 8192 cells.
    # (And at 32768 cells, where a wave has several tiles and the next one's loads run under the products.)
    for kind, t, cells in (("q8_0", ops.TYPE_Q8_0, 8192), ("q4_0", ops.TYPE_Q4_0, 8192), ("q8_0", ops.TYPE_Q8_0, 32768),
                           ("q4_0", ops.TYPE_Q4_0, 32768)):
        name = f"attn_vec_{kind}_d256_h16_kv8_cells{cells}_rows1"
        if not want(name):
            continue
        d_, heads, kv_heads = 256, 16, 8
        g = synth.rng(240)
        k_host = oracle.kv_quantize(t, g.standard_normal((cells * kv_heads, d_), dtype=np.float32)).reshape(cells, -1)
        v_host = oracle.kv_quantize(t, g.standard_normal((cells * kv_heads, d_), dtype=np.float32)).reshape(cells, -1)
        q_host = g.standard_normal((heads, 1, d_), dtype=np.float32)
        mask_host = np.zeros((2, cells), dtype=np.float16)
        mask_host[:, cells - 37:] = -np.inf
        kd, vd = dev(k_host), dev(v_host)
        copies = max(2, -(-ROTATE_BYTES // (2 * kd.numel())))
        ks = [kd] + [kd.clone() for _ in range(copies - 1)]
        vs = [vd] + [vd.clone() for _ in range(copies - 1)]
        qd, md = dev(q_host), dev(mask_host.view(np.int16)).view(torch.float16)
        out_d = torch.empty((1, heads, d_), dtype=torch.float32, device=device)
        scratch = torch.empty(8 << 20, dtype=torch.uint8, device=device)
        scale = 1.0 / 16.0
        us = timed(lambda i: ops.attn_vec_quant(t, qd, ks[i % copies], vs[i % copies], md, d_, heads, kv_heads, cells, scale,
                                                out=out_d, scratch=scratch), 4 * copies)
        bytes_ = 2 * kd.numel() + heads * d_ * 8 + cells * 2
        entry = {"workload": f"attention over a {kind.upper()} KV cache, head size 256, 16 heads over 8 KV heads, 1 query row, "
                             f"{cells} cells (both launches: the splits and their combination); not one of the benchmark's five configurations",
                 "roofline": hbm_roofline(name, "AttnVecQuantKernel + AttnCombineKernel", bytes_, us)}
        if cpu:
            entry["cpu_baseline"] = cpu_leg(
                lambda: oracle.attention_quant(t, q_host, k_host, v_host, d_, heads, kv_heads, 1, cells, scale, mask=mask_host,
                                               threads=threads),
                bytes_ / 1e9, "GB/s", 2.0, "the whole attention", threads)
        out[name] = entry
        del ks, vs, kd, vd
        torch.cuda.empty_cache()

    # Config 5: EXL3 linear 4096 x 14336 at 4 bits, 3INST codebook.
    exl3_names = [f"exl3_linear_4096x14336_4bpw_m{m}" for m in (1, 16)]
    if any(want(nm) for nm in exl3_names) or want("exl3_multi_linear_4096x2x14336_4bpw_m1") or want("exl3_linear_4096x14336_4bpw_m2048_reconstructed"):
        k, n, bits = 4096, 14336, 4
        trellis, suh, svh = synth.exl3_weights(k, n, bits, 208)
        t0 = dev(trellis)
        trellises = [t0] + [t0.clone() for _ in range(-(-ROTATE_BYTES // t0.numel()) - 1)]
        suh_d = dev(suh.view(np.int16)).view(torch.float16)
        svh_d = dev(svh.view(np.int16)).view(torch.float16)
        for m in (1, 16):
            name = f"exl3_linear_4096x14336_4bpw_m{m}"
            if not want(name):
                continue
            x_host = synth.rng(209).standard_normal((m, k)).astype(np.float16)
            xs = dev(x_host.view(np.int16)).view(torch.float16)
            us = timed(lambda i: ops.exl3_linear(trellises[i % len(trellises)], suh_d, svh_d, k, n, bits,
                                                 ops.EXL3_3INST, xs), 2 * len(trellises))
            bytes_ = t0.numel() + 2 * k + 2 * n + m * (k * 2 + n * 4)
            entry = {"workload": f"EXL3 trellis-coded linear 4096 x 14336, 4 bits a weight, 3INST codebook, {m} row(s) of fp16: "
                                 "input transform, product, output transform",
                     "roofline": hbm_roofline(name, "the linear's launches (ProductKernel<3INST, 4> dominant)", bytes_, us)}
            if cpu:
                entry["cpu_baseline"] = cpu_leg(
                    lambda: oracle.exl3_linear(trellis, suh.view(np.uint16), svh.view(np.uint16), k, n, bits, 0, x_host, threads=threads),
                    t0.numel() / 1e9, "GB/s", 2.5, f"the whole linear at {m} row(s)", threads)
            out[name] = entry
        # The same linear at a prefill's rows through the fused reconstruction path (the reference's choice from 1,024
        # rows): the weights to F16 once, then a plain F16 product.
        if want("exl3_linear_4096x14336_4bpw_m2048_reconstructed"):
            m = 2048
            xs = dev(synth.rng(210).standard_normal((m, k)).astype(np.float16).view(np.int16)).view(torch.float16)
            lib = ops._lib.load()
            wbuf = torch.empty(k * n * 2, dtype=torch.uint8, device=device)
            both_us = event_us(lambda i: ops.exl3_linear_reconstructed(trellises[i % len(trellises)], suh_d, svh_d, k, n, bits,
                                                                       ops.EXL3_3INST, xs, f32=False, fused=True, w=wbuf), 20, warm=40)
            wt = torch.empty((k, n), dtype=torch.float16, device=device)
            recon_us = event_us(lambda i: ops.exl3_reconstruct(trellises[i % len(trellises)], suh_d, svh_d, k, n, bits,
                                                               ops.EXL3_3INST, fused=True), 20, warm=20)
            del wt
            flops = 2.0 * m * k * n
            product_us = both_us - recon_us
            out["exl3_linear_4096x14336_4bpw_m2048_reconstructed"] = {
                "workload": "EXL3 linear 4096 x 14336, 4 bits a weight, 2048 rows of fp16 through the fused reconstruction path: "
                            "the weights to fp16 (both transforms applied), then a plain fp16 product, fp32 sums, fp16 out",
                "path_us": round(both_us, 1), "reconstruction_us": round(recon_us, 1),
                "TFLOP/s_of_the_path": round(flops / both_us / 1e6, 1),
                "roofline": {"bound": "mfma", "achieved": round(flops / product_us / 1e6, 1), "peak": 2500.0, "unit": "TFLOP/s",
                             "frac": round(flops / product_us / 1e6 / 2500.0, 4), "traffic": None,
                             "kernel": "GemmKernelHalf (v_mfma_f32_16x16x32_f16): the path's time less the reconstruction's",
                             "algorithmic_flops_per_launch": int(flops), "avg_launch_us": round(product_us, 2)}}
        if want("exl3_multi_linear_4096x2x14336_4bpw_m1"):
            xs = dev(synth.rng(209).standard_normal((1, k)).astype(np.float16).view(np.int16)).view(torch.float16)
            half = len(trellises) // 2
            side = lambda i: (trellises[i % len(trellises)], suh_d, svh_d, k, n, bits, ops.EXL3_3INST)
            us = timed(lambda i: ops.exl3_multi_linear(side(i), side(i + half), xs), len(trellises))
            bytes_ = 2 * (t0.numel() + 2 * k + 2 * n) + k * 2 + 2 * (k * 2 + n * 4)
            out["exl3_multi_linear_4096x2x14336_4bpw_m1"] = {"roofline": hbm_roofline("exl3_multi_linear_4096x2x14336_4bpw_m1",
                                                                                     "exl3.multi_linear's launches", bytes_, us)}
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
        # The same at 4 and 16 input rows (a launch for every four rows).
        for rows in (4, 16):
            xr = dev(synth.activations(rows, k, 306))
            yr = torch.empty((rows, n), dtype=torch.float32, device=device)
            us = graph_us(lambda i: ops.decode_vector(decoder, ws[i % count], xr, out=yr), 2 * count)
            bytes_ = bytes_w + rows * (k * 4 + n * 4)
            out[f"decode_vector_{ops.DECODERS[decoder].replace('.', '_')}_4096x14336_rows{rows}"] = {
                "us": round(us, 2), "GB/s": round(bytes_ / us / 1e3, 1), "frac_hbm_peak": round(bytes_ / us / 1e3 / HBM_PEAK_GBPS, 4),
                "TFLOP/s": round(2.0 * rows * n * k / us / 1e6, 1)}
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


def measured_traffic(args):
    if args.tokens == 1 and args.variant == -1:
        return PROFILED_TRAFFIC["q4_k_gate_up_geglu_b1_one_launch" if args.fused else "q4_k_gate_up_geglu_b1"]
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
    ap.add_argument("--two-launches", action="store_true",
                    help="a step is llmp.q8_1 followed by llmp.vecq over its Q8_1 blocks (the reference's two "
                         "operations) instead of the one launch that quantizes the activations in the kernel")
    ap.add_argument("--fused", action="store_true", help="the default since the one launch became the faster step; kept for old command lines")
    ap.add_argument("--eager", action="store_true", help="launch each step from Python instead of a graph")
    ap.add_argument("--only", default=None,
                    help="run one of the other configurations alone (its key in other_configs) and print its entry: "
                         "what the profiler runs")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus above 1 is not built")
    args.fused = not args.two_launches

    import numpy as np
    import torch

    from llmp_amd import ops, synth

    device = torch.device("cuda:0")
    if args.calibrate_copy:
        # A copy of known size (WEIGHT_BYTES read, WEIGHT_BYTES written) for scaling the hardware counters.
        whole = torch.randint(0, 255, (WEIGHT_BYTES,), dtype=torch.uint8, device=device)
        target = torch.empty_like(whole)
        for _ in range(20):
            target.copy_(whole)
        torch.cuda.synchronize()
        del whole, target
    if args.only is not None:
        print(json.dumps({"other_configs": other_configs(device, args, only=args.only), "data": "synthetic",
                          "launch": "eager" if args.eager else "hip graph"}))
        return
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

    def two_launches(i):
        c = i % copies
        ops.quantize_q8_1(x32, out=q8.view(1, args.tokens, -1))
        ops.vecq(ops.TYPE_Q4_K, ups[c], q8, K, N, gate=gates[c], tokens=args.tokens, glu=ops.GLU_GEGLU,
                 variant=args.variant, out=out)

    def one_launch(i):
        c = i % copies
        ops.vecq_fused(ops.TYPE_Q4_K, ups[c], xd, K, N, gate=gates[c], tokens=args.tokens,
                       glu=ops.GLU_GEGLU, variant=args.variant, out=out)

    step = one_launch if args.fused else two_launches

    def kernel_only(i):
        c = i % copies
        ops.vecq(ops.TYPE_Q4_K, ups[c], q8, K, N, gate=gates[c], tokens=args.tokens, glu=ops.GLU_GEGLU,
                 variant=args.variant, out=out)

    # Decode steps are replayed as captured graphs (the reference's launch contexts capture
    # them too, src/kernels/ggml/launch.h:34-48): one graph of W steps, one of K steps.
    side = torch.cuda.Stream()

    def capture(body, count, first):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(count):
                body(first + i)
        return graph

    def timed_region(body):
        """Milliseconds of the K timed calls of body(i), by HIP events on the launching stream, right behind its W
        warm-up calls: both graphs are captured first (capturing is host work of milliseconds with the device idle,
        and the W warm-up steps are to run just ahead of the timed ones, not ahead of that gap)."""
        warm = timed = None
        if not args.eager:
            warm = capture(body, args.warmup, 0) if args.warmup > 0 else None
            timed = capture(body, args.steps, args.warmup)
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if args.eager:
            for i in range(args.warmup):
                body(i)
        elif warm is not None:
            warm.replay()
        t0 = time.perf_counter()
        begin.record()
        if args.eager:
            for i in range(args.steps):
                body(args.warmup + i)
        else:
            timed.replay()
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end), (time.perf_counter() - t0) * 1e3

    step(0)
    torch.cuda.synchronize()
    total_ms, wall_ms = timed_region(step)
    # The dominant kernel alone (the mat-vec over ready Q8_1 blocks), the same rotation.
    kernel_ms, _ = timed_region(kernel_only if not args.fused else step)
    kernel_us = kernel_ms / args.steps * 1e3
    # Beside it, the other form of the step and the mat-vec over ready Q8_1 blocks alone (not part of `value`).
    other_ms, _ = timed_region(two_launches if args.fused else one_launch)
    matvec_ms, _ = timed_region(kernel_only) if args.fused else (kernel_ms, None)
    ms = total_ms / args.steps
    value = WEIGHT_BYTES / (ms * 1e-3) / 1e9
    achieved = algorithmic_bytes(args.tokens) / (kernel_us * 1e-6) / 1e9
    line = {
        "metric": "Q-matvec weight GB/s at batch 1 (Q4_K fused gate/up GEGLU mat-vec)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot (Q4_K x Q8_1), fp32 accumulate", "data": "synthetic",
        "parity": "int32 sub-block sums bit-exact; fp32 outputs |got - want| <= 1e-3 * max(|want|, 1e-3 * rms(want)) "
                  "against the CPU oracle (a relative bound with an RMS floor, looser than a strict max-rel 1e-3)",
        "config": {"workload": f"GGML Q4_K fused gate/up GEGLU MMVQ, K={K}, N=2x{N}, batch {args.tokens}, "
                               + ("bf16 activations quantized to q8_1 in the kernel, one launch" if args.fused else "fp32 activations through llmp.q8_1, two launches")
                               + ", fp32 out",
                   "weight_copies_rotated": copies, "variant": args.variant, "launch": "eager" if args.eager else "hip graph",
                   "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(args),
                     "kernel": "VecQFlat<FormatQ4K, glu, bf16 activations quantized under the first tile's loads> (the step's one launch)"
                               if args.fused else "VecQFlatQ4K (llmp.vecq, Q4_K, GLU)",
                     "algorithmic_bytes_per_launch": algorithmic_bytes(args.tokens),
                     "avg_launch_us": round(kernel_us, 3), "host_wall_ms_per_step": round(wall_ms / args.steps, 6)},
    }
    other = {"us": round(other_ms / args.steps * 1e3, 3),
             "GB/s": round(WEIGHT_BYTES / (other_ms / args.steps * 1e-3) / 1e9, 1),
             "matvec_over_ready_q8_1_us": round(matvec_ms / args.steps * 1e3, 3)}
    line["two_launch_step" if args.fused else "one_launch_step"] = other
    del gates, ups
    torch.cuda.empty_cache()
    # Beside the roofline: what a launch that only reads the same bytes takes on this box (not part of `value`).
    line["read_only_launch"] = read_only_launch(device, algorithmic_bytes(args.tokens), kernel_us, args.eager)
    if not args.no_extras:
        line["other_configs"] = other_configs(device, args)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(gate, up, x)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
