"""The MXFP8 GEMM's tile timeline: when a workgroup's waves start, have their first stages, pass steps 1 and 16,
finish the last step and queue their stores, and the shader clock meanwhile. Needs the instrumented build
(`make -C llmp_amd/csrc trace`).

    python -m llmp_amd.gemm_timeline
    python -m llmp_amd.gemm_timeline probe      # the matrix pipe alone: a step's 48 products from registers, in a loop"""
import ctypes as C, os, sys
import numpy as np, torch
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from llmp_amd import _lib
_lib.SO_PATH = os.environ.get("LLMP_TRACE_SO", os.path.join(ROOT, "llmp_amd", "lib", "libllmp_hip_trace.so"))
from llmp_amd import ops
lib = _lib.load()
lib.llmp_hip_gemm_trace_set.argtypes = [C.c_void_p]
dev = torch.device("cuda:0")
if len(sys.argv) > 1 and sys.argv[1] == "probe":
    # The matrix pipe alone: the kernel's 48 products of a step from registers, nothing between them, on every CU.
    lib.llmp_hip_gemm_probe_products.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    # (A build with -DLLMP_GEMM_PROBE_BETWEEN=6 streams `slots` x 64 KB of `data`: LLMP_PROBE_STREAM_MB says how much.)
    slots = max(1, int(os.environ.get("LLMP_PROBE_STREAM_MB", "0")) * 16)
    cus = lib.llmp_hip_compute_units()
    ticks = torch.zeros(1, dtype=torch.int64, device=dev)
    sink = torch.zeros(cus * 256, dtype=torch.float32, device=dev)
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(0, 256, (126 * 256 * 4,), generator=g, dtype=torch.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x38  # no NaN codes
    for name, data in (("zeros", torch.zeros(126 * 256, dtype=torch.int32)), ("random E4M3 codes", codes.view(torch.int32))):
        data = data.to(dev)
        if slots > 1:
            data = data.repeat(-(-slots * 65536 // (data.numel() * 4)))
        for groups in (cus, 1):
            iters = 20000 if slots == 1 else 2000
            b, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            assert lib.llmp_hip_gemm_probe_products(data.data_ptr(), iters, groups, slots, ticks.data_ptr(), sink.data_ptr(), None) == 0
            b.record()
            assert lib.llmp_hip_gemm_probe_products(data.data_ptr(), iters, groups, slots, ticks.data_ptr(), sink.data_ptr(), None) == 0
            e.record(); torch.cuda.synchronize()
            ns = b.elapsed_time(e) * 1e6 / (48 * iters)
            t = int(ticks.item()) / (48 * iters)
            print(f"{name:18s} {groups:3d} workgroups: {t:.2f} ticks of the shader counter a product, {ns:.2f} ns a product -> {t / ns:.2f} GHz, "
                  f"{groups * 4 * 65536 / ns / 1e6:.2f} PFLOP/s")
    sys.exit(0)
m, n, k = 2048, 12288, 4096
g = torch.Generator().manual_seed(3)
a = torch.randn((m, k), generator=g).to(dev).to(torch.bfloat16)
w = (torch.randn((n, k), generator=g) * 0.02).to(dev)
ac, asc = ops.mxfp8_quantize(a); wc, wsc = ops.mxfp8_quantize(w)
d = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
for _ in range(5): ops.mxfp8_gemm(ac, asc, wc, wsc, out=d)
torch.cuda.synchronize()
b, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
b.record()
for _ in range(20): ops.mxfp8_gemm(ac, asc, wc, wsc, out=d)
e.record(); torch.cuda.synchronize()
print(f"gemm {b.elapsed_time(e) / 20 * 1e3:.1f} us (untraced)")
trace = torch.zeros(512 * 8 * 16, dtype=torch.int64, device=dev)
assert lib.llmp_hip_gemm_trace_set(trace.data_ptr()) == 0
for r in range(3):
    trace.zero_(); torch.cuda.synchronize()
    ops.mxfp8_gemm(ac, asc, wc, wsc, out=d); torch.cuda.synchronize()
tr = trace.cpu().numpy().reshape(-1, 16).astype(np.float64)
tr = tr[tr[:, 0] > 0]  # the buffer has room for eight waves a workgroup
lib.llmp_hip_gemm_trace_set(None)
t0 = tr[:, 0].min()
print("waves:", len(tr), "(a workgroup a CU, its tiles one after the other)")
names = ["start", "(cycle counter)", "first stages landed", "step 1", "step 16", "last step done", "(cycle counter)", "stores queued"]
for label, base in (("first tile", 0), ("last tile", 8)):
    print(label)
    for j, nm in enumerate(names):
        if j in (1, 6) or (base and j in (0, 2)): continue
        rel = (tr[:, base + j] - t0) / 100
        print(f"  {nm:22s} min {rel.min():7.2f} median {np.median(rel):7.2f} max {rel.max():7.2f}")
    per = tr[:, base:base + 8]
    if base == 0:
        print(f"  per wave: start->landed {np.median(per[:,2]-per[:,0])/100:.2f}  landed->step1 {np.median(per[:,3]-per[:,2])/100:.2f}", end="")
    else:
        print(f"  per wave: first tile's stores queued->step1 {np.median(per[:,3]-tr[:,7])/100:.2f}", end="")
    print(f"  step1->step16 {np.median(per[:,4]-per[:,3])/100:.2f} (15 steps)  step16->last {np.median(per[:,5]-per[:,4])/100:.2f} (16 steps)  last step->stores queued {np.median(per[:,7]-per[:,5])/100:.2f}")
cyc = tr[:, 6] - tr[:, 1]; us = (tr[:, 5] - tr[:, 2]) / 100
print("first tile: shader cycles between slot 1 and 6: median %.0f; us between 2 and 5: %.2f -> clock about %.2f GHz" % (np.median(cyc), np.median(us), np.median(cyc) / np.median(us) / 1e3))
cyc = tr[:, 14] - tr[:, 9]; us = (tr[:, 13] - tr[:, 10]) / 100
print("last tile: shader cycles between its first stages landed and its last step: median %.0f in %.2f us -> clock about %.2f GHz" % (np.median(cyc), np.median(us), np.median(cyc) / np.median(us) / 1e3))
print("launch by stamps: %.1f us" % ((tr[:, 15].max() - t0) / 100))
