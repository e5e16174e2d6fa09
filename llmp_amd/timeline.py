"""When the waves of a streaming mat-vec launch start, pass the barrier, see their tiles land and finish: the
timeline behind the tuning of llmp.vecq's one-token form.

Needs the instrumented build of the library (`make -C llmp_amd/csrc trace`, which compiles the Q4_K and Q8_0
units with -DLLMP_VECQ_TRACE into lib/libllmp_hip_trace.so; the product library carries no instrumentation).
Lane 0 of every wave stores the 100 MHz clock at eight points; the stamps themselves slow a launch by about a
fifth, so the first line prints the same launches' untraced time beside them.

    python -m llmp_amd.timeline [cfg2|cfg1] [variant]

cfg2: the Q4_K gate/up pair 3840 -> 2 x 15360; cfg1: Q8_0 4096 x 4096. One token, weights rotated cold."""
import ctypes as C, os, sys
import numpy as np, torch
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from llmp_amd import _lib
_lib.SO_PATH = os.path.join(ROOT, "llmp_amd", "lib", "libllmp_hip_trace.so")
from llmp_amd import ops, synth
lib = _lib.load()
lib.llmp_hip_trace_set.argtypes = [C.c_void_p]
which = sys.argv[1] if len(sys.argv) > 1 else "cfg2"
warm = len(sys.argv) > 3 and sys.argv[3] == "warm"
variant = int(sys.argv[2]) if len(sys.argv) > 2 else -1
dev = torch.device("cuda:0")
if which == "cfg2":
    K, N, t, glu = 3840, 15360, ops.TYPE_Q4_K, ops.GLU_GEGLU
    g0, u0 = torch.from_numpy(synth.q4_k_weights(N, K, 101)).to(dev), torch.from_numpy(synth.q4_k_weights(N, K, 102)).to(dev)
else:
    K, N, t, glu = 4096, 4096, ops.TYPE_Q8_0, ops.GLU_NONE
    u0 = torch.from_numpy(synth.q8_0_weights(N, K, 201)).to(dev); g0 = None
copies = max(2, -(-(384 << 20) // (u0.numel() * (2 if g0 is not None else 1))))
ups = [u0] + [u0.clone() for _ in range(copies - 1)]
gates = [g0] + [g0.clone() for _ in range(copies - 1)] if g0 is not None else [None] * copies
q8 = ops.quantize_q8_1(torch.from_numpy(synth.activations(1, K, 103)).to(dev))
out = torch.empty((1, 1, N), dtype=torch.float32, device=dev)
def launch(i):
    if warm: i = 0
    ops.vecq(t, ups[i % copies], q8, K, N, gate=gates[i % copies], glu=glu, variant=variant, out=out)
for i in range(3 * copies): launch(i)
torch.cuda.synchronize()
b, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
b.record()
for i in range(20 * copies): launch(i)
e.record(); torch.cuda.synchronize()
print(f"{which} variant {variant}: {b.elapsed_time(e) / (20 * copies) * 1e3:.2f} us a launch (eager, untraced)")
waves_max = 1 << 14
trace = torch.zeros(waves_max * 8, dtype=torch.int64, device=dev)
lib.llmp_hip_trace_set_q8.argtypes = [C.c_void_p]
assert lib.llmp_hip_trace_set(trace.data_ptr()) == 0 and lib.llmp_hip_trace_set_q8(trace.data_ptr()) == 0
runs = []
for r in range(5):
    trace.zero_(); torch.cuda.synchronize()
    launch(r + 1)
    torch.cuda.synchronize()
    runs.append(trace.cpu().numpy().reshape(-1, 8).copy())
lib.llmp_hip_trace_set(None); lib.llmp_hip_trace_set_q8(None)
names = ["start", "tile1 queued, part staged", "past the barrier", "tile1 landed", "tile1 stored", "tile2 landed", "tile2 stored", "wave done"]
for r, tr in enumerate(runs[3:]):
    live = tr[:, 0] != 0
    tr = tr[live].astype(np.float64); print('  launch length by the stamps: %.2f us' % ((tr[:,7].max() - tr[:,0].min())/100))
    t0 = tr[:, 0].min()
    print(f"run {r}: {live.sum()} waves; all times us after the first wave's start (100 MHz clock)")
    for j, name in enumerate(names):
        col = tr[:, j]; col = col[col != 0]
        if col.size == 0: continue
        rel = (col - t0) / 100.0
        print(f"  {name:14s} n={col.size:5d} min {rel.min():6.2f}  p10 {np.percentile(rel,10):6.2f}  median {np.median(rel):6.2f}  p90 {np.percentile(rel,90):6.2f}  max {rel.max():6.2f}")
    d1 = (tr[:, 4] - tr[:, 3]) / 100.0
    ok = (tr[:, 4] != 0) & (tr[:, 3] != 0)
    print(f"  compute of tile1 (landed->stored): median {np.median(d1[ok]):.2f} max {d1[ok].max():.2f}")
    ok2 = (tr[:, 5] != 0) & (tr[:, 4] != 0)
    d2 = (tr[:, 5] - tr[:, 4]) / 100.0
    if ok2.any(): print(f"  wait for tile2 (tile1 stored->tile2 landed): median {np.median(d2[ok2]):.2f} max {d2[ok2].max():.2f}")
