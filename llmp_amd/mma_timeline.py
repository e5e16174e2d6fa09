"""When the waves of the matrix-core mat-vec (Q4_K) start, have their tokens staged and finish each of their first
steps: the timeline behind the tuning of llmp.vecq's several-token form.

Needs the instrumented build of the library (`make -C llmp_amd/csrc trace`: lib/libllmp_hip_trace.so; the product
library carries no instrumentation). Lane 0 of every wave stores the 100 MHz clock at sixteen points.

    python -m llmp_amd.mma_timeline [dense TOKENS | rows TOKENS | sorted TOKENS]

dense: the Q4_K gate/up pair 3840 -> 2 x 15360 at TOKENS tokens (default 8) through the 16 x 16 form; rows: the same
through the row-a-lane form (stamps: start, loads asked for, tokens staged, pieces 1 .. 10 landed, last piece
multiplied, loads drained, end); sorted: the gate/up pair of 128
experts 2048 -> 2 x 768, TOKENS tokens (default 512) routed top-8 and sorted by expert."""
import ctypes as C, os, sys
import numpy as np, torch
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from llmp_amd import _lib
_lib.SO_PATH = os.path.join(ROOT, "llmp_amd", "lib", "libllmp_hip_trace.so")
from llmp_amd import ops, synth
lib = _lib.load()
lib.llmp_hip_trace_set_mma.argtypes = [C.c_void_p]
lib.llmp_hip_trace_set_rows.argtypes = [C.c_void_p]
which = sys.argv[1] if len(sys.argv) > 1 else "dense"
dev = torch.device("cuda:0")
D = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
if which in ("dense", "rows"):
    tokens = int(sys.argv[2]) if len(sys.argv) > 2 else 8
    K, N = 3840, 15360
    g0, u0 = D(synth.q4_k_weights(N, K, 101)), D(synth.q4_k_weights(N, K, 102))
    copies = 6
    ups, gates = [u0] + [u0.clone() for _ in range(copies - 1)], [g0] + [g0.clone() for _ in range(copies - 1)]
    q8 = ops.quantize_q8_1(D(synth.activations(tokens, K, 103)))
    out = torch.empty((tokens, 1, N), dtype=torch.float32, device=dev)
    def launch(i):
        ops.vecq(ops.TYPE_Q4_K, ups[i % copies], q8, K, N, gate=gates[i % copies], glu=ops.GLU_GEGLU, tokens=tokens,
                 variant=9 if which == "dense" else 10, out=out)
else:
    tokens = int(sys.argv[2]) if len(sys.argv) > 2 else 512
    hidden, ffn, experts, used = 2048, 768, 128, 8
    per = ffn * (hidden // 256)
    copies = int(sys.argv[3]) if len(sys.argv) > 3 else 3
    w0 = D(synth.q4_k_weights(experts * 2 * ffn, hidden, 71).reshape(experts, -1))
    ws = [w0] + [w0.clone() for _ in range(copies - 1)]
    g = synth.rng(5)
    ids = np.stack([g.permutation(experts)[:used] for _ in range(tokens)]).astype(np.int32)
    route = ops.moe_route(D(ids), experts)
    counts = np.diff(route.offsets.cpu().numpy())
    print("rows an expert: min %d, mean %.1f, max %d; passes of 32: %d" % (counts.min(), counts.mean(), counts.max(), np.sum((counts + 31) // 32)))
    sq8 = ops.quantize_q8_1_rows(D(synth.activations(tokens, hidden, 73)), route.token)
    def launch(i):
        w = ws[i % copies]
        ops.vecq_sorted(ops.TYPE_Q4_K, w.view(-1)[per * 144:], sq8, route.offsets, hidden, ffn, experts, gate=w,
                        stride_expert=2 * per, glu=ops.GLU_SWIGLU)
for i in range(3 * copies): launch(i)
torch.cuda.synchronize()
b, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
b.record()
for i in range(20 * copies): launch(i)
e.record(); torch.cuda.synchronize()
print(f"{which} {tokens} tokens: {b.elapsed_time(e) / (20 * copies) * 1e3:.2f} us a launch (eager, untraced)")
trace = torch.zeros((1 << 15) * 16, dtype=torch.int64, device=dev)
assert lib.llmp_hip_trace_set_mma(trace.data_ptr()) == 0 and lib.llmp_hip_trace_set_rows(trace.data_ptr()) == 0
runs = []
for r in range(4):
    trace.zero_(); torch.cuda.synchronize()
    launch(r + 1)
    torch.cuda.synchronize()
    runs.append(trace.cpu().numpy().reshape(-1, 16).copy())
lib.llmp_hip_trace_set_mma(None); lib.llmp_hip_trace_set_rows(None)
names = ["start", "first weights asked for", "tokens staged"] + ["step %d done" % (i + 1) for i in range(10)] + ["", "", "wave done"]
if which == "rows":
    names = ["start", "loads asked for", "tokens staged"] + ["piece %d landed" % (i + 1) for i in range(10)] + ["last piece multiplied", "loads drained", "wave done"]
tr = runs[-1]
tr = tr[tr[:, 0] != 0].astype(np.float64)
t0 = tr[:, 0].min()
print("waves %d; launch length by the stamps %.2f us" % (len(tr), (tr[:, 15].max() - t0) / 100))
for s, name in enumerate(names):
    if not name: continue
    col = tr[:, s]; col = col[col != 0]
    if len(col) == 0: continue
    col = (col - t0) / 100
    print("%-24s waves %5d  min %7.2f  median %7.2f  p90 %7.2f  max %7.2f us" % (name, len(col), col.min(), np.median(col), np.percentile(col, 90), col.max()))
if which == "rows":
    raise SystemExit
steps = tr[:, 3:13]
ok = (steps != 0).all(axis=1)
if ok.any():
    d = np.diff(steps[ok], axis=1) / 100
    print("a step (median over waves), steps 2..10: " + " ".join("%.2f" % x for x in np.median(d, axis=0)))
done = (tr[:, 15] - t0) / 100
print("wave done: p10 %.1f p50 %.1f p90 %.1f max %.1f" % tuple(np.percentile(done, [10, 50, 90, 100])))
count, segments = tr[:, 13], tr[:, 14]
print("steps a wave: min %d median %d max %d; segments: min %d median %d max %d" % (count.min(), np.median(count), count.max(), segments.min(), np.median(segments), segments.max()))
for lo in range(0, int(count.max()) + 1, 4):
    pick = (count >= lo) & (count < lo + 4)
    if pick.any(): print("  waves of %2d..%2d steps: %4d, done at median %.1f us, segments median %.1f" % (lo, lo + 3, pick.sum(), np.median(done[pick]), np.median(segments[pick])))
cycles = tr[:, 12] - tr[:, 11]
span = (tr[:, 15] - tr[:, 0]) / 100
print("shader clock over a wave's life: median %.2f GHz (min %.2f, max %.2f)" % (np.median(cycles / span) / 1e3, (cycles / span).min() / 1e3, (cycles / span).max() / 1e3))
