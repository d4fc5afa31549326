"""Per-work-item timeline of the forward kernel on one of the benchmark configurations.

Needs the library built with the timeline hooks (`make -C flash-attn-rtx5060_amd timeline`, which compiles the
kernels with -DFA_TIMELINE into lib/libfa_fwd_timeline.so; the shipped library carries none of it).  Prints, per
phase of a work item (take + prologue, tile loop, epilogue, first-rows path), the mean and maximum duration and
its share, the numbers of steady and fill/drain iterations with a least-squares time per iteration of each kind,
the shader clock while running, and the spread of the workgroups' start and end times.

usage: python flash-attn-rtx5060_amd/probes/item_timeline.py c3 [library]      (env SCHED, REPS)"""
import sys, os, ctypes
REPO = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, REPO); sys.path.insert(0, os.path.join(REPO, 'tests'))
import numpy as np, torch
from __graft_entry__ import load_package
from parity_util import make_inputs, to_torch
fa = load_package()
W = {"c1": (1, 4, 256, 64, 0, False, -1, 1.0, 0.0, 1.0, 27), "c2": (4, 16, 2048, 64, 0, True, -1, 1.0, 0.0, 1.0, 28),
     "c3": (2, 32, 8192, 128, 0, True, -1, 1.0, 0.0, 1.0, 29), "c4": (1, 32, 16384, 128, 1, True, 1024, 1.0, 0.0, 1.0, 30),
     "c5": (1, 64, 32768, 128, 0, True, -1, 0.5, 0.01, 8.0, 31)}
w = sys.argv[1]; path = sys.argv[2] if len(sys.argv) > 2 else os.path.join(REPO, 'flash-attn-rtx5060_amd', 'lib', 'libfa_fwd_timeline.so')
SCHED = int(os.environ.get('SCHED', '0'))
L = ctypes.CDLL(os.path.abspath(path))
L.fa_fwd.argtypes = [ctypes.POINTER(fa.FaFwdParams), ctypes.c_void_p]
L.fa_debug_set_timeline.argtypes = [ctypes.c_void_p]
L.fa_sched_num_items.restype = ctypes.c_longlong; L.fa_sched_num_items.argtypes = [ctypes.c_int] * 4
B, H, S, D, dtype, causal, wl, sigma, frac, mult, seed = W[w]
q, k, v = make_inputs(fa, (B, H, S, D), dtype, seed, sigma, frac, mult)
tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
out = torch.empty_like(tq); lse = torch.empty((B, H, S), dtype=torch.float32, device='cuda')
n = L.fa_sched_num_items(B, H, S, D)
buf = torch.zeros((n, 16), dtype=torch.int64, device='cuda')
assert L.fa_debug_set_timeline(ctypes.c_void_p(buf.data_ptr())) == 0
p = fa.make_params(B, H, S, D, tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), out.data_ptr(), lse.data_ptr(), None, causal, wl, -1, dtype, SCHED)
stream = torch.cuda.current_stream().cuda_stream
for _ in range(int(os.environ.get('REPS', '20'))): assert L.fa_fwd(ctypes.byref(p), ctypes.c_void_p(stream)) == 0
torch.cuda.synchronize()
t = buf.cpu().numpy()
t0 = t[:, 2].min(); span = (t[:, 6].max() - t0) / 100.0
ph = {"take->prologue done": t[:, 3] - t[:, 2], "tile loop": t[:, 4] - t[:, 3], "epilogue": t[:, 5] - t[:, 4], "first rows": t[:, 6] - t[:, 5]}
cyc = (t[:, 14] - t[:, 10]).sum() / max(1, (t[:, 6] - t[:, 2]).sum()) * 100.0 / 1000.0
print(f"{w} sched={SCHED}: {n} items, span {span:.1f} us, shader clock while running {cyc:.3f} GHz")
tot = (t[:, 6] - t[:, 2]).sum()
for name, d in ph.items():
    print(f"  {name:22s} mean {d.mean()/100:.2f} us  max {d.max()/100:.2f} us  share of item time {100*d.sum()/tot:.1f} %")
print(f"  take -> Q landed       mean {(t[:, 15] - t[:, 2]).mean()/100:.2f} us  max {(t[:, 15] - t[:, 2]).max()/100:.2f} us")
gen, st = t[:, 7], t[:, 8]
loop = (t[:, 4] - t[:, 3]) / 100.0
# least squares: loop time = a*generic + b*steady
A = np.stack([gen, st], axis=1).astype(np.float64)
coef, *_ = np.linalg.lstsq(A, loop, rcond=None)
print(f"  iterations per item: generic {gen.mean():.1f}, steady {st.mean():.1f};  fit: {coef[0]:.3f} us per generic, {coef[1]:.3f} us per steady iteration")
cu = t[:, 1]
busy = {}
for row in t:
    busy.setdefault(int(row[1]), []).append((row[2], row[6]))
b = np.array([sum(e - s for s, e in v) for v in busy.values()]) / 100.0
first = np.array([min(s for s, e in v) for v in busy.values()]); last = np.array([max(e for s, e in v) for v in busy.values()])
print(f"  {len(busy)} hardware slots; busy per slot mean {b.mean():.1f} us (min {b.min():.1f}, max {b.max():.1f}); first start spread {(first.max()-first.min())/100:.1f} us; last end spread {(last.max()-last.min())/100:.1f} us")
t1v = t[:, 9] & 0xffffffff
fr = t[t1v == t1v.min()]
print("  last-phase duration by last tile index (first 3 classes):", [(int(x), round(float((t[t1v == x][:, 6] - t[t1v == x][:, 5]).mean()) / 100, 2)) for x in sorted(set(t1v.tolist()))[:3]])
if len(fr): print(f"  items with the first-rows path: {len(fr)}, mean {((fr[:,6]-fr[:,5]).mean())/100:.2f} us, end at {((fr[:,6]-t0).mean())/100:.1f} us after start (span {span:.1f})")
