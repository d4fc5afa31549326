"""The library under HIP graph capture: fa_fwd (work-queue schedule, whose per-XCD counters every launch leaves
zeroed) and fa_bwd recorded once with torch.cuda.CUDAGraph and replayed on new inputs, each replay compared with
an eager call.  Neither entry point allocates, synchronises or records a memset, so capture needs nothing special;
the first (eager) call resolves the counters' device address, which is not a stream operation."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,sched", [((2, 8, 1024, 128), 3), ((1, 4, 256, 64), 1), ((4, 16, 2048, 64), 0)])
def test_forward_and_backward_replayed_from_a_graph(fa, shape, sched):
    import torch
    B, H, S, D = shape
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v, do = (torch.randn(shape, device="cuda", generator=g).half() for _ in range(4))
    o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")

    def run(out, out_lse):
        fa.flash_attention_forward(q, k, v, causal=True, out=out, lse=out_lse, sched=sched)
        return fa.flash_attention_backward(q, k, v, out, out_lse, do, causal=True)

    run(o, lse)                                     # eager warm-up: loads the kernels, resolves the work-queue address
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            grads = run(o, lse)
    torch.cuda.synchronize()
    for replay in range(4):
        for t in (q, k, v, do):                     # new contents in the captured tensors
            t.copy_(torch.randn(shape, device="cuda", generator=g).half())
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (o, lse, *grads)]
        o2, lse2 = torch.empty_like(o), torch.empty_like(lse)
        want = [o2, lse2, *run(o2, lse2)]
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.int32 if a.dtype == torch.float32 else torch.int16),
                               b.view(torch.int32 if b.dtype == torch.float32 else torch.int16)), (replay, shape, sched)


@pytest.mark.parametrize("sched", [0, 3])
def test_grouped_heads_in_bshd_storage_with_alibi_replayed_from_a_graph(fa, sched):
    """The strided flavour of the regular kernels (tensors stored [B,S,H,D], 8 query heads on 2 K/V heads, ALiBi
    slopes) captured once and replayed on new contents: every replay equals an eager call bit for bit."""
    import numpy as np
    import torch
    B, H, Hk, S, D = 2, 8, 2, 1024, 128
    g = torch.Generator(device="cuda").manual_seed(5)
    q = torch.randn((B, S, H, D), device="cuda", generator=g).half().transpose(1, 2)
    k, v = (torch.randn((B, S, Hk, D), device="cuda", generator=g).half().transpose(1, 2) for _ in range(2))
    slopes = torch.from_numpy(np.power(2.0, -8.0 / H * (np.arange(H) + 1)).astype(np.float32)).cuda()
    o = torch.empty((B, S, H, D), device="cuda", dtype=torch.float16).transpose(1, 2)
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")
    kw = dict(causal=True, window_left=300, alibi_slopes=slopes, sched=sched)
    fa.flash_attention_forward(q, k, v, out=o, lse=lse, **kw)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            fa.flash_attention_forward(q, k, v, out=o, lse=lse, **kw)
    torch.cuda.synchronize()
    for replay in range(3):
        for t in (q, k, v):
            t.copy_(torch.randn(t.shape, device="cuda", generator=g).half())
        graph.replay()
        torch.cuda.synchronize()
        o2, lse2 = fa.flash_attention_forward(q, k, v, **kw)
        torch.cuda.synchronize()
        assert torch.equal(o.contiguous().view(torch.int16), o2.contiguous().view(torch.int16)) and torch.equal(lse, lse2), (replay, sched)


def test_more_captured_queue_launches_than_counter_sets(fa):
    """Every captured queue launch owns a counter set; a device has 240 of them for captured launches, further ones
    walk the fixed order.  300 launches captured into one graph, replayed three times on new inputs: every launch's
    output must be the eager result's bits."""
    import torch
    shape = (1, 8, 1024, 64)
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v = (torch.randn(shape, device="cuda", generator=g).half() for _ in range(3))
    outs = [torch.empty_like(q) for _ in range(300)]
    lse = torch.empty(shape[:3], dtype=torch.float32, device="cuda")
    fa.flash_attention_forward(q, k, v, causal=True, out=outs[0], lse=lse, sched=3)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for o in outs:
                fa.flash_attention_forward(q, k, v, causal=True, out=o, lse=lse, sched=3)
    torch.cuda.synchronize()
    for replay in range(3):
        for t in (q, k, v):
            t.copy_(torch.randn(shape, device="cuda", generator=g).half())
        graph.replay()
        torch.cuda.synchronize()
        want, _ = fa.flash_attention_forward(q, k, v, causal=True, sched=1)
        torch.cuda.synchronize()
        for o in outs:
            assert torch.equal(o.view(torch.int16), want.view(torch.int16)), replay


FIRST_CALL_SCRIPT = r"""
import ctypes, sys
sys.path.insert(0, {repo!r}); sys.path.insert(0, {tests!r})
import torch
from __graft_entry__ import load_package
fa = load_package()
L = fa.lib()
assert L.fa_init() == fa.FA_OK
# decoding-shaped problem with key splits through the entry point that allocates nothing, queue schedule forced:
# the capture below is the library's FIRST launch in this process
B, H, Hk, S, Skv, D = 2, 8, 2, 4, 2048, 128
g = torch.Generator(device="cuda").manual_seed(3)
q = torch.randn((B, H, S, D), device="cuda", generator=g).half()
k, v = (torch.randn((B, Hk, Skv, D), device="cuda", generator=g).half() for _ in range(2))
o = torch.full_like(q, float("nan"))
lse = torch.full((B, H, S), float("nan"), dtype=torch.float32, device="cuda")
p = fa.make_params(B, H, S, D, q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), causal=True,
                   n_kv_heads=Hk, S_kv=Skv, split_num=4, sched=3)
torch.cuda.synchronize()
side = torch.cuda.Stream()
graph = torch.cuda.CUDAGraph()
with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
        st = L.fa_fwd_split_static(ctypes.byref(p), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
assert st == fa.FA_OK, st
torch.cuda.synchronize()
for replay in range(3):
    for t in (q, k, v):
        t.copy_(torch.randn(t.shape, device="cuda", generator=g).half())
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    want, want_lse = fa.flash_attention_forward(q, k, v, causal=True, splits=4, sched=3)
    torch.cuda.synchronize()
    assert torch.equal(o.view(torch.int16), want.view(torch.int16)) and torch.equal(lse, want_lse), replay
print("captured first call ok")
"""


def test_capture_as_the_first_call_after_fa_init():
    """fa_init() does everything that is not a stream operation (device arrays' addresses, CU count, the LDS
    opt-in of every kernel), so a stream capture may contain the library's very first launch.  Needs a process of
    its own: in this one the library has long been used."""
    import os
    import subprocess
    import sys
    tests = os.path.dirname(os.path.abspath(__file__))
    repo = os.path.dirname(tests)
    proc = subprocess.run([sys.executable, "-c", FIRST_CALL_SCRIPT.format(repo=repo, tests=tests)], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=300)
    assert proc.returncode == 0 and "captured first call ok" in proc.stdout, proc.stdout[-3000:]
