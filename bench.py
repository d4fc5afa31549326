"""Headline benchmark: FlashAttention forward TFLOPS on one MI355X, fp16, hd128, causal, seqlen 8192
(batch 2, heads 32), synthetic seeded N(0,1) inputs resident in HBM.  Prints ONE JSON line.

A step is one forward pass over the whole batch through the C ABI (fa_fwd) on torch's current stream.
`roofline` prices the kernel against the dense fp16 MFMA peak with the algorithmic FLOPs 4*B*H*D*pairs
(pairs = unmasked (query,key) pairs per head); its duration is measured with HIP events on that stream.
`cpu_baseline` times the CPU oracle (a port of the reference's CPU verifier) on a bounded row sample of the
same workload on this machine's host cores and extrapolates to the whole problem.
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO)
sys.path.insert(0, os.path.join(REPO, "tests"))

PEAK_TFLOPS = 2516.6   # 256 CU x 4096 FLOP/clk/CU x 2.4 GHz: dense fp16 = bf16 MFMA ("2.5 PFLOP/s")

# HBM bytes per launch of the attention kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this
# script, each scaled by what the same counter reads for a plain 512 MiB copy kernel (FETCH_SIZE counts are
# worth 2.000 KiB, WRITE_SIZE counts 1.000 KiB).  c3: 426.3 MB read + 136.4 MB written (runs differ by a few per
# cent with the L2 hit rate of the K/V re-reads: 561 to 592 MB); c2 51.1 + 17.3; c4 644.0 + 136.3.
MEASURED_HBM_BYTES = {"c3": 562.7e6, "c2": 68.4e6, "c4": 780.3e6}
TRAFFIC_SOURCE = {"c3": "profiles/fa_fwd_pipelined_c3_pmc.md", "c2": "profiles/fa_fwd_pipelined_c2_pmc.md",
                  "c4": "profiles/fa_fwd_pipelined_c4_pmc.md"}
# the same for the backward kernels together on c3's shape (profiles/fa_bwd_c3_backward.md): the five-product form
# 5723.9 MB read + 4777.0 MB written (8.6 GB of it the dS blocks, written once and read once), the seven-product
# form 1756.4 MB read + 414.9 MB written
MEASURED_BWD_HBM_BYTES = {"c3": {"five": 10500.9e6, "seven": 2171.3e6}}

WORKLOADS = {
    # name: (B, H, S, D, dtype(0 fp16, 1 bf16), causal, window_left, sigma, row_fraction, row_mult, seed)
    "c1": (1, 4, 256, 64, 0, False, -1, 1.0, 0.0, 1.0, 27),
    "c2": (4, 16, 2048, 64, 0, True, -1, 1.0, 0.0, 1.0, 28),
    "c3": (2, 32, 8192, 128, 0, True, -1, 1.0, 0.0, 1.0, 29),
    "c4": (1, 32, 16384, 128, 1, True, 1024, 1.0, 0.0, 1.0, 30),
    "c5": (1, 64, 32768, 128, 0, True, -1, 0.5, 0.01, 8.0, 31),
}


# Few queries behind long keys (decoding): HBM-bound, not part of the headline metric.
DECODE_WORKLOADS = {
    # name: (B, H, Hk, S, S_kv, D, seed)
    "d1": (16, 32, 8, 1, 8192, 128, 41),       # grouped K/V heads
    "d2": (4, 32, 32, 1, 32768, 128, 42),      # one K/V head per query head, long keys
}
PEAK_HBM_GBS = 8000.0


def decode_bench(args):
    """One JSON line for a decode workload: a step is one forward pass of S new queries per head against S_kv
    keys through fa_fwd with key splits; the roofline is HBM (K and V read once, Q, O and logsumexp)."""
    import numpy as np
    import torch
    from __graft_entry__ import load_package
    from parity_util import TOL, errors, from_torch, make_inputs, to_torch
    import oracle_binding as ob

    fa = load_package()
    fa.lib()
    B, H, Hk, S, Skv, D, seed = DECODE_WORKLOADS[args.workload]
    q, _, _ = make_inputs(fa, (B, H, S, D), 0, seed)
    _, k, v = make_inputs(fa, (B, Hk, Skv, D), 0, seed + 100)
    tq, tk, tv = (to_torch(x, 0) for x in (q, k, v))
    out = torch.empty_like(tq)
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")

    def step():
        fa.flash_attention_forward(tq, tk, tv, causal=True, out=out, lse=lse, splits="auto")
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    gpu_ms = e0.elapsed_time(e1) / args.steps
    algo_bytes = 2 * B * Hk * Skv * D * 2 + 2 * B * H * S * D * 2 + B * H * S * 4
    # parity: the queries are the last S rows of the square S_kv problem (rows are independent)
    rep = H // Hk
    qpad = np.zeros((B, H, Skv, D), dtype=np.uint16)
    qpad[:, :, Skv - S:, :] = q
    heads = np.arange(0, B * H, max(1, (B * H) // 64))
    rows = (heads[:, None] * Skv + (Skv - S) + np.arange(S)[None, :]).reshape(-1).astype(np.int64)
    o_ref, lse_ref = ob.rows(qpad, np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1), rows, 0, None, True, -1, -1)
    sel = (heads[:, None] * S + np.arange(S)[None, :]).reshape(-1)
    err = errors(ob.to_f32(from_torch(out), 0).reshape(-1, D)[sel], ob.to_f32(o_ref, 0), lse.cpu().numpy().reshape(-1)[sel], lse_ref)
    err["rows_checked"] = int(len(rows))
    err["within_tolerance"] = bool(err["nonfinite"] == 0 and err["max_abs"] <= TOL[0]["max_abs"] and err["rel_l2"] <= TOL[0]["rel_l2"]
                                   and err["lse_abs"] <= TOL[0]["lse_abs"])
    print(json.dumps({
        "metric": "attn decode, K/V + Q + O bytes per second, 1 GPU", "value": round(algo_bytes / (wall_ms * 1e-3) / 1e9, 1),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: fp16 B{B} H{H} (K/V heads {Hk}) S{S} S_kv{Skv} D{D} causal, key splits auto",
                   "seed": seed, "algorithmic_bytes": algo_bytes},
        "roofline": {"bound": "hbm", "achieved": round(algo_bytes / (gpu_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(algo_bytes / (gpu_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "traffic": None,
                     "kernel_ms_avg": round(gpu_ms, 5)},
        "parity": err}))


def backward_bench(args):
    """One JSON line for the backward pass (fa_bwd; --bwd-form picks the five- or the seven-product form) on a forward workload's shape:
    a step is one backward pass over the whole batch; FLOPs are 2.5 x the forward's (five products over the
    unmasked pairs instead of two).  Parity: one head against torch's fp32 attention and autograd on the GPU
    (the fp64 gradient oracle checks small shapes in tests/)."""
    import numpy as np
    import torch
    from __graft_entry__ import load_package
    from parity_util import make_inputs, to_torch

    fa = load_package()
    fa.lib()
    B, H, S, D, dtype, causal, wl, sigma, frac, mult, seed = WORKLOADS[args.workload]
    q, k, v = make_inputs(fa, (B, H, S, D), dtype, seed, sigma, frac, mult)
    do, _, _ = make_inputs(fa, (B, H, S, D), dtype, seed + 1000)
    if args.kv_heads:
        if H % args.kv_heads:
            sys.exit("bench.py: --kv-heads must divide the number of heads")
        k, v = (np.ascontiguousarray(x[:, :args.kv_heads]) for x in (k, v))
    tq, tk, tv, tdo = (to_torch(x, dtype) for x in (q, k, v, do))
    if args.layout == "bshd":
        tq, tk, tv, tdo = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (tq, tk, tv, tdo))
    slopes = np.power(2.0, -8.0 / H * (np.arange(H) + 1)).astype(np.float32) if args.alibi else None
    kw = dict(causal=causal, window_left=wl, dropout_prob=args.dropout, seed=48,
              alibi_slopes=torch.from_numpy(slopes).cuda() if args.alibi else None)
    o, lse = fa.flash_attention_forward(tq, tk, tv, exact_first_rows=True, **kw)      # the pairing fa_bwd.h asks for
    grads = [None]

    def step():
        grads[0] = fa.flash_attention_backward(tq, tk, tv, o, lse, tdo, five_products="auto" if args.bwd_form == "five" else False, **kw)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    gpu_ms = e0.elapsed_time(e1) / args.steps
    flops = fa.lib().fa_bwd_algorithmic_flops(B, H, S, D, int(causal), wl, -1)
    # parity on the last head (with grouped K/V heads: the last query head alone, so only dQ is comparable)
    qf, kf, vf = (t[-1, -1].float().requires_grad_(True) for t in (tq, tk, tv))
    i = torch.arange(S, device="cuda")
    vis = torch.ones((S, S), dtype=torch.bool, device="cuda")
    if causal:
        vis &= i[None, :] <= i[:, None]
    if wl >= 0:
        vis &= i[:, None] - i[None, :] <= wl
    sc = (qf @ kf.T) * float(np.float32(1.0 / np.sqrt(D)))
    if args.alibi:
        sc = sc - float(slopes[-1]) * (i[:, None] - i[None, :]).abs().float()
    pm = torch.softmax(sc.masked_fill(~vis, float("-inf")), dim=-1)
    if args.dropout > 0:
        from parity_util import numpy_keep_mask
        thr = fa.lib().fa_dropout_threshold(args.dropout)
        pm = pm * torch.from_numpy(numpy_keep_mask(48, B * H - 1, S, thr).astype(np.float32) * (256.0 / (256 - thr))).cuda()
    (pm @ vf).backward(tdo[-1, -1].float())
    err = {}
    for name, got, want in list(zip(("dQ", "dK", "dV"), grads[0], (qf.grad, kf.grad, vf.grad)))[:1 if args.kv_heads else 3]:
        d = got[-1, -1].float() - want
        err[name] = {"rel_l2": float(d.norm() / want.norm()), "max_abs": float(d.abs().max()), "max_ref": float(want.abs().max())}
    tf = flops / (wall_ms * 1e-3) / 1e12
    plain = args.dropout == 0 and args.layout == "bhsd" and not args.kv_heads and not args.alibi      # the reference's layout
    # (the five-product form exists for regular lengths in any storage order and head grouping, with dropout or with ALiBi, not with both)
    form = "five" if (args.bwd_form == "five" and not (args.alibi and args.dropout > 0) and S % 128 == 0) else "seven"
    print(json.dumps({
        "metric": "attn backward TFLOPS (dQ, dK, dV), 1 GPU", "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if dtype else "fp16", "data": "synthetic",
        "config": {"workload": f"{args.workload} backward: {'bf16' if dtype else 'fp16'} B{B} H{H} S{S} D{D}"
                               f"{' causal' if causal else ''}{f' window_left {wl}' if wl >= 0 else ''}"
                               f"{', ALiBi' if args.alibi else ''}{f' dropout {args.dropout}' if args.dropout > 0 else ''}"
                               f"{', stored [B,S,H,D]' if args.layout == 'bshd' else ''}"
                               f"{f', {args.kv_heads} K/V heads' if args.kv_heads else ''}",
                   "seed": seed, "algorithmic_flops": flops},
        "roofline": {"bound": "mfma", "achieved": round(flops / (gpu_ms * 1e-3) / 1e12, 2), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / (gpu_ms * 1e-3) / 1e12 / PEAK_TFLOPS, 4),
                     "traffic": MEASURED_BWD_HBM_BYTES.get(args.workload, {}).get(form) if plain else None,
                     "kernel_ms_avg": round(gpu_ms, 5),
                     "kernels": "fa_bwd_prepare + fa_bwd_dkdv (writes dS) + fa_bwd_dq_from_ds" if form == "five" else "fa_bwd_dq + fa_bwd_dkdv"},
        "parity_vs_torch_fp32_one_head": err}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (the core clock of an idle MI355X needs some hundred milliseconds of load to settle: with a handful of
    # warm-up steps of a 1 ms kernel the timed region still runs through the ramp and reads about 5 % low)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + sorted(DECODE_WORKLOADS))
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="before the warm-up steps, keep the GPU busy with the same kernel for this long: an idle MI355X "
                         "raises its clock over some hundred milliseconds of load, and the timed steps are meant to "
                         "measure the sustained rate (0 disables; reported as settle_ms)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU time of the baseline sample; 0 disables")
    ap.add_argument("--check-rows", type=int, default=1024, help="rows verified against the oracle; 0 disables")
    ap.add_argument("--sched", type=int, default=0, choices=(0, 1, 2, 3), help="0 library default, 1 dispatch, 2 persistent snake, 3 persistent queue")
    ap.add_argument("--alibi", action="store_true", help="add the ALiBi bias with slopes 2^(-8/H*(h+1)) (not the headline metric)")
    ap.add_argument("--sigma", type=float, default=None,
                    help="override the standard deviation of the inputs (0 = all-zero tensors: the same instruction "
                         "stream without data-dependent switching power; not the headline metric)")
    ap.add_argument("--dropout", type=float, default=0.0, help="dropout probability (not the headline metric), seed 48")
    ap.add_argument("--layout", default="bhsd", choices=("bhsd", "bshd"),
                    help="bshd: the same values stored [B,S,H,D] and passed as strided views (not the headline metric)")
    ap.add_argument("--kv-heads", type=int, default=0, metavar="N",
                    help="K and V with N heads, shared by groups of query heads (not the headline metric)")
    ap.add_argument("--backward", action="store_true", help="time the backward pass on the workload's shape (not the headline metric)")
    ap.add_argument("--bwd-form", default="five", choices=("five", "seven"),
                    help="--backward: five = dS blocks through a B*H*S*S-element workspace and dQ as one product over them "
                         "(reference layout only; other problems fall back to seven); seven = S and dP recomputed by both kernels")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run one plain device-to-device copy kernel of this size (for scaling rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters to bytes)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (the path shards by (batch, head) with no "
                 "communication, but no multi-GPU run is part of this benchmark)")

    if args.workload in DECODE_WORKLOADS:
        return decode_bench(args)
    if args.backward:
        return backward_bench(args)

    import numpy as np
    import torch
    from __graft_entry__ import load_package
    from parity_util import TOL, errors, from_torch, make_inputs, sample_rows, to_torch

    fa = load_package()
    fa.lib()    # raises if the HIP library is missing: there is no fallback path
    B, H, S, D, dtype, causal, wl, sigma, frac, mult, seed = WORKLOADS[args.workload]
    if args.sigma is not None:
        sigma = args.sigma
    shape = (B, H, S, D)
    q, k, v = make_inputs(fa, shape, dtype, seed, sigma, frac, mult)
    if args.kv_heads:
        if H % args.kv_heads:
            sys.exit("bench.py: --kv-heads must divide the number of heads")
        k, v = (np.ascontiguousarray(x[:, :args.kv_heads]) for x in (k, v))
    tq, tk, tv = (to_torch(x, dtype) for x in (q, k, v))
    if args.layout == "bshd":
        tq, tk, tv = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (tq, tk, tv))
    out = torch.empty_like(tq)
    lse = torch.empty((B, H, S), dtype=torch.float32, device="cuda")

    slopes = np.power(2.0, -8.0 / H * (np.arange(H) + 1)).astype(np.float32) if args.alibi else None
    tslopes = torch.from_numpy(slopes).cuda() if args.alibi else None

    def step():
        fa.flash_attention_forward(tq, tk, tv, causal=causal, window_left=wl, out=out, lse=lse, sched=args.sched,
                                   alibi_slopes=tslopes, dropout_prob=args.dropout, seed=48)

    def timed(n_warmup, n_steps):
        # exactly n_steps launches back to back, one HIP event on the launch stream in front of the first and one
        # behind the last (an event between two launches is a packet of its own and costs a 60 us kernel 4 us of
        # gap); the kernel's average duration is the events' distance over the number of launches
        for _ in range(n_warmup):
            step()
        torch.cuda.synchronize()
        e_first, e_last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e_first.record()
        for _ in range(n_steps):
            step()
        e_last.record()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n_steps, e_first.elapsed_time(e_last) / n_steps

    # The same protocol without the clock-settle phase, on the still idle chip (reported next to the headline as
    # `without_settle`, so that figures taken with and without the phase can be compared like for like).
    cold_wall_ms, cold_kernel_ms = timed(args.warmup, args.steps) if args.settle_ms > 0 else (None, None)
    # clock settle (untimed, reported): launches back to back until the wall clock says settle_ms have passed
    settle_steps = 0
    if args.settle_ms > 0:
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
            for _ in range(8):
                step()
            settle_steps += 8
            torch.cuda.synchronize()
    wall_ms, avg_kernel_ms = timed(args.warmup, args.steps)        # the timed region of the headline figure
    # (a second, untimed pass with an event after every launch, for the spread only)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    ev[0].record()
    for i in range(args.steps):
        step()
        ev[i + 1].record()
    torch.cuda.synchronize()
    kernel_ms = [ev[i].elapsed_time(ev[i + 1]) for i in range(args.steps)]

    if args.copy_calibration > 0:
        src = torch.empty(args.copy_calibration << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)              # one elementwise copy kernel: reads and writes exactly this many bytes
        torch.cuda.synchronize()

    flops = fa.lib().fa_algorithmic_flops(B, H, S, D, int(causal), wl, -1)
    tflops = flops / (wall_ms * 1e-3) / 1e12
    kernel_tflops = flops / (avg_kernel_ms * 1e-3) / 1e12
    algo_bytes = 4 * B * H * S * D * 2 + B * H * S * 4

    variant = (args.alibi or args.dropout > 0 or args.sigma is not None or args.layout != "bhsd"
               or args.kv_heads)                                                  # not the headline problem
    result = {
        "metric": ("attn fwd TFLOPS + % of fp16 MFMA peak, hd128 causal seq 8192, 1 GPU" if args.workload == "c3" and not variant
                   else f"attn fwd TFLOPS + % of MFMA peak, workload {args.workload}, 1 GPU"),
        "value": round(tflops, 2), "unit": "TFLOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms": args.settle_ms, "settle_steps": settle_steps,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dtype else "fp16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {'bf16' if dtype else 'fp16'} B{B} H{H} S{S} D{D} "
                               f"{'causal' if causal else 'non-causal'}{f' window_left {wl}' if wl >= 0 else ''}, "
                               f"scale 1/sqrt({D}), fp32 accumulate, O + logsumexp{', ALiBi' if args.alibi else ''}"
                               f"{f', dropout {args.dropout}' if args.dropout else ''}"
                               f"{', stored [B,S,H,D]' if args.layout == 'bshd' else ''}"
                               f"{f', {args.kv_heads} K/V heads' if args.kv_heads else ''}",
                   "seed": seed, "sigma": sigma, "algorithmic_flops": flops, "algorithmic_bytes": algo_bytes},
        "pct_of_peak": round(100.0 * tflops / PEAK_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(kernel_tflops, 2), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(kernel_tflops / PEAK_TFLOPS, 4), "traffic": None if variant else MEASURED_HBM_BYTES.get(args.workload),
                     "traffic_source": None if variant else TRAFFIC_SOURCE.get(args.workload),
                     "kernel_ms_avg": round(avg_kernel_ms, 5), "kernel_ms_median": round(float(np.median(kernel_ms)), 5),
                     "kernel_ms_min": round(float(np.min(kernel_ms)), 5),
                     "kernel_ms_avg_from": "two events around the timed launches", "kernel_ms_median_min_from": "a second pass with an event after every launch"},
    }
    if cold_wall_ms is not None:
        result["without_settle"] = {"value": round(flops / (cold_wall_ms * 1e-3) / 1e12, 2), "ms_per_step": round(cold_wall_ms, 5),
                                    "kernel_ms_avg": round(cold_kernel_ms, 5),
                                    "frac": round(flops / (cold_kernel_ms * 1e-3) / 1e12 / PEAK_TFLOPS, 4),
                                    "note": "same steps and warm-up, run first, before the clock-settle phase"}

    drop = (fa.lib().fa_dropout_threshold(args.dropout), 48)
    rep = H // k.shape[1]
    kf, vf = (np.repeat(x, rep, axis=1) if rep > 1 else x for x in (k, v))      # the oracle takes one K/V head per query head
    if args.check_rows > 0:
        import oracle_binding as ob
        rows = sample_rows(shape, args.check_rows, seed)
        o_ref, lse_ref = ob.rows(q, kf, vf, rows, dtype, None, causal, wl, -1, slopes, dropout=drop)
        err = errors(ob.to_f32(from_torch(out.contiguous()), dtype).reshape(-1, D)[rows], ob.to_f32(o_ref, dtype),
                     lse.cpu().numpy().reshape(-1)[rows], lse_ref)
        err["rows_checked"] = int(len(rows))
        grow = 256.0 / (256 - drop[0])      # kept probabilities, and their rounding differences, are scaled by this
        err["within_tolerance"] = bool(err["nonfinite"] == 0 and err["max_abs"] <= TOL[dtype]["max_abs"] * grow
                                       and err["rel_l2"] <= TOL[dtype]["rel_l2"] * grow and err["lse_abs"] <= TOL[dtype]["lse_abs"])
        result["parity"] = err

    if args.cpu_seconds > 0:
        import oracle_binding as ob
        cores = ob.default_threads()
        rng = np.random.default_rng(seed)
        # size the sample from a probe large enough that the per-head set-up (K and V widened once per head
        # touched) no longer dominates its time
        total = B * H * S

        def timed_rows(n_rows):
            rows_ = np.sort(rng.choice(total, size=n_rows, replace=False))
            t_ = time.perf_counter()
            ob.rows(q, kf, vf, rows_, dtype, None, causal, wl, -1, slopes, threads=cores, dropout=drop)
            return rows_, time.perf_counter() - t_
        # The cost of a sample is a fixed part (K and V widened once per head touched) plus a part per row: two small
        # samples give both, and the third is sized so that all three together stay near the target.
        n1, n2 = min(total, 4096), min(total, 32768)
        _, t1 = timed_rows(n1)
        sample, dt = timed_rows(n2)
        n = n2
        if n2 > n1:
            per_row = max((dt - t1) / (n2 - n1), 1e-8)
            fixed = max(dt - per_row * n2, 0.0)
            want = int((args.cpu_seconds - t1 - dt - fixed) / per_row)
            if want > 2 * n2:
                n = min(total, want)
                spent = t1 + dt
                sample, dt = timed_rows(n)
                # (the small samples run on cold caches and overestimate the cost per row: when the sized sample
                # left more than its own time of the target unused, one more is sized from its rate)
                left = args.cpu_seconds - spent - dt
                if n < total and left > dt:
                    n = min(total, int(left / (dt / n)))
                    sample, dt = timed_rows(n)
        pairs = 0
        for r in sample.tolist():
            i = r % S
            lo = max(0, i - wl) if wl >= 0 else 0
            hi = i if causal else S - 1
            pairs += hi - lo + 1
        cpu_tflops = 4.0 * D * pairs / dt / 1e12
        result["cpu_baseline"] = {
            "value": round(cpu_tflops, 5), "unit": "TFLOPS", "cores": cores, "kind": "port",
            "sample": (f"all {n} query rows of the same workload ({pairs} unmasked pairs): the whole problem, {dt:.1f} s on {cores} threads"
                       if n >= B * H * S else
                       f"{n} uniformly sampled query rows of the same workload ({pairs} unmasked pairs), {dt:.1f} s on {cores} threads; "
                       f"at that rate the whole problem would take {flops / (cpu_tflops * 1e12):.0f} s"),
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
