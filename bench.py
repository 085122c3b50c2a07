#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2]

A step is one forward + backward pass of ``flash_attention`` (public API, autograd) over one batch
of synthetic bf16 inputs that already sit in HBM.  Before the W warm-up steps the same step runs untimed
for ``--prewarm-seconds`` (default 0.5 s), so that the K timed steps see the clocks of a loaded device
rather than the ramp from idle.  Default workload: causal, B=1, H=32, T=8192,
D=128 -- the configuration the target of the metric is quoted on.  ``value`` counts matmul-only
FLOPs with the reference's convention (benchmark/flash_benchmark.py:95-103 of the reference):
forward 4*B*H*M*N*D, backward 2.5x that, halved under the causal mask.

The JSON line also carries
  * ``roofline``: the dK/dV backward kernel (the longest launch of a step) against the dense bf16
    MFMA peak, its launches timed with HIP events on the stream they run on;
  * ``cpu_baseline``: the plain-torch fp32 oracle timed on the host cores on a bounded sample
    (a few heads of the same workload);
  * ``kernels``: every launch of a step with its own counted FLOPs and time (median over 5 groups of
    20 back-to-back launches, HIP events on the launch stream);
  * ``other_flash_workloads``: the remaining flash configurations of the workload list as records of
    their own (B=4 H=16 T=2048; head size 64; Tq=1024 against Tk=8192), forward + backward through
    the public API;
  * ``matrix_pipe_ceiling``: what a loop of nothing but bf16 matrix instructions reaches on the same device with
    random and with constant operands (the device lowers its clock under a busy matrix pipe, more so the more
    the operand bits toggle): the ceiling that applies to a kernel working on real data;
  * ``paged_decode``: the paged-attention decode configuration (64 sequences, 32 query / 8 kv heads,
    head 128, block 16, context lengths uniform in [512, 8192]) as achieved HBM GB/s;
  * ``splitkv_decode`` (dense decode over 32768 keys, three K/V sets in rotation so that no launch is
    served from the last-level cache), ``piecewise`` and ``total_attention`` with rooflines of their own.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16/fp16 MFMA peak
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E peak

# HBM traffic per launch at the default workloads, from rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE,
# KiB per dispatch), each scaled by what the same counter reads for a plain 1 GiB device copy
# (FETCH_SIZE reads 0.5 GiB for 1 GiB fetched -> x2.0; WRITE_SIZE reads 1.0 GiB -> x1.0);
# profiles/hbm_traffic_per_kernel_pmc.txt holds the counter values and the commands.  Bytes.
TRAFFIC_BYTES = {
    "fa_fwd": 566863713,              # 256-row forward: 499 MB read + 68 MB written
    "fa_bwd_dkdv_ds": 3058307985,     # dS kept: 743 MB read + 2.32 GB written
    "fa_bwd_dq_from_ds": 2430783746,  # 2.36 GB read + 67 MB written
    "paged_attn": 1031160173,          # 1.027 GB read + 4 MB written
    "splitkv": 538571646,              # split kernel + merge
    "piecewise": 4786597015,           # forward + delta + dK/dV (dS kept) + the two dQ-from-dS launches
    "total_attention": 170694858,
}

WORKLOADS = {
    "c3": dict(B=1, H=32, T=8192, D=128, name="flash_attention fwd+bwd causal bf16 B=1 H=32 T=8192 D=128"),
    "c2": dict(B=4, H=16, T=2048, D=128, name="flash_attention fwd+bwd causal bf16 B=4 H=16 T=2048 D=128"),
    "c3_d64": dict(B=1, H=32, T=8192, D=64, name="flash_attention fwd+bwd causal bf16 B=1 H=32 T=8192 D=64"),
}


def causal_pairs(M, N):
    """Unmasked (query, key) pairs under the bottom-right aligned causal mask."""
    if M == N:
        return M * (M + 1) // 2
    return sum(min(max(m + N - M + 1, 0), N) for m in range(M))


def timed_launches(fn, iters, torch, groups=5):
    """Duration in ms of one ``fn``: the median over ``groups`` groups of the mean of ``iters``
    back-to-back launches, each group bracketed by HIP events on the current stream (the stream the
    C entry points launch on)."""
    for _ in range(3):
        fn()
    means = []
    for _ in range(groups):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        stop.synchronize()
        means.append(start.elapsed_time(stop) / iters)
    means.sort()
    return means[len(means) // 2]


def flash_step_leg(torch, B, H, Tq, Tk, D, iters=20):
    """One more flash_attention forward + backward configuration, public API, as a small record.  Groups of 20
    back-to-back calls, like the per-kernel timings: a group's first launch and its two event records cost some
    tens of microseconds once, which groups of 5 calls of 0.1-0.3 ms each showed as 5-10 % of a call."""
    import flagattention_amd as flag_attn
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(10086)
    mk = lambda T: torch.randn(B, H, T, D, device=dev, dtype=torch.bfloat16, generator=g)
    q, k, v, do = mk(Tq).requires_grad_(), mk(Tk).requires_grad_(), mk(Tk).requires_grad_(), mk(Tq)
    sm_scale = 1.0 / math.sqrt(D)
    ms_fwd = timed_launches(lambda: flag_attn.flash_attention(q, k, v, causal=True, sm_scale=sm_scale), iters, torch)
    o = flag_attn.flash_attention(q, k, v, causal=True, sm_scale=sm_scale)
    ms_bwd = timed_launches(lambda: torch.autograd.grad(o, (q, k, v), do, retain_graph=True), iters, torch)
    flop = 7 * 2.0 * B * H * causal_pairs(Tq, Tk) * D
    tf = flop / ((ms_fwd + ms_bwd) * 1e-3) / 1e12
    return {"workload": f"flash_attention fwd+bwd causal bf16 B={B} H={H} Tq={Tq} Tk={Tk} D={D}",
            "ms_fwd": round(ms_fwd, 4), "ms_bwd": round(ms_bwd, 4), "counted_gflop": round(flop / 1e9, 2),
            "value": round(tf, 1), "unit": "TFLOP/s", "frac_of_mfma_peak": round(tf / PEAK_BF16_TFLOPS, 4)}


def flash_step_bench(args, torch):
    import flagattention_amd as flag_attn
    from flagattention_amd import _abi, _lib

    lib = _lib.get()
    w = WORKLOADS[args.workload]
    B, H, T, D = w["B"], w["H"], w["T"], w["D"]
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(10086)
    mk = lambda: torch.randn(B, H, T, D, device=dev, dtype=torch.bfloat16, generator=g)
    q, k, v, do = mk().requires_grad_(), mk().requires_grad_(), mk().requires_grad_(), mk()
    sm_scale = 1.0 / math.sqrt(D)

    def step():
        o = flag_attn.flash_attention(q, k, v, causal=True, sm_scale=sm_scale)
        return torch.autograd.grad(o, (q, k, v), do)

    # Untimed pre-warm by time, not by count: the step loop is the first GPU work of the process, and a device
    # that starts from its idle clocks takes about 100 ms of continuous load to settle (a kernel trace of the
    # cold loop shows back-to-back launches with no gaps whose durations fall by 15-30 % over the first 40
    # steps: profiles/step_loop_cold_start_kernel_trace.txt).  --warmup steps follow, then the timed steps.
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < args.prewarm_seconds:
        for _ in range(5):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    pairs = causal_pairs(T, T)
    matmul = 2.0 * B * H * pairs * D          # one (T x T) x D product under the mask
    fwd_flops, bwd_flops = 2 * matmul, 5 * matmul
    value = (fwd_flops + bwd_flops) / (ms_per_step * 1e-3) / 1e12

    # ---- per-kernel launch times (C entry points, same stream) ----
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    o = torch.empty_like(qd)
    lse = torch.empty(B, H, T, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
    _abi.fa_fwd(lib, qd, kd, vd, o, lse, True, sm_scale)
    from flagattention_amd.flash import ds_heads_per_launch
    launches = [
        # name, callable, counted FLOPs of the launch
        ("fa_fwd", lambda: _abi.fa_fwd(lib, qd, kd, vd, o, lse, True, sm_scale), 2 * matmul),
        ("fa_bwd_delta", lambda: _abi.fa_bwd_delta(lib, o, do, delta), 0.0),
    ]
    if ds_heads_per_launch(lib, B, H, 1, T, T, D) >= B * H:   # the launches the backward above made
        ds = torch.empty(lib.fa_bwd_ds_workspace_mib(B, H, T, T) << 20, dtype=torch.uint8, device=dev)
        dkdv_name = "fa_bwd_dkdv_ds"
        launches += [
            # S, dP, dV, dK: four of the five counted backward products are produced here; dS is kept
            (dkdv_name, lambda: _abi.fa_bwd_dkdv_ds(lib, qd, kd, vd, do, lse, delta, dk, dv, ds, True, sm_scale), 4 * matmul),
            # dQ = dS K: the fifth product, bound by reading dS back
            ("fa_bwd_dq_from_ds", lambda: _abi.fa_bwd_dq_from_ds(lib, kd, ds, dq, True, sm_scale), 1 * matmul),
        ]
    else:
        dkdv_name = "fa_bwd_dkdv"
        launches += [
            (dkdv_name, lambda: _abi.fa_bwd_dkdv(lib, qd, kd, vd, do, lse, delta, dk, dv, True, sm_scale), 4 * matmul),
            # dQ; the S and dP it recomputes are not counted a second time
            ("fa_bwd_dq", lambda: _abi.fa_bwd_dq(lib, qd, kd, vd, do, lse, delta, dq, True, sm_scale), 1 * matmul),
        ]
    kernels = {}
    for name, fn, flops in launches:
        ms = timed_launches(fn, 20, torch)
        kernels[name] = {"ms": round(ms, 4), "counted_gflop": round(flops / 1e9, 2),
                         "tflops": round(flops / (ms * 1e-3) / 1e12, 1) if flops else None}
        if args.workload == "c3" and name in TRAFFIC_BYTES:
            kernels[name]["hbm_traffic_bytes"] = TRAFFIC_BYTES[name]
    if "fa_bwd_dq_from_ds" in kernels:   # algorithmic bytes: the visible dS blocks once, k and dq once
        ds_bytes = B * H * pairs * 2 + 2 * qd.numel() * 2
        kernels["fa_bwd_dq_from_ds"]["hbm_gbs"] = round(ds_bytes / (kernels["fa_bwd_dq_from_ds"]["ms"] * 1e-3) / 1e9, 1)
    dk_ms = kernels[dkdv_name]["ms"]
    achieved = 4 * matmul / (dk_ms * 1e-3) / 1e12
    roofline = {"kernel": dkdv_name + "_kernel" if dkdv_name == "fa_bwd_dkdv" else "fa_bwd_dkdv_kernel (dS kept)",
                "bound": "mfma", "achieved": round(achieved, 1),
                "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                # measured for the default workload's dS-kept launch only
                "traffic": TRAFFIC_BYTES["fa_bwd_dkdv_ds"] if args.workload == "c3" and dkdv_name == "fa_bwd_dkdv_ds" else None}
    step_frac = value / PEAK_BF16_TFLOPS
    return w, ms_per_step, value, roofline, kernels, step_frac


def cpu_baseline(args, torch):
    """The fp32 oracle on the host cores over a bounded sample: 8 of the 32 heads at T = 8192 (all 32 of the
    batch-1 slice at T = 2048)."""
    from oracle import flash_attention
    w = WORKLOADS[args.workload]
    T, D = w["T"], w["D"]
    heads = 8 if T >= 8192 else 32
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(10086)
    mk = lambda: torch.randn(1, heads, T, D, generator=g).to(torch.bfloat16)
    q, k, v, do = mk().requires_grad_(), mk().requires_grad_(), mk().requires_grad_(), mk()
    best = float("inf")
    for rep in range(2):
        t0 = time.perf_counter()
        for h in range(heads):  # head by head: one T x T fp32 score matrix alive at a time
            qs, ks, vs = (t[:, h:h + 1].detach().requires_grad_() for t in (q, k, v))
            o = flash_attention(qs, ks, vs, True, upcast=True)
            torch.autograd.grad(o, (qs, ks, vs), do[:, h:h + 1])
        best = min(best, time.perf_counter() - t0)
    flops = 7 * 2.0 * heads * causal_pairs(T, T) * D
    return {"value": round(flops / best / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{heads} of {w['H'] * w['B']} (batch, head) slices of the same workload, fp32 oracle "
                      f"fwd+bwd, best of 2, {best:.2f} s"}


def matrix_pipe_ceiling(torch):
    """What a loop of nothing but 32x32x16 bf16 matrix instructions reaches on this device (fa_probe_mfma: one
    wavefront per SIMD, operands in registers), with random and with constant operands.  The clock the device
    grants a busy matrix pipe depends on the operand values; the published peak assumes its top clock."""
    from flagattention_amd import _abi, _lib
    lib = _lib.get()
    sink = torch.empty(lib.fa_num_cus() * 256, dtype=torch.float32, device="cuda:0")
    out = {}
    for name, rnd in (("random_operands", True), ("constant_operands", False)):
        iters = 100000   # ~30 ms per launch: the clock needs tens of milliseconds of this load to settle
        flop = _abi.fa_probe_mfma(lib, sink, iters, random_operands=rnd)
        ms = timed_launches(lambda: _abi.fa_probe_mfma(lib, sink, iters, random_operands=rnd), 2, torch, groups=3)
        out[name] = round(flop / (ms * 1e-3) / 1e12, 1)
    return {"kernel": "fa_probe_mfma (matrix instructions only, 1 wavefront per SIMD, bf16)", "unit": "TFLOP/s", **out,
            "frac_of_published_peak": round(out["random_operands"] / PEAK_BF16_TFLOPS, 4)}


def paged_bench(torch, iters=50, groups=5, zeros=False):
    import flagattention_amd as flag_attn
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(10086)
    seqs, Hq, Hkv, D, bs = 64, 32, 8, 128, 16
    ctx = torch.randint(512, 8193, (seqs,), device=dev, generator=g, dtype=torch.int32)
    blocks_per_seq = (ctx + bs - 1) // bs
    num_blocks = int(blocks_per_seq.sum().item())
    max_ctx = int(ctx.max().item())
    max_blocks = (max_ctx + bs - 1) // bs
    perm = torch.randperm(num_blocks, device=dev, generator=g)
    bt = torch.zeros(seqs, max_blocks, dtype=torch.int64, device=dev)
    start = 0
    for s, n in enumerate(blocks_per_seq.tolist()):
        bt[s, :n] = perm[start:start + n]
        start += n
    q = torch.randn(seqs, Hq, D, device=dev, dtype=torch.float16, generator=g)
    kc = torch.randn(num_blocks, Hkv, bs, D, device=dev, dtype=torch.float16, generator=g)
    vc = torch.randn(num_blocks, Hkv, bs, D, device=dev, dtype=torch.float16, generator=g)
    if zeros:   # same launch and traffic, operand values that toggle nothing (profile mode only)
        q.zero_(), kc.zero_(), vc.zero_()
    scale = D ** -0.5
    fn = lambda: flag_attn.paged_attention(q, kc, vc, ctx, bt, scale, max_ctx)
    ms = timed_launches(fn, iters, torch, groups)
    total_ctx = int(ctx.sum().item())
    kv_bytes = total_ctx * Hkv * D * 2 * 2
    algo = kv_bytes + 2 * q.numel() * 2 + 8 * num_blocks
    gbs = algo / (ms * 1e-3) / 1e9
    return {"workload": "paged_attention decode fp16 seqs=64 Hq=32 Hkv=8 D=128 block=16 ctx~U[512,8192]",
            "ms": round(ms, 4), "algorithmic_bytes": algo, "value": round(gbs, 1), "unit": "GB/s",
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": TRAFFIC_BYTES["paged_attn"]}}


def splitkv_bench(torch, iters=48, groups=5, sets=3):
    """Dense split-KV decode through flash_attention: q (4, 32, 1, 128), k/v (4, 8, 32768, 128) fp16."""
    import flagattention_amd as flag_attn
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(10086)
    B, H, Hk, N, D = 4, 32, 8, 32768, 128
    q = torch.randn(B, H, 1, D, device=dev, dtype=torch.float16, generator=g)
    # Three distinct K/V sets (3 x 537 MB) used in turn: a launch never finds its keys and values in
    # the 256 MB last-level cache left there by the launch before it.
    sets = [(torch.randn(B, Hk, N, D, device=dev, dtype=torch.float16, generator=g),
             torch.randn(B, Hk, N, D, device=dev, dtype=torch.float16, generator=g)) for _ in range(sets)]
    turn = [0]

    def launch():
        k, v = sets[turn[0] % len(sets)]
        turn[0] += 1
        return flag_attn.flash_attention(q, k, v, causal=False)

    ms = timed_launches(launch, iters, torch, groups)
    k = sets[0][0]
    algo = 2 * k.numel() * 2 + 2 * q.numel() * 2
    gbs = algo / (ms * 1e-3) / 1e9
    return {"workload": "flash_attention decode fp16 q=(4,32,1,128) k/v=(4,8,32768,128) (split-KV path), "
                        f"{len(sets)} K/V sets in rotation",
            "ms": round(ms, 4), "algorithmic_bytes": algo, "value": round(gbs, 1), "unit": "GB/s",
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": TRAFFIC_BYTES["splitkv"]}}


def piecewise_bench(torch, iters=10, groups=5):
    """piecewise_attention forward + backward, causal bf16 B=2 H=32 T=4096 D=128, threshold 1024.
    FLOPs counted as for flash attention (one dot product per score), not with the reference's
    1.5x / 1.6x convention for its two score products (benchmark/piecewise_benchmark.py:98-110)."""
    import flagattention_amd as flag_attn
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(10086)
    B, H, T, D, w = 2, 32, 4096, 128, 1024
    ts = [torch.randn(B, H, T, D, device=dev, dtype=torch.bfloat16, generator=g).requires_grad_() for _ in range(5)]
    do = torch.randn(B, H, T, D, device=dev, dtype=torch.bfloat16, generator=g)
    ms_fwd = timed_launches(lambda: flag_attn.piecewise_attention(*ts, w, causal=True), iters, torch, groups)
    o = flag_attn.piecewise_attention(*ts, w, causal=True)
    ms_bwd = timed_launches(lambda: torch.autograd.grad(o, ts, do, retain_graph=True), iters, torch, groups)
    fwd = 4.0 * B * H * causal_pairs(T, T) * D
    tf = (fwd * 3.5) / ((ms_fwd + ms_bwd) * 1e-3) / 1e12
    return {"workload": "piecewise_attention fwd+bwd causal bf16 B=2 H=32 T=4096 D=128 dist_threshold=1024",
            "ms_fwd": round(ms_fwd, 4), "ms_bwd": round(ms_bwd, 4), "counted_gflop": round(fwd * 3.5 / 1e9, 2),
            "value": round(tf, 1), "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": TRAFFIC_BYTES["piecewise"]}}


def total_attention_bench(torch, iters=20, groups=5):
    """total_attention (column sums of P) at the benchmark shape: one product, 2 * pairs * D per head."""
    import flagattention_amd as flag_attn
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(10086)
    B, H, T, D = 1, 32, 8192, 128
    q, k, v = (torch.randn(B, H, T, D, device=dev, dtype=torch.bfloat16, generator=g) for _ in range(3))
    _, L, _, _, _ = flag_attn.flash_attention(q, k, v, causal=True, return_log_normalizer=True)
    ms = timed_launches(lambda: flag_attn.total_attention(q, k, L, True, D ** -0.5), iters, torch, groups)
    flop = 2.0 * B * H * causal_pairs(T, T) * D
    tf = flop / (ms * 1e-3) / 1e12
    return {"workload": "total_attention causal bf16 B=1 H=32 T=8192 D=128", "ms": round(ms, 4),
            "counted_gflop": round(flop / 1e9, 2), "value": round(tf, 1), "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": TRAFFIC_BYTES["total_attention"]}}


def profile_kernel(args, torch):
    """A handful of launches of one kernel at the benchmark's shapes, nothing else on the device."""
    from flagattention_amd import _abi, _lib
    lib = _lib.get()
    dev = "cuda:0"
    if args.profile_kernel == "copy":
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"profiled": "copy", "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return
    whole_legs = {"mfma_probe": lambda: matrix_pipe_ceiling(torch),
                  "paged_attn": lambda: paged_bench(torch, iters=50 if args.timed else 2, groups=5 if args.timed else 1,
                                                    zeros=args.operands == "zeros"),
                  "splitkv": lambda: splitkv_bench(torch, iters=3, groups=1),
                  "piecewise": lambda: piecewise_bench(torch, iters=2, groups=1),
                  "total_attention": lambda: total_attention_bench(torch, iters=2, groups=1)}
    if args.profile_kernel in whole_legs:
        print(json.dumps({"profiled": args.profile_kernel, **whole_legs[args.profile_kernel]()}))
        return
    w = WORKLOADS[args.workload]
    B, H, T, D = w["B"], w["H"], w["T"], w["D"]
    g = torch.Generator(device=dev).manual_seed(10086)
    if args.operands == "zeros":   # the same instruction stream and memory traffic on operands that toggle nothing
        mk = lambda: torch.zeros(B, H, T, D, device=dev, dtype=torch.bfloat16)
    else:
        mk = lambda: torch.randn(B, H, T, D, device=dev, dtype=torch.bfloat16, generator=g)
    q, k, v, do = mk(), mk(), mk(), mk()
    sm_scale = 1.0 / math.sqrt(D)
    o, lse = torch.empty_like(q), torch.empty(B, H, T, device=dev, dtype=torch.float32)
    delta = torch.empty_like(lse)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    _abi.fa_fwd(lib, q, k, v, o, lse, True, sm_scale)
    _abi.fa_bwd_delta(lib, o, do, delta)
    ds = torch.empty(lib.fa_bwd_ds_workspace_mib(B, H, T, T) << 20, dtype=torch.uint8, device=dev)
    if D == 128:   # the dS hand-over is the head-size-128 route; smaller heads recompute dS in fa_bwd_dq
        _abi.fa_bwd_dkdv_ds(lib, q, k, v, do, lse, delta, dk, dv, ds, True, sm_scale)
    fn = {"fa_fwd": lambda: _abi.fa_fwd(lib, q, k, v, o, lse, True, sm_scale),
          "fa_bwd_dkdv": lambda: _abi.fa_bwd_dkdv(lib, q, k, v, do, lse, delta, dk, dv, True, sm_scale),
          "fa_bwd_dkdv_ds": lambda: _abi.fa_bwd_dkdv_ds(lib, q, k, v, do, lse, delta, dk, dv, ds, True, sm_scale),
          "fa_bwd_dq_from_ds": lambda: _abi.fa_bwd_dq_from_ds(lib, k, ds, dq, True, sm_scale),
          "fa_bwd_dq": lambda: _abi.fa_bwd_dq(lib, q, k, v, do, lse, delta, dq, True, sm_scale)}[args.profile_kernel]
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    if args.hold_seconds > 0:   # keep the kernel running back to back, e.g. to read the clock it settles at
        import time
        t0 = time.time()
        while time.time() - t0 < args.hold_seconds:
            for _ in range(50):
                fn()
            torch.cuda.synchronize()
    out = {"profiled": args.profile_kernel, "workload": w["name"], "operands": args.operands}
    if args.timed:
        out["ms"] = round(timed_launches(fn, 20, torch, 5), 4)
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="c3")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--profile-kernel", choices=["fa_fwd", "fa_bwd_dkdv", "fa_bwd_dkdv_ds", "fa_bwd_dq", "fa_bwd_dq_from_ds",
                                                  "paged_attn", "splitkv", "piecewise", "total_attention", "copy", "mfma_probe"],
                    help="run only this launch a few times (for rocprofv3 counter passes); 'copy' is a plain "
                         "1 GiB device copy used to calibrate FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--hold-seconds", type=float, default=0.0,
                    help="with --profile-kernel: afterwards repeat the launch for this long")
    ap.add_argument("--operands", choices=["random", "zeros"], default="random",
                    help="with --profile-kernel on a flash kernel: standard-normal operands (the benchmark's) or zeros; "
                         "the difference in time is what the device's power management takes")
    ap.add_argument("--timed", action="store_true", help="with --profile-kernel on a flash kernel: also time the launch")
    ap.add_argument("--no-paged", action="store_true")
    ap.add_argument("--prewarm-seconds", type=float, default=0.5,
                    help="untimed steps run for this long before the counted --warmup steps (0 = none)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (every (batch, head) slice "
                 "is independent and would shard over batch or heads with no exchange). Run with --gpus 1.")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the kernels have no CPU fallback")

    if args.profile_kernel:
        profile_kernel(args, torch)
        return
    w, ms, value, roofline, kernels, step_frac = flash_step_bench(args, torch)
    out = {
        "metric": "TFLOP/s flash_attn fwd/bwd bf16 D=128 causal; paged decode HBM GB/s",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": w["name"], "batch": w["B"], "heads": w["H"], "seq_len": w["T"], "head_dim": w["D"]},
        "frac_of_mfma_peak": round(step_frac, 4),
        "roofline": roofline,
        "kernels": kernels,
    }
    out["matrix_pipe_ceiling"] = matrix_pipe_ceiling(torch)
    if not args.no_paged:
        # The other flash configurations of the workload list, as records of their own.
        legs = {"c2": (4, 16, 2048, 2048, 128), "c3": (1, 32, 8192, 8192, 128),
                "c3_d64": (1, 32, 8192, 8192, 64), "cross_length": (1, 32, 1024, 8192, 128)}
        legs.pop(args.workload, None)
        out["other_flash_workloads"] = {name: flash_step_leg(torch, *shape) for name, shape in legs.items()}
        out["paged_decode"] = paged_bench(torch)
        out["splitkv_decode"] = splitkv_bench(torch)
        out["piecewise"] = piecewise_bench(torch)
        out["total_attention"] = total_attention_bench(torch)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
