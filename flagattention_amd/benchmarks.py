"""Throughput sweeps of the operators: ``python -m flagattention_amd.benchmarks {flash,piecewise,decode,paged}``.

The sweeps are the ones of the reference's benchmark scripts, restated without ``triton.testing``:

* flash / piecewise (``benchmark/flash_benchmark.py:23-36, 45-58``, ``piecewise_benchmark.py:22-35``):
  sequence lengths 512 ... 32768 at a constant token count (batch = 32768 / T, heads = 2048 / D),
  D in {64, 128}, fwd and bwd, causal or not; TFLOP/s with ``4 B H T^2 D`` per forward (halved when
  causal) and 2.5x that per backward (``flash_benchmark.py:95-103``); piecewise is counted the same
  way (one dot product per score), not with the reference's 1.5x / 1.6x convention.
* decode (``flash_decoding_benchmark.py:22-47``): batch 2, heads 2048 / D, one query token against
  512 ... 2^19 keys through ``flash_attention``; reported in GB/s of K/V read.
* paged (``paged_benchmark.py:87-115``): 64 query heads, context 512 ... 16384 for
  {1, 32, 64} sequences x group {1, 8} x head {64, 128} x block {16, 32}; GB/s of K/V read once per
  kv head (the reference prints a pseudo TFLOP/s, ``paged_benchmark.py:184``, given here as well).

Each point: 5 warm-up calls, then the median of 20 event-timed calls.  ``--points N`` stops every
sweep after N measured points (a check that the sweeps run, not a measurement).
"""
import argparse
import statistics

import torch

import flagattention_amd as flag_attn


def _median_ms(fn, warmup=5, reps=20):
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(reps):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    return statistics.median(times)


def flash_flops(B, H, T, D, causal, mode):
    """Counted FLOPs of one call: only the matrix products (``flash_benchmark.py:95-103``)."""
    macs = 2.0 * B * H * T * T * D          # Q K^T and P V
    if mode == "bwd":
        macs *= 2.5                          # Q K^T, dO V^T, P^T dO, dS^T Q, dS K
    flops = 2.0 * macs
    return flops * 0.5 if causal else flops


def kv_bytes(rows, heads_kv, D, itemsize=2):
    """Bytes of keys and values that a decode call has to read: ``rows`` key rows per kv head."""
    return 2 * rows * heads_kv * D * itemsize


def paged_pseudo_flops(num_seqs, heads_q, ctx, D):
    """The figure the reference's paged sweep prints (``paged_benchmark.py:184``)."""
    return 2.0 * num_seqs * heads_q * 2 * ctx * D


class _Budget:
    """Counts measured points; a sweep asks ``spent()`` before each one."""

    def __init__(self, points):
        self.left = points

    def spent(self):
        if self.left is None:
            return False
        self.left -= 1
        return self.left < 0


def _dense_sweep(piecewise, quick, points=None):
    lengths = [2 ** i for i in range(9, 16)]
    budget, records = _Budget(points), []
    for mode in ("fwd", "bwd"):
        for causal in (False, True):
            for D in (64, 128):
                for dtype in ((torch.bfloat16,) if quick else (torch.float16, torch.bfloat16)):
                    row = []
                    for T in lengths[::2] if quick else lengths:
                        if budget.spent():
                            return records
                        B, H = 32768 // T, 2048 // D
                        n_in = 5 if piecewise else 3
                        ins = [torch.randn(B, H, T, D, dtype=dtype, device="cuda", requires_grad=(mode == "bwd"))
                               for _ in range(n_in)]
                        if piecewise:
                            fn = lambda: flag_attn.piecewise_attention(*ins, T // 2, causal=causal)
                        else:
                            fn = lambda: flag_attn.flash_attention(*ins, causal=causal)
                        flops = flash_flops(B, H, T, D, causal, mode)
                        if mode == "bwd":
                            o = fn()
                            do = torch.randn_like(o)
                            fn = lambda: torch.autograd.grad(o, ins, do, retain_graph=True)
                        ms = _median_ms(fn)
                        records.append(dict(op="piecewise" if piecewise else "flash", mode=mode, causal=causal, D=D,
                                            dtype=str(dtype)[6:], B=B, H=H, T=T, ms=ms, flops=flops,
                                            tflops=flops / (ms * 1e-3) / 1e12))
                        row.append(f"{T}: {records[-1]['tflops']:6.1f}")
                        del ins
                    name = "piecewise" if piecewise else "flash"
                    print(f"{name} {mode} causal={int(causal)} D={D} {str(dtype)[6:]:8s} TFLOP/s  " + "  ".join(row),
                          flush=True)
    return records


def _decode_sweep(quick, points=None):
    budget, records = _Budget(points), []
    for D in (64, 128):
        row = []
        for N in [2 ** i for i in range(9, 20, 2 if quick else 1)]:
            if budget.spent():
                return records
            B, H = 2, 2048 // D
            q = torch.randn(B, H, 1, D, dtype=torch.float16, device="cuda")
            k = torch.randn(B, H, N, D, dtype=torch.float16, device="cuda")
            v = torch.randn(B, H, N, D, dtype=torch.float16, device="cuda")
            ms = _median_ms(lambda: flag_attn.flash_attention(q, k, v, causal=False))
            nbytes = kv_bytes(B * N, H, D)
            records.append(dict(op="decode", D=D, B=B, H=H, N=N, ms=ms, bytes=nbytes, gbs=nbytes / (ms * 1e-3) / 1e9))
            row.append(f"{N}: {records[-1]['gbs']:6.0f}")
        print(f"decode D={D} float16 GB/s  " + "  ".join(row), flush=True)
    return records


def _paged_sweep(quick, points=None):
    heads_q = 64
    budget, records = _Budget(points), []
    for num_seqs in (1, 32, 64):
        for group in (1, 8):
            for D in (64, 128):
                for block in ((16,) if quick else (16, 32)):
                    heads_kv = heads_q // group
                    row = []
                    for ctx in [2 ** i for i in range(9, 15, 2 if quick else 1)]:
                        if budget.spent():
                            return records
                        blocks_per_seq = -(-ctx // block)
                        num_blocks = num_seqs * blocks_per_seq
                        q = torch.randn(num_seqs, heads_q, D, dtype=torch.float16, device="cuda")
                        kc = torch.randn(num_blocks, heads_kv, block, D, dtype=torch.float16, device="cuda")
                        vc = torch.randn_like(kc)
                        lens = torch.full((num_seqs,), ctx, dtype=torch.int32, device="cuda")
                        table = torch.randperm(num_blocks, device="cuda").reshape(num_seqs, blocks_per_seq).int()
                        ms = _median_ms(lambda: flag_attn.paged_attention(q, kc, vc, lens, table, D ** -0.5, ctx))
                        nbytes = kv_bytes(num_seqs * ctx, heads_kv, D)
                        gbs = nbytes / (ms * 1e-3) / 1e9
                        pseudo = paged_pseudo_flops(num_seqs, heads_q, ctx, D) / (ms * 1e-3) / 1e12
                        records.append(dict(op="paged", num_seqs=num_seqs, group=group, D=D, block=block, ctx=ctx,
                                            ms=ms, bytes=nbytes, gbs=gbs, pseudo_tflops=pseudo))
                        row.append(f"{ctx}: {gbs:6.0f} ({pseudo:5.1f})")
                    print(f"paged seqs={num_seqs} group={group} D={D} block={block} GB/s (pseudo TFLOP/s)  " + "  ".join(row),
                          flush=True)
    return records


SWEEPS = ("flash", "piecewise", "decode", "paged")


def run(which, quick=False, points=None):
    """Runs one sweep, prints its table and returns one record per measured point."""
    if not torch.cuda.is_available():
        raise SystemExit("the sweeps need a GPU: the kernels have no CPU fallback")
    return {"flash": lambda: _dense_sweep(False, quick, points), "piecewise": lambda: _dense_sweep(True, quick, points),
            "decode": lambda: _decode_sweep(quick, points), "paged": lambda: _paged_sweep(quick, points)}[which]()


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("which", choices=SWEEPS)
    ap.add_argument("--quick", action="store_true", help="every other size, one dtype")
    ap.add_argument("--points", type=int, default=None, help="stop after this many measured points")
    args = ap.parse_args(argv)
    run(args.which, args.quick, args.points)


if __name__ == "__main__":
    main()
