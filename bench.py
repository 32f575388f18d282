"""Benchmark of the single-GPU attention path on one MI355X.

Headline workload (``config.workload = "c3_rank_share"``): one context-parallel
rank's share of ring sliding-window attention — bf16, batch 1, local chunk 8192
tokens of a 65536-token sequence (virtual cp 8), 32 q / 8 kv heads, head_dim
128, window 4096: band attention on the rank's own chunk plus the upper-right
4096 x 4096 corner against the previous rank's chunk held in HBM (the reference
computes two blocks and merges them by LSE; here the two key ranges are one band
pass, the two-block form being timed beside it); forward + backward through
autograd.  One "step" = one such forward + backward.  ``value`` = window-effective TFLOP/s =
14 * D * pairs * Hq / time with pairs = 8192 * 4097 unmasked (query, key) pairs
per head.  Inputs are synthetic N(0,1), seeded, resident in HBM before timing.

Prints ONE JSON line.  ``python bench.py`` defaults to 1 GPU and finishes in
about a minute; ``--gpus N`` with N > 1 is refused (this build is single-GPU).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0     # MI355X HBM3E
# HBM bytes per launch (read + written) of the two roofline kernels at the shapes timed below,
# from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --pmc-pass`, each counter
# scaled by what it reads for the 1 GiB device copy of that pass (FETCH_SIZE x2.0, WRITE_SIZE
# x1.0); the summary is profiles/c3_step_kernels_hbm_traffic_pmc.txt.
DKDV_HBM_BYTES_PER_LAUNCH = 757.4e6
MERGE_HBM_BYTES_PER_LAUNCH = 5452.6e6
# Untimed steps before the W warm-up steps: an idle GPU takes some tens of milliseconds of load to
# settle its clocks (the first launches of a run take up to a third longer than the later ones), and
# W = 5 steps are 10 ms.
SPINUP_STEPS = 40


def band_pairs(length: int, w: int) -> int:
    return length * (length + 1) // 2 if length <= w + 1 else (w + 1) * length - w * (w + 1) // 2


def event_ms(fn, n, warm=3):
    """Median duration of fn() on torch's current stream (the stream the C ABI launches
    on), measured with HIP events."""
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
    evs[0].record()
    for i in range(n):
        fn()
        evs[i + 1].record()
    torch.cuda.synchronize()
    ts = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(n))
    return ts[len(ts) // 2], sum(ts) / len(ts)


def cpu_baseline(seconds_budget: float = 25.0):
    """The oracle (PyTorch masked softmax, fp32, autograd) on the host cores.

    ``value`` = the reference's own CPU-runnable case (fp32, batch 1, seq 1024, 4 q = 4 kv
    heads, head_dim 64, window 256, seed 0, scale 1/8, dO ~ N(0,1)): 2 warm-up + 5 timed
    forward+backward passes, median, converted with that case's 0.83 GFLOP.  Beside it a
    bounded sample of the headline workload's structure scaled down (4096 queries against
    8192 keys = own + previous chunk, window 2048, 4 q / 1 kv heads, head_dim 128)."""
    import torch

    from oracle import attention_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)

    def run(sq, sk, hq, hk, d, w, seed, warm, n_max, budget):
        torch.manual_seed(seed)
        q = torch.randn(1, sq, hq, d)
        k = torch.randn(1, sk, hk, d)
        v = torch.randn(1, sk, hk, d)
        do = torch.randn(1, sq, hq, d)
        fn = lambda: O.attention_fwd_bwd(  # noqa: E731
            lambda q, k, v: O.window_attention(q, k, v, d ** -0.5, (w, 0), True), q, k, v, do)
        for _ in range(warm):
            fn()
        ts = []
        t_start = time.perf_counter()
        while len(ts) < n_max and (time.perf_counter() - t_start < budget or len(ts) < 2):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        return ts[len(ts) // 2], len(ts)

    t1, n1 = run(1024, 1024, 4, 4, 64, 256, 0, 2, 5, seconds_budget / 2)
    c1_flops = 14 * 64 * band_pairs(1024, 256) * 4
    # sample of the rank share: queries = last 4096 positions of 8192 keys, window 2048
    sq, sk, hq, hk, d, w = 4096, 8192, 4, 1, 128, 2048
    t, n = run(sq, sk, hq, hk, d, w, 0, 1, 5, seconds_budget / 2)
    pairs = sq * (w + 1)  # every query has a full window inside the two chunks
    return {
        "value": c1_flops / t1 / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "threads": torch.get_num_threads(),
        "kind": "port",
        "sample": "oracle fp32 fwd+bwd (autograd) of the CPU case: batch 1, seq 1024, 4 q = 4 kv "
                  f"heads, head_dim 64, window 256, seed 0; median of {n1} passes {t1 * 1e3:.1f} ms "
                  f"= {c1_flops / t1 / 1e9:.1f} GFLOP/s",
        "c1_ms": t1 * 1e3,
        "scaled_down_rank_share": {
            "TFLOP/s": 14 * d * pairs * hq / t / 1e12, "ms": t * 1e3, "passes": n,
            "what": "4096 queries x 8192 keys (own + previous chunk), window 2048, 4 q / 1 kv "
                    "heads, head_dim 128, fp32"},
    }


def log_uniform_lengths(total, lo, hi, seed):
    """Sequence lengths drawn log-uniform in [lo, hi] until they cover ``total``, the last one
    truncated (the generator of the packed configuration)."""
    import math

    import torch

    g = torch.Generator().manual_seed(seed)
    lens = []
    while sum(lens) < total:
        x = math.exp(math.log(lo) + torch.rand(1, generator=g).item() * (math.log(hi) - math.log(lo)))
        lens.append(int(x))
    lens[-1] -= sum(lens) - total
    if lens[-1] == 0:
        lens.pop()
    return lens


def global_pairs_of_rows(cu, w, row0, row1, n_sink=0):
    """Visible (query, key) pairs of the packed rows [row0, row1): every row sees
    min(position in its sequence, w) + 1 keys, plus the sinks that lie before its window."""
    total = 0
    for a, b in zip(cu[:-1], cu[1:]):
        lo, hi = max(a, row0), min(b, row1)
        for p in range(lo, hi):
            pos = p - a
            total += min(pos, w) + 1 + max(0, min(n_sink, pos - w))
    return total


def _mk(dev):
    import torch

    return lambda *shape: torch.randn(*shape, device=dev, dtype=torch.bfloat16)


def clock_probe(dev, qd, kd, vd, prev, do, S, W, seconds=4.0):
    """Shader clock under each kernel of the step's band: every kernel is launched back to back
    for ``seconds`` while a thread asks ``rocm-smi --showclocks`` five times a second; reported
    are the median ``sclk`` of the readings taken after the first second and the kernel's launch
    time over the same period.  The published matrix peak is priced at 2400 MHz."""
    import re
    import statistics
    import subprocess
    import threading
    import time

    import torch

    from ring_swa.ops import attn_bwd, attn_fwd
    from ring_swa.ops.band_attn import bwd_workspace_bytes

    tk, tv = prev[0][:, S - W:], prev[1][:, S - W:]
    dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
    dtk, dtv = torch.empty_like(tk), torch.empty_like(tv)
    big, big2 = (torch.empty(1 << 28, dtype=torch.float32, device=dev) for _ in range(2))
    with torch.no_grad():
        o_b, lse_b = attn_fwd(qd, tk, tv, None, (W, 0), True, second=(kd, vd))
        ws = torch.empty(bwd_workspace_bytes(qd, tk, second_rows=S), dtype=torch.uint8, device=dev)
        band = lambda ph: attn_bwd(qd, tk, tv, o_b, lse_b, do, dq, dtk, dtv, None, (W, 0), True,  # noqa: E731
                                   workspace=ws, phases=ph, second=(kd, vd, dk, dv), handoff=False)
        band(7)
        kernels = [("attn_fwd_kernel", lambda: attn_fwd(qd, tk, tv, None, (W, 0), True, second=(kd, vd))),
                   ("attn_bwd_dkdv_kernel", lambda: band(2)),
                   ("attn_bwd_dq_kernel", lambda: band(4)),
                   ("device copy of 1 GiB", lambda: big2.copy_(big))]
        out = {}
        for name, fn in kernels:
            reads, stop = [], threading.Event()

            def sample():
                while not stop.is_set():
                    try:
                        txt = subprocess.run(["rocm-smi", "--showclocks", "--csv"], capture_output=True,
                                             text=True, timeout=20).stdout
                        m = re.search(r"\((\d+)Mhz\)[^()]*$", txt.strip().splitlines()[-1]) if txt.strip() else None
                        if m:
                            reads.append((time.time(), int(m.group(1))))
                    except (OSError, subprocess.SubprocessError):
                        pass
                    time.sleep(0.2)

            th = threading.Thread(target=sample)
            th.start()
            t0, times = time.time(), []
            while time.time() - t0 < seconds:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(50):
                    fn()
                e1.record()
                torch.cuda.synchronize()
                times.append(e0.elapsed_time(e1) / 50)
            stop.set()
            th.join()
            late = [mhz for (t, mhz) in reads if t - t0 > 1.0]
            out[name] = {"sclk_MHz_median": statistics.median(late) if late else None, "readings": len(late),
                         "launch_ms_median": statistics.median(times[len(times) // 4:])}
            time.sleep(1.0)
    return {"clock_probe": out, "nominal_MHz": 2400}


def case_c2(dev):
    """Configuration 2: plain single-GPU sliding-window attention, batch 2, seq 8192, 32 q = 32
    kv heads, head_dim 128, window 1000.  Returns (forward, backward, pairs x batch x heads)."""
    import torch

    from ring_swa.ops import attn_bwd, attn_fwd

    mk = _mk(dev)
    q2, k2, v2, do2 = (mk(2, 8192, 32, 128) for _ in range(4))
    o2, l2 = attn_fwd(q2, k2, v2, None, (1000, 0), True)
    g2 = [torch.empty_like(q2) for _ in range(3)]
    fwd = lambda: attn_fwd(q2, k2, v2, None, (1000, 0), True)  # noqa: E731
    bwd = lambda: attn_bwd(q2, k2, v2, o2, l2, do2, *g2, None, (1000, 0), True)  # noqa: E731
    return fwd, bwd, band_pairs(8192, 1000) * 2 * 32


def case_c4(dev):
    """Configuration 4: a pack of 32768 tokens (log-uniform lengths in [64, 16384], seed 0),
    32 q / 8 kv heads, head_dim 128, window 2048.  Two steps (forward + backward): one rank
    slice of virtual cp 4 whose chunk starts inside a sequence (diagonal packed block +
    rectangle on the previous chunk + merge), and the whole pack in one call."""
    import itertools

    import torch

    import ring_swa

    mk = _mk(dev)
    T4, CP4, W4, HQ, HK, D = 32768, 4, 2048, 32, 8, 128
    lens4 = log_uniform_lengths(T4, 64, 16384, seed=0)
    cu4 = [0] + list(itertools.accumulate(lens4))
    s4 = T4 // CP4
    r4 = next(r for r in range(1, CP4) if (r * s4) not in cu4)
    q4, do4 = mk(T4, HQ, D), mk(T4, HQ, D)
    k4, v4 = mk(T4, HK, D), mk(T4, HK, D)
    sl = slice(r4 * s4, (r4 + 1) * s4)
    ps = slice((r4 - 1) * s4, r4 * s4)
    qr, kr, vr = (t[sl].clone().requires_grad_() for t in (q4, k4, v4))
    pr = torch.stack([k4[ps], v4[ps]]).requires_grad_()
    do_r = do4[sl]

    @torch.enable_grad()
    def c4_slice():
        for t in (qr, kr, vr, pr):
            t.grad = None
        ring_swa.ring_rank_share_attn_varlen(qr, kr, vr, [pr], W4, cu4, CP4, r4).backward(do_r)

    cu4_dev = torch.tensor(cu4, dtype=torch.int32, device=dev)
    qg4, kg4, vg4 = (t.clone().requires_grad_() for t in (q4, k4, v4))

    @torch.enable_grad()
    def c4_whole():
        for t in (qg4, kg4, vg4):
            t.grad = None
        ring_swa.ring_sliding_window_attn_varlen(qg4, kg4, vg4, W4, cu4_dev, cp_size=1).backward(do4)

    info = {"sequences": len(lens4), "rank": r4,
            "pairs_slice": global_pairs_of_rows(cu4, W4, r4 * s4, (r4 + 1) * s4),
            "pairs_whole": sum(band_pairs(n, W4) for n in lens4)}
    return c4_slice, c4_whole, info


def case_c5(dev, impl, n_sink):
    """Configuration 5: packed streaming-LLM attention, 65536 tokens in 4 sequences (cut points
    inside the kernels' tiles), 32 q / 8 kv heads, head_dim 128, sinks + window 4092, sink keys
    scaled by 4.  Returns the forward + backward step and its pair count."""
    import torch

    import ring_swa

    mk = _mk(dev)
    T5, W5, HQ, HK, D = 65536, 4092, 32, 8, 128
    g5 = torch.Generator().manual_seed(0)
    cuts = sorted((torch.randperm(T5 // 1024 - 1, generator=g5)[:3] + 1).tolist())
    cu5 = [0] + [c * 1024 + 37 + 64 * i for i, c in enumerate(cuts)] + [T5]
    lens5 = [b - a for a, b in zip(cu5[:-1], cu5[1:])]
    cu5_dev = torch.tensor(cu5, dtype=torch.int32, device=dev)
    torch.manual_seed(5)
    q5, do5 = mk(T5, HQ, D), mk(T5, HQ, D)
    k5, v5 = mk(T5, HK, D), mk(T5, HK, D)
    for c in cu5[:-1]:
        k5[c:c + n_sink] *= 4
    qg, kg, vg = (t.requires_grad_() for t in (q5, k5, v5))
    kw = {} if n_sink == 1 else {"num_sink_tokens": n_sink}

    @torch.enable_grad()
    def c5_step():
        for t in (qg, kg, vg):
            t.grad = None
        ring_swa.ring_streaming_llm_attn_varlen(qg, kg, vg, W5, cu5_dev, cp_size=1, impl=impl,
                                                **kw).backward(do5)

    return c5_step, {"lengths": lens5, "pairs": global_pairs_of_rows(cu5, W5, 0, T5, n_sink)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the per-kernel / merge extras")
    ap.add_argument("--pmc-pass", action="store_true",
                    help="counter-collection pass: launch a 1 GiB device copy (the known-size "
                         "calibration kernel) and every hot kernel twice, then exit")
    ap.add_argument("--clock-probe", action="store_true",
                    help="loop each kernel of the step's band for a few seconds and print the shader "
                         "clock rocm-smi reads meanwhile (one JSON line; no timing claims)")
    ap.add_argument("--trace", choices=["c2", "c4", "c5"],
                    help="kernel-trace pass: run only that configuration's step a few times "
                         "(under rocprofv3 --kernel-trace --stats) and exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build covers the single-GPU path only; run with --gpus 1 "
                 "(one rank's share of the ring is emulated on that GPU)")

    import __graft_entry__ as entry

    entry.ensure_built()
    import torch

    import ring_swa
    from ring_swa.ops import attn_bwd, attn_fwd, merge_attn_out
    from ring_swa.ops.band_attn import bwd_workspace_bytes

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(0)

    # ---- headline workload ------------------------------------------------------
    S, HQ, HK, D, W, CP, RANK = 8192, 32, 8, 128, 4096, 8, 1
    mk = lambda *shape: torch.randn(*shape, device=dev, dtype=torch.bfloat16)  # noqa: E731
    q, k, v = mk(1, S, HQ, D).requires_grad_(), mk(1, S, HK, D).requires_grad_(), \
        mk(1, S, HK, D).requires_grad_()
    prev = mk(2, 1, S, HK, D).requires_grad_()
    do = mk(1, S, HQ, D)
    pairs_diag = band_pairs(S, W)
    pairs_off = W * (W + 1) // 2
    pairs = pairs_diag + pairs_off
    assert pairs == S * (W + 1)
    flops = 14 * D * pairs * HQ

    def step():
        for t in (q, k, v, prev):
            t.grad = None
        out = ring_swa.ring_rank_share_attn(q, k, v, [prev], W, CP, RANK)
        out.backward(do)

    if args.trace:
        if args.trace == "c2":
            f2, b2, _ = case_c2(dev)
            steps = [lambda: (f2(), b2())]
        elif args.trace == "c4":
            steps = list(case_c4(dev)[:2])
        else:
            steps = [case_c5(dev, "fused", 4)[0]]
        for fn in steps:
            for _ in range(args.steps):
                fn()
        torch.cuda.synchronize()
        print(json.dumps({"trace_pass": args.trace, "steps": args.steps}))
        return

    if args.clock_probe:
        print(json.dumps(clock_probe(dev, q.detach(), k.detach(), v.detach(), prev.detach(), do, S, W)))
        return

    if args.pmc_pass:
        with torch.no_grad():
            src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
            dst = torch.empty_like(src)
            qd, kd, vd = q.detach(), k.detach(), v.detach()
            dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
            acc = torch.randn(1, 131072, HQ, D, device=dev)
            lacc = torch.randn(1, HQ, 131072, device=dev, dtype=torch.float64)
            new = torch.randn(1, 131072, HQ, D, device=dev, dtype=torch.bfloat16)
            lnew = torch.randn(1, HQ, 131072, device=dev)
            tk, tv = prev.detach()[0][:, S - W:], prev.detach()[1][:, S - W:]
            dtk, dtv = torch.empty_like(tk), torch.empty_like(tv)
            for _ in range(2):
                dst.copy_(src)  # reads 1 GiB, writes 1 GiB
                o_d, lse_d = attn_fwd(qd, kd, vd, None, (W, 0), True)
                attn_bwd(qd, kd, vd, o_d, lse_d, do, dq, dk, dv, None, (W, 0), True)
                merge_attn_out(acc, lacc, new, lnew)
                # the rank step's band: keys = previous chunk's tail, then the own chunk
                o_b, lse_b = attn_fwd(qd, tk, tv, None, (W, 0), True, second=(kd, vd))
                attn_bwd(qd, tk, tv, o_b, lse_b, do, dq, dtk, dtv, None, (W, 0), True,
                         second=(kd, vd, dk, dv))
                # the same backward on the dS hand-off route (dK/dV kernel <..., 1> stores its
                # dS tiles, attn_bwd_dq_ds_kernel reads them)
                attn_bwd(qd, tk, tv, o_b, lse_b, do, dq, dtk, dtv, None, (W, 0), True,
                         second=(kd, vd, dk, dv), handoff=True)
            torch.cuda.synchronize()
        print(json.dumps({"pmc_pass": "done", "copy_bytes_each_way": 1 << 30}))
        return

    for _ in range(SPINUP_STEPS + args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    value = flops / (ms * 1e-3) / 1e12

    rec = {
        "metric": "fwd+bwd window-effective TFLOP/s + % bf16 MFMA peak; merge GB/s, 1 MI355X",
        "value": value,
        "unit": "TFLOP/s",
        "pct_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "spinup_steps": SPINUP_STEPS,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "c3_rank_share",
            "detail": "1 rank of virtual cp 8: chunk 8192 of seq 65536, 32 q / 8 kv heads, head_dim "
                      "128, window 4096; fwd+bwd via autograd; route one_pass: the previous chunk's "
                      "last 4096 rows and the own chunk, each where it lies, as one band pass "
                      "(ms_per_step_two_blocks / ms_per_step_ring_dtypes: the reference's two blocks + "
                      "LSE merge, with 16-bit and with fp32 / fp64 accumulators)",
            "route": "one_pass",
            "ring_dtypes": False,
            "batch": 1, "chunk": S, "heads_q": HQ, "heads_kv": HK, "head_dim": D, "window": W,
            "pairs_per_head": pairs, "flops_per_step": flops,
        },
    }

    # the same step with the reference's accumulator types (fp32 output, fp64 LSE, merged
    # through the block operators; two cast passes)
    def step_ring_dtypes():
        for t in (q, k, v, prev):
            t.grad = None
        out = ring_swa.ring_rank_share_attn(q, k, v, [prev], W, CP, RANK, ring_dtypes=True)
        out.backward(do)

    # ... and as the reference's two blocks merged in 16 bits (own-chunk block, previous-chunk
    # corner block merged in the second forward's epilogue, dq summed in the own-chunk dQ kernel)
    def step_two_blocks():
        for t in (q, k, v, prev):
            t.grad = None
        out = ring_swa.ring_rank_share_attn(q, k, v, [prev], W, CP, RANK, one_pass=False)
        out.backward(do)

    for name, fn in (("ms_per_step_ring_dtypes", step_ring_dtypes),
                     ("ms_per_step_two_blocks", step_two_blocks)):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        rec[name] = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- roofline of the dominant kernel: the backward dK/dV kernel on the step's band ----
    # (8192 queries against the previous chunk's 4096-row tail and the own chunk, window 4096:
    # the launch the step makes; the own-chunk block alone is timed with the extras)
    # Algorithmic FLOPs per visible (query, key) pair and q head: forward 4 D (S, PV);
    # dK/dV kernel 8 D (S, dP, dV, dK); dQ kernel 6 D (S, dP, dQ); the backward as a whole
    # is credited 10 D (S and dP counted once), as in the headline metric.
    with torch.no_grad():
        qd, kd, vd = q.detach(), k.detach(), v.detach()
        o_d, lse_d = attn_fwd(qd, kd, vd, None, (W, 0), True)
        dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
        ws = torch.empty(bwd_workspace_bytes(qd, kd), dtype=torch.uint8, device=dev)
        bwd = lambda ph: attn_bwd(qd, kd, vd, o_d, lse_d, do, dq, dk, dv, None, (W, 0), True,  # noqa: E731
                                  workspace=ws, phases=ph)
        bwd(7)
        n = 5 if args.no_extras else 20
        PREP, DKDV, DQ = 1, 2, 4
        fl_pair = D * pairs_diag * HQ
        tk, tv = prev.detach()[0][:, S - W:], prev.detach()[1][:, S - W:]
        dtk, dtv = torch.empty_like(tk), torch.empty_like(tv)
        o_b, lse_b = attn_fwd(qd, tk, tv, None, (W, 0), True, second=(kd, vd))
        ws_b = torch.empty(bwd_workspace_bytes(qd, tk, second_rows=S), dtype=torch.uint8, device=dev)
        band = lambda ph: attn_bwd(qd, tk, tv, o_b, lse_b, do, dq, dtk, dtv, None, (W, 0), True,  # noqa: E731
                                   workspace=ws_b, phases=ph, second=(kd, vd, dk, dv))
        band(7)
        fl_band = D * pairs * HQ
        dkdv_med, dkdv_avg = event_ms(lambda: band(DKDV), n)
        rec["roofline"] = {
            "kernel": "attn_bwd_dkdv_kernel<bf16,128> (the step's band: 8192 queries x "
                      "[4096-row tail of the previous chunk | own chunk 8192], window 4096)",
            "bound": "mfma",
            "achieved": 8 * fl_band / (dkdv_avg * 1e-3) / 1e12,
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": 8 * fl_band / (dkdv_avg * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
            "traffic": DKDV_HBM_BYTES_PER_LAUNCH,
            "avg_launch_ms": dkdv_avg,
            "median_launch_ms": dkdv_med,
            "flops_per_launch": 8 * fl_band,
        }
        if not args.no_extras:
            band_fwd, _ = event_ms(lambda: attn_fwd(qd, tk, tv, None, (W, 0), True,
                                                    second=(kd, vd)), 20)
            band_dq, _ = event_ms(lambda: band(DQ), 20)
            band_prep, _ = event_ms(lambda: band(PREP), 20)
            dkdv_med, dkdv_avg = event_ms(lambda: bwd(DKDV), n)
            fwd_med, _ = event_ms(lambda: attn_fwd(qd, kd, vd, None, (W, 0), True), 20)
            dq_med, _ = event_ms(lambda: bwd(DQ), 20)
            prep_med, _ = event_ms(lambda: bwd(PREP), 20)
            bwd_med, _ = event_ms(lambda: bwd(7), 20)
            tf = lambda fl, ms_: fl / ms_ / 1e9  # noqa: E731
            rec["kernels"] = {
                "fwd_step_band": {"ms": band_fwd, "TFLOP/s": tf(4 * fl_band, band_fwd),
                                  "flops_per_pair": "4 D"},
                "bwd_dkdv_step_band": {"ms": rec["roofline"]["median_launch_ms"],
                                       "TFLOP/s": tf(8 * fl_band, rec["roofline"]["median_launch_ms"]),
                                       "flops_per_pair": "8 D"},
                "bwd_dq_step_band": {"ms": band_dq, "TFLOP/s": tf(6 * fl_band, band_dq),
                                     "flops_per_pair": "6 D"},
                "bwd_prep_step_band": {"ms": band_prep},
                "fwd_own_chunk": {"ms": fwd_med, "TFLOP/s": tf(4 * fl_pair, fwd_med),
                                  "flops_per_pair": "4 D"},
                "bwd_dkdv_own_chunk": {"ms": dkdv_med, "TFLOP/s": tf(8 * fl_pair, dkdv_med),
                                       "flops_per_pair": "8 D"},
                "bwd_dq_own_chunk": {"ms": dq_med, "TFLOP/s": tf(6 * fl_pair, dq_med),
                                     "flops_per_pair": "6 D"},
                "bwd_prep_own_chunk": {"ms": prep_med},
                "bwd_own_chunk_all_kernels": {"ms": bwd_med, "TFLOP/s": tf(10 * fl_pair, bwd_med),
                                              "flops_per_pair": "10 D (window-effective)"},
            }
            # the band's backward on the dS hand-off route, beside the recomputing one above
            ws_h = torch.empty(bwd_workspace_bytes(qd, tk, second_rows=S, window_size=(W, 0), causal=True,
                                                   handoff=True), dtype=torch.uint8, device=dev)
            hand = lambda ph: attn_bwd(qd, tk, tv, o_b, lse_b, do, dq, dtk, dtv, None, (W, 0), True,  # noqa: E731
                                       workspace=ws_h, phases=ph, second=(kd, vd, dk, dv), handoff=True)
            hand(7)
            h_dkdv, _ = event_ms(lambda: hand(DKDV), 20)
            h_dq, _ = event_ms(lambda: hand(DQ), 20)
            h_all, _ = event_ms(lambda: hand(7), 20)
            r_all, _ = event_ms(lambda: band(7), 20)
            rec["kernels"]["bwd_step_band_ds_handoff"] = {
                "dkdv_ms": h_dkdv, "dq_ms": h_dq, "all_kernels_ms": h_all,
                "recompute_all_kernels_ms": r_all, "ds_bytes": ws_h.numel() - ws_b.numel(),
                "note": "opt-in route: the dK/dV kernel stores its 16-bit dS tiles (2 bytes per pair "
                        "and head), the dQ kernel only multiplies them with K"}
            del ws_h
            # The dK/dV launch of the own-chunk block alone leaves a quarter of the compute
            # units idle in its tail (256 blocks of unequal length on 256 units); in the
            # two-block form of the rank step the previous-chunk dK/dV launch of the second
            # stream fills them.  The pair, launched that way, is timed here for reference.
            pk, pv_ = prev.detach()[0][:, S - W:], prev.detach()[1][:, S - W:]
            o_p, lse_p = o_d[:, :W], lse_d[:, :, :W]
            dqp = torch.empty_like(qd[:, :W])
            dkp, dvp = torch.empty_like(pk), torch.empty_like(pv_)
            ws_p = torch.empty(bwd_workspace_bytes(qd[:, :W], pk), dtype=torch.uint8, device=dev)
            side = torch.cuda.Stream(dev)
            attn_bwd(qd[:, :W], pk, pv_, o_p, lse_p, do[:, :W], dqp, dkp, dvp, None, (0, S), False,
                     workspace=ws_p, phases=PREP)

            def dkdv_pair():
                side.wait_stream(torch.cuda.current_stream(dev))
                with torch.cuda.stream(side):
                    attn_bwd(qd[:, :W], pk, pv_, o_p, lse_p, do[:, :W], dqp, dkp, dvp, None,
                             (0, S), False, workspace=ws_p, phases=DKDV)
                bwd(DKDV)
                torch.cuda.current_stream(dev).wait_stream(side)

            pair_med, _ = event_ms(dkdv_pair, 20)
            rec["kernels"]["bwd_dkdv_own_and_previous_chunk_concurrent"] = {
                "ms": pair_med, "TFLOP/s": tf(8 * D * pairs * HQ, pair_med),
                "pct_bf16_mfma_peak": 100.0 * tf(8 * D * pairs * HQ, pair_med) / PEAK_BF16_TFLOPS,
                "flops_per_pair": "8 D", "note": "two launches on two streams, as in the two-block form of the rank step"}
            # the other GPU configurations of the suite (see the case_* functions)
            f2, b2, p2 = case_c2(dev)
            f2_ms, _ = event_ms(f2, 10)
            b2_ms, _ = event_ms(b2, 10)
            rec["c2_swa_b2_s8192_h32_w1000"] = {
                "fwd_ms": f2_ms, "bwd_ms": b2_ms, "TFLOP/s": tf(14 * 128 * p2, f2_ms + b2_ms),
                "pct_bf16_mfma_peak": tf(14 * 128 * p2, f2_ms + b2_ms) / PEAK_BF16_TFLOPS * 100}
            del f2, b2
            c4_slice, c4_whole, info4 = case_c4(dev)
            t_slice, _ = event_ms(c4_slice, 10)
            t_whole, _ = event_ms(c4_whole, 10)
            rate = lambda p_, t_: {"ms": t_, "pairs_per_head": p_, "TFLOP/s": tf(14 * D * p_ * HQ, t_),  # noqa: E731
                                   "pct_bf16_mfma_peak": tf(14 * D * p_ * HQ, t_) / PEAK_BF16_TFLOPS * 100}
            rec["c4_varlen_t32768_w2048"] = {
                "sequences": info4["sequences"], "rank": info4["rank"],
                "rank_slice": rate(info4["pairs_slice"], t_slice),
                "whole_pack_one_call": rate(info4["pairs_whole"], t_whole)}
            del c4_slice, c4_whole
            c5 = {}
            for n_sink in (1, 4):
                for impl in ("fused", "split"):
                    c5_step, info5 = case_c5(dev, impl, n_sink)
                    t5, _ = event_ms(c5_step, 5, warm=2)
                    c5["lengths"] = info5["lengths"]
                    c5[f"{impl}_sinks{n_sink}"] = rate(info5["pairs"], t5)
                    del c5_step
            rec["c5_slm_varlen_t65536_w4092"] = c5
            # a pack of 4096 sequences of 16 tokens (8 q / 2 kv heads, window 8): every block has
            # to find its sequence among 4096 -- a linear search took milliseconds here
            n_seq, L_seq = 4096, 16
            cu_m = torch.arange(0, (n_seq + 1) * L_seq, L_seq, dtype=torch.int32, device=dev)
            qm, dom = mk(n_seq * L_seq, 8, D), mk(n_seq * L_seq, 8, D)
            km, vm = mk(n_seq * L_seq, 2, D), mk(n_seq * L_seq, 2, D)
            gm = [torch.empty_like(t) for t in (qm, km, vm)]

            def many():
                om, lm = attn_fwd(qm, km, vm, None, (8, 0), True, cu_m, cu_m)
                attn_bwd(qm, km, vm, om, lm, dom, *gm, None, (8, 0), True, cu_m, cu_m)

            rec["pack_of_4096_sequences_of_16_fwd_bwd_ms"] = event_ms(many, 10)[0]
            del qm, dom, km, vm, gm
            T5 = 65536
            # the merge of that configuration's split path: all tokens x 32 heads, 16-bit
            # outputs and fp32 LSE on both sides (780 bytes per row)
            acc = torch.randn(1, T5, HQ, D, device=dev).bfloat16()
            lacc = torch.randn(1, HQ, T5, device=dev)
            new = torch.randn(1, T5, HQ, D, device=dev).bfloat16()
            lnew = torch.randn(1, HQ, T5, device=dev)
            med, avg = event_ms(lambda: merge_attn_out(acc, lacc, new, lnew), 20)
            nbytes = T5 * HQ * (6 * D + 12)
            merge_c5 = {"rows": T5 * HQ, "bytes": nbytes, "us": med * 1e3, "GB/s": nbytes / med / 1e6,
                        "pct_hbm_peak": nbytes / med / 1e6 / PEAK_HBM_GBPS * 100,
                        "dtypes": "o bf16, new o bf16, lse fp32, new lse fp32"}
            del acc, lacc, new, lnew
            # merge kernel: rank-share shape (rows [:4096] x 32 heads) and the sweep's top point
            merges = {}
            for name, rows_s in (("c3_rows4096", 4096), ("sweep_s131072", 131072)):
                acc = torch.randn(1, rows_s, HQ, D, device=dev)
                lacc = torch.randn(1, HQ, rows_s, device=dev, dtype=torch.float64)
                new = torch.randn(1, rows_s, HQ, D, device=dev, dtype=torch.bfloat16)
                lnew = torch.randn(1, HQ, rows_s, device=dev)
                med, avg = event_ms(lambda: merge_attn_out(acc, lacc, new, lnew), 20)
                nbytes = rows_s * HQ * (10 * D + 20)
                merges[name] = {"rows": rows_s * HQ, "bytes": nbytes, "us": med * 1e3,
                                "GB/s": nbytes / med / 1e6,
                                "dtypes": "o fp32, new o bf16, lse fp64, new lse fp32"}
                if name == "sweep_s131072":
                    # the same number of bytes through the library's plain copy kernel (half
                    # read, half written), same run: what a kernel that only moves memory reaches
                    from ring_swa.ops.lse_merge import stream_copy

                    src = torch.empty(nbytes // 2 // 16 * 16, dtype=torch.uint8, device=dev)
                    dst = torch.empty_like(src)
                    cmed, cavg = event_ms(lambda: stream_copy(dst, src), 20)
                    rec["copy_GBps"] = 2 * src.numel() / cavg / 1e6
                    merges["sweep_s131072"]["copy_kernel_same_bytes"] = {
                        "us": cavg * 1e3, "GB/s": rec["copy_GBps"],
                        "merge_over_copy": (nbytes / avg) / (2 * src.numel() / cavg)}
                    del src, dst
                    rec["roofline_merge"] = {
                        "kernel": "merge_kernel<float,bf16,16>", "bound": "hbm",
                        "achieved": nbytes / avg / 1e6, "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                        "frac": nbytes / avg / 1e6 / PEAK_HBM_GBPS,
                        "traffic": MERGE_HBM_BYTES_PER_LAUNCH,
                        "avg_launch_ms": avg, "bytes_per_launch": nbytes}
                del acc, lacc, new, lnew
            # the reference's merge-only sweep (ring_swa/ops/merge.py:257-302): B 1, H 32, D 128
            sweep = {}
            for rows_s in (1024, 4096, 16384, 65536, 131072):
                acc = torch.randn(1, rows_s, HQ, D, device=dev)
                lacc = torch.randn(1, HQ, rows_s, device=dev, dtype=torch.float64)
                new = torch.randn(1, rows_s, HQ, D, device=dev, dtype=torch.bfloat16)
                lnew = torch.randn(1, HQ, rows_s, device=dev)
                med, _ = event_ms(lambda: merge_attn_out(acc, lacc, new, lnew), 20)
                sweep[f"s{rows_s}"] = {"us": med * 1e3,
                                       "GB/s": rows_s * HQ * (10 * D + 20) / med / 1e6}
                del acc, lacc, new, lnew
            merges["sweep_ring_dtypes"] = sweep
            merges["c5_rows65536_naive_dtypes"] = merge_c5
            rec["merge"] = merges
            rec["merge_GBps"] = merges["sweep_s131072"]["GB/s"]

    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
