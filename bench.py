#!/usr/bin/env python3
"""Headline benchmark: fp16 GEMV bandwidth over the Llama2-7B decode sweep on one MI355X.

A step is one pass of the hot path over the four decode shapes (N<-K): 4096<-4096 (wq/wk/wv/wo),
11008<-4096 (w1/w3), 4096<-11008 (w2, split-K) and 32000<-4096 (classifier), each through
tl_matmul2d_f16 with M == 1.  Inputs are resident in HBM before the timed region; weights rotate
over several buffer sets (> 1 GB in total) so every launch streams W from HBM, not from the
256 MB Infinity Cache.

Prints ONE JSON line.  `value` = algorithmic bytes of a step / wall time of a step (GB/s,
decimal).  `roofline` = the GEMV kernel against the 8 TB/s HBM peak, from a HIP event pair
recorded on the launch stream around the timed region.  `cpu_baseline` = the CPU oracle
(a port of the reference's OpenMP CPU<half>::matmul2d) timed on this host on the same sweep.
`extra` carries per-shape GEMV numbers, prefill HGEMM TFLOP/s (against the published MFMA peak and
against the MFMA rate this chip sustains out of registers) and Llama2-7B decode tok/s.

`--workload hgemm` times only the prefill HGEMM shapes (step = one pass over the M=2048 shapes)
and prints the same kind of line with an MFMA roofline; it exists so that the MFMA profile under
profiles/ can be taken from a committed command.  `--workload decode` does the same for the
Llama2-7B decode step (step = one generated token of the fused driver after a 128-token prompt).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published

SWEEP = [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)]
# prefill shapes (M, N, K)
HGEMM_SHAPES = [(2048, 4096, 4096), (2048, 11008, 4096), (2048, 32000, 4096), (2048, 4096, 11008),
                (512, 4096, 4096), (512, 11008, 4096), (512, 32000, 4096), (512, 4096, 11008),
                (128, 4096, 4096), (128, 11008, 4096), (128, 32000, 4096), (128, 4096, 11008)]

# HBM bytes per GEMV launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), averaged over
# the four sweep launches and scaled by the same counters' reading for a copy kernel of known
# size (FETCH_SIZE x 1.9997 KiB, WRITE_SIZE x 1.0000 KiB); algorithmic bytes per launch are 119,050,624.
# Counters cannot be read inside this process: the figure comes from the profile named beside it and is
# reported with that source, not re-measured by a bench run.
GEMV_TRAFFIC_BYTES_PER_LAUNCH = 119_420_779
GEMV_TRAFFIC_SOURCE = "profiles/gemv_decode_sweep_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command)"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["gemv", "hgemm", "decode", "gemv_timeline", "gemv_grid", "hgemm_timeline"], default="gemv")
    ap.add_argument("--rows", default="2048",
                    help="--workload hgemm: row counts M of the prefill shapes that form the timed step, comma separated, "
                         "from 16 (the four projections of a 16-token prompt), 128, 512, 2048")
    ap.add_argument("--splitk-merge", type=int, default=0, choices=[0, 1, 2],
                    help="--workload hgemm: where a split K is added up (tl_set_hgemm_splitk_merge): 0/2 second kernel, "
                         "1 inside the GEMM launch")
    ap.add_argument("--hgemm-variant", default="",
                    help="--workload hgemm: force one kernel variant by name (tl_hgemm_variant_name), default dispatch")
    ap.add_argument("--vendor-reference", action="store_true",
                    help="--workload hgemm: time torch.matmul (hipBLASLt) on the same operands next to the library, "
                         "alternating, and report both per shape in extra.hgemm_prefill")
    ap.add_argument("--no-extra", action="store_true", help="skip the HGEMM / per-shape / model extras")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch plain 256 MiB copies (strided_copy_kernel) so that a rocprofv3 --pmc run "
                         "of this command holds a kernel of known HBM traffic next to the GEMV")
    return ap.parse_args()


def cpu_baseline_gemv(budget_s: float = 10.0):
    """Time the CPU oracle on the full decode sweep (all four shapes, every row)."""
    import numpy as np
    from oracle import oracle
    from tensorlib_amd import synth
    mats = []
    for i, (N, K) in enumerate(SWEEP):
        mats.append((synth.normal_f16(10 + i, (N, K), 0.02), synth.normal_f16(20 + i, (1, K), 1.0)))
    oracle.matmul2d(mats[0][1], mats[0][0])  # warm-up (thread pool, tables)
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 5000):
        t0 = time.perf_counter()
        for W, x in mats:
            oracle.matmul2d(x, W)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    total_bytes = sum(synth.gemv_bytes(N, K) for N, K in SWEEP)
    return {
        "value": round(total_bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": oracle.max_threads(),
        "kind": "port",
        "sample": f"full decode sweep (4 GEMVs, {total_bytes} B), median of {len(times)} passes, "
                  f"{med * 1e3:.1f} ms per pass",
    }


def cpu_baseline_hgemm():
    """Time the CPU oracle on 16 rows of X of the 2048x4096x4096 prefill GEMM (0.27 G multiply-adds)."""
    import numpy as np
    from oracle import oracle
    from tensorlib_amd import synth
    rows, N, K = 16, 4096, 4096
    A = synth.normal_f16(30, (rows, K), 1.0)
    B = synth.normal_f16(31, (N, K), 0.02)
    oracle.matmul2d(A, B)
    times = []
    for _ in range(7):
        t0 = time.perf_counter()
        oracle.matmul2d(A, B)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {
        "value": round(2.0 * rows * N * K / med / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": oracle.max_threads(),
        "kind": "port",
        "sample": f"{rows} rows of X of the 2048x4096x4096 shape ({rows}x{N}x{K}), median of 7 runs, "
                  f"{med * 1e3:.1f} ms; full shape would take {med * 2048 / rows:.2f} s (extrapolated)",
    }


def cpu_baseline_llama2_decode(k: int = 6):
    """Time k single-token decode steps of the CPU oracle's Llama2 op chain at Llama2-7B size (32 layers of
    dim 4096 / hidden 11008 / 32 heads, vocabulary 32000, context 128..128+k).  Bounded sample: the 32 layers
    cycle over two distinct random-init weight sets (2 x 405 MB, far beyond the host caches, so every GEMV still
    streams its matrix from memory as 32 distinct layers would) instead of 13 GB drawn fresh; the embedding table
    shares the classifier's array.  Arithmetic per step is exactly that of the full model."""
    import numpy as np
    from oracle import oracle
    from oracle.llama2_oracle import Llama2Oracle
    from tensorlib_amd import synth
    dim, hidden, L, H, vocab = 4096, 11008, 32, 32, 32000
    w = {"classifier": synth.normal_f16(900, (vocab, dim), 0.02), "final_norm": synth.normal_f16(901, (dim,), 1.0)}
    w["tok_emb"] = w["classifier"]
    distinct = 2
    for s in range(distinct):
        base = {"att_norm": synth.normal_f16(910 + 20 * s, (dim,), 1.0), "ffn_norm": synth.normal_f16(911 + 20 * s, (dim,), 1.0)}
        for i, n in enumerate(("wq", "wk", "wv", "wo")):
            base[n] = synth.normal_f16(912 + 20 * s + i, (dim, dim), 0.02)
        base["w1"] = synth.normal_f16(916 + 20 * s, (hidden, dim), 0.02)
        base["w3"] = synth.normal_f16(917 + 20 * s, (hidden, dim), 0.02)
        base["w2"] = synth.normal_f16(918 + 20 * s, (dim, hidden), 0.02)
        for l in range(s, L, distinct):
            for n, a in base.items():
                w[f"{n}.{l}"] = a
    start = 128
    m = Llama2Oracle(w, dim, hidden, L, H, vocab, start + k + 1, 1e-5)
    for l in range(L):   # a context of 128 positions already in the cache
        m.cache_k[l][:start] = synth.normal_f16(950, (start, H, dim // H), 1.0)
        m.cache_v[l][:start] = synth.normal_f16(951, (start, H, dim // H), 1.0)
    toks = synth.token_ids(960, k + 1, vocab)
    m.forward(toks[:1], start)   # warm-up step (thread pool, page faults)
    times = []
    for i in range(k):
        t0 = time.perf_counter()
        m.forward(toks[i + 1:i + 2], start + 1 + i)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return {"value": round(1.0 / med, 3), "unit": "tok/s", "cores": oracle.max_threads(), "kind": "port",
            "sample": f"{k} teacher-forced single-token steps of the oracle's op chain at Llama2-7B size, context 129..{start + k}, "
                      f"layers cycling over {distinct} distinct weight sets; median {med * 1e3:.0f} ms per token"}


def time_region(fn, reps: int, torch):
    """Run fn() reps times between a HIP event pair on the current (= library) stream; returns
    (wall seconds, event seconds)."""
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) * 1e-3


def mfma_sustained(dev):
    """MFMA rate out of registers: constant operands vs operands changing with every instruction, for the 32x32x16
    instruction (the ring kernels') and the 16x16x32 one (the AGPR kernels')."""
    import ctypes
    out = {}
    for name, mode in (("constant_operands", 0), ("changing_operands", 1), ("constant_operands_16x16x32", 2),
                       ("changing_operands_16x16x32", 3)):
        v = ctypes.c_double()
        from tensorlib_amd._lib import check
        check(dev.lib.tl_measure_mfma_rate_f16(mode, ctypes.byref(v)), "tl_measure_mfma_rate_f16")
        out[name] = round(v.value, 1)
    return out


def hgemm_table(dev, randn, torch, synth, sustained_tf, shapes=None, vendor=False):
    """Per-shape times of tl_matmul2d_f16 with W streamed from HBM.  vendor: also time torch.matmul (hipBLASLt / rocBLAS
    behind it) on the same operands, alternating with the library in three rounds, minimum kept for both: a reference
    point on the same box, not a product path."""
    hg = {}
    for (M, N, K) in (shapes or HGEMM_SHAPES):
        A = randn((M, K), 1.0)
        # W rotates over enough copies (>= 600 MB) that every launch streams it from HBM, as a forward pass
        # over 32 layers does; one 33-180 MB matrix used again and again would sit in the 256 MB memory-side cache
        nb = max(2, -(-600_000_000 // (N * K * 2)))
        Bs = [randn((N, K), 0.02) for _ in range(nb)]
        C = torch.empty((M, N), device="cuda", dtype=torch.float16)
        it = [0]

        def one():
            it[0] += 1
            dev.matmul2d(A, Bs[it[0] % nb], C)
        for _ in range(5):
            one()
        reps = 40
        _, ev1 = time_region(one, reps, torch)
        vendor_us = None
        if vendor:
            def other():
                it[0] += 1
                torch.matmul(A, Bs[it[0] % nb].T, out=C)
            for _ in range(5):
                other()
            vendor_ev = []
            for _ in range(3):
                vendor_ev.append(time_region(other, reps, torch)[1])
                ev1 = min(ev1, time_region(one, reps, torch)[1])
            vendor_us = min(vendor_ev) / reps * 1e6
        del Bs
        us = ev1 / reps * 1e6
        tf = synth.gemm_flops(M, N, K) / us / 1e6
        ai = synth.gemm_flops(M, N, K) / synth.gemm_min_bytes(M, N, K)
        bound_tf = min(MFMA_FP16_PEAK_TFLOPS, ai * HBM_PEAK_GBS / 1e3)
        plan = dev.hgemm_last_plan()
        hg[f"{M}x{N}x{K}"] = {"us": round(us, 1), "TFLOP/s": round(tf, 1), "kernel": plan[0], "k_splits": plan[1],
                              "frac_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS, 4),
                              "bound": "mfma" if bound_tf >= MFMA_FP16_PEAK_TFLOPS else "hbm",
                              "frac_of_bound": round(tf / bound_tf, 4),
                              "frac_of_sustained_mfma": round(tf / sustained_tf, 4)}
        if vendor_us is not None:
            hg[f"{M}x{N}x{K}"]["torch_matmul_us"] = round(vendor_us, 1)
            hg[f"{M}x{N}x{K}"]["us_over_torch_matmul_us"] = round(us / vendor_us, 3)
    return hg


def gemv_timeline(dev, randn, torch, launches: int):
    """Where the time of a 4096<-4096 GEMV launch goes: `launches` back-to-back launches of the stamped build of the
    dispatch's kernel (tl_gemv_f16_stamped), each on its own matrix (> 1 GB in rotation, so W comes from HBM) and
    its own stamp buffer.  Per launch: all workgroups started / first workgroup done / 10, 50, 90, 100 % of the
    workgroups done, in microseconds after the first workgroup's start, and the period from one launch's first
    start to the next one's (the share of it outside the first-start-to-last-end window is what the launch
    boundary costs).  Medians over the launches; the GPU's constant counter ticks every 10 ns."""
    import ctypes
    import numpy as np
    from tensorlib_amd._lib import check
    N = K = 4096
    launches = max(8, min(launches, 200))
    nbuf = 32
    Ws = [randn((N, K), 0.02) for _ in range(nbuf)]
    x = randn((1, K), 1.0)
    y = torch.empty((1, N), device="cuda", dtype=torch.float16)
    wgs = N // 2
    stamps = torch.zeros((launches, wgs, 2), device="cuda", dtype=torch.int64)
    n = ctypes.c_int(0)

    def run():
        for i in range(launches):
            check(dev.lib.tl_gemv_f16_stamped(x.data_ptr(), Ws[i % nbuf].data_ptr(), y.data_ptr(), N, K,
                                              stamps[i].data_ptr(), 2 * wgs, ctypes.byref(n)), "tl_gemv_f16_stamped")
    run()
    torch.cuda.synchronize()
    wall, ev = time_region(run, 1, torch)
    assert n.value == wgs
    t = stamps.cpu().numpy().astype(np.float64) * 0.01   # us
    start, end = t[:, :, 0], t[:, :, 1]
    first = start.min(axis=1)
    rel_end = np.sort(end - first[:, None], axis=1)
    rel_start = start - first[:, None]
    q = lambda a, f: float(np.median(a[:, min(wgs - 1, int(f * wgs))]))
    period = np.diff(first)
    window = rel_end[:, -1]
    return {
        "metric": "time line of a 4096<-4096 fp16 GEMV launch (stamped build of the dispatch's kernel)",
        "launches": launches, "workgroups": wgs, "us_per_launch_hip_events": round(ev / launches * 1e6, 2),
        "all_workgroups_started_us": round(float(np.median(rel_start.max(axis=1))), 2),
        "first_workgroup_done_us": round(q(rel_end, 0.0), 2),
        "workgroups_done_us": {"10%": round(q(rel_end, 0.10), 2), "50%": round(q(rel_end, 0.50), 2),
                               "90%": round(q(rel_end, 0.90), 2), "100%": round(float(np.median(window)), 2)},
        "period_first_start_to_next_first_start_us": round(float(np.median(period)), 2),
        "outside_window_us": round(float(np.median(period - window[:-1])), 2),
        "bytes": 2 * N * K + 2 * K + 2 * N,
        "streaming_rate_between_10_and_90_pct_GBs": round(0.8 * 2 * N * K / (q(rel_end, 0.90) - q(rel_end, 0.10)) / 1e3, 1),
    }


def hgemm_timeline(dev, randn, torch, synth, launches: int):
    """Where the time of a launch of the AGPR GEMM kernels goes, for the four M = 2048 prefill shapes and 512x32000x4096:
    every workgroup stamps the GPU's constant 100 MHz counter at its first instruction and after its last store
    (tl_set_hgemm_stamps).  `launches` back-to-back calls of tl_matmul2d_f16 per shape, W rotating over >= 600 MB.
    Per shape, medians over the launches, microseconds after the first workgroup's start: the last workgroup's start,
    mean / shortest / longest workgroup, 10 / 50 / 90 / 100 % of the workgroups done, and the period to the next
    launch's first start (what lies between the window and the period is the launch boundary).  A call that goes out
    as two launches (whole rounds of 256x256 tiles, then the remaining columns) reports the second one's workgroups
    where both wrote a stamp slot and is marked."""
    import numpy as np
    launches = max(6, min(launches, 40))
    cap = 2 * 4096
    out = {}
    for (M, N, K) in [s for s in HGEMM_SHAPES if s[0] == 2048] + [(512, 32000, 4096)]:
        A = randn((M, K), 1.0)
        nb = max(2, -(-600_000_000 // (N * K * 2)))
        Bs = [randn((N, K), 0.02) for _ in range(nb)]
        C = torch.empty((M, N), device="cuda", dtype=torch.float16)
        for i in range(4):
            dev.matmul2d(A, Bs[i % nb], C)
        stamps = torch.zeros((launches, cap), device="cuda", dtype=torch.int64)
        torch.cuda.synchronize()
        try:
            for i in range(launches):
                dev.lib.tl_set_hgemm_stamps(stamps[i].data_ptr(), cap)
                dev.matmul2d(A, Bs[i % nb], C)
        finally:
            dev.lib.tl_set_hgemm_stamps(None, 0)
        torch.cuda.synchronize()
        plan = dev.hgemm_last_plan()
        st = stamps.cpu().numpy().astype(np.float64) * 0.01   # us
        n = int((st[0] != 0).sum() // 2)
        if n == 0:
            out[f"{M}x{N}x{K}"] = {"kernel": plan[0], "note": "no stamped kernel served this shape"}
            continue
        t = st[:, :2 * n].reshape(launches, n, 2)
        first = t[:, :, 0].min(axis=1)
        start, end = t[:, :, 0] - first[:, None], t[:, :, 1] - first[:, None]
        dur = end - start
        ends = np.sort(end, axis=1)
        q = lambda f: round(float(np.median(ends[:, min(n - 1, int(f * n))])), 1)
        window = ends[:, -1]
        flops = synth.gemm_flops(M, N, K)
        period = float(np.median(np.diff(first)))
        out[f"{M}x{N}x{K}"] = {
            "kernel": plan[0], "workgroups_stamped": n, "two_launches": bool(np.median(start.max(axis=1)) > 5.0),
            "last_start_us": round(float(np.median(start.max(axis=1))), 1),
            "workgroup_us": {"mean": round(float(np.median(dur.mean(axis=1))), 1), "min": round(float(np.median(dur.min(axis=1))), 1),
                             "max": round(float(np.median(dur.max(axis=1))), 1)},
            "workgroups_done_us": {"10%": q(0.10), "50%": q(0.50), "90%": q(0.90), "100%": round(float(np.median(window)), 1)},
            "period_us": round(period, 1), "outside_window_us": round(float(np.median(np.diff(first) - window[:-1])), 1),
            "TFLOP/s_at_period": round(flops / period / 1e6, 1),
        }
    return {"metric": "time line of the AGPR fp16 GEMM kernels (workgroup time stamps)", "launches": launches, "shapes": out}


def gemv_grid_experiments(dev, randn, torch, synth):
    """The plain streaming GEMV under capped, persistent grids and with four rows per wavefront pass, W from HBM:
    4096<-4096 and 12288<-4096, every configuration timed over 200 launches on > 1 GB of rotating matrices."""
    names = dev.gemv_variants()
    out = {}
    for (N, K) in ((4096, 4096), (12288, 4096)):
        nbuf = max(2, int(1.0e9 // (N * K * 2)) + 1)
        Ws = [randn((N, K), 0.02) for _ in range(nbuf)]
        x = randn((1, K), 1.0)
        y = torch.empty((1, N), device="cuda", dtype=torch.float16)
        idx = [0]

        def one():
            dev.matmul2d(x, Ws[idx[0] % nbuf], y)
            idx[0] += 1
        rows = {}
        configs = [("dispatch (2 rows per pass, one row block per workgroup)", 0, 0)]
        v2, v4 = names.index("stream_w4r2u2s4x1"), names.index("stream_w4r4u2s4x1")
        for k in (2, 4, 8):
            configs.append((f"2 rows per pass, grid capped at {k} workgroups per CU (persistent)", v2, 4 * k))
        configs.append(("4 rows per pass, one row block per workgroup", v4, 1 << 20))
        for k in (2, 4, 8):
            configs.append((f"4 rows per pass, grid capped at {k} workgroups per CU (persistent)", v4, 4 * k))
        for name, variant, wpc in configs:
            dev.set_gemv_variant(variant)
            dev.lib.tl_set_gemv_grid_waves_per_cu(wpc)
            best = None
            for _ in range(3):
                for _ in range(10):
                    one()
                _, ev = time_region(one, 200, torch)
                us = ev / 200 * 1e6
                best = us if best is None else min(best, us)
            rows[name] = {"us": round(best, 2), "frac_hbm": round(synth.gemv_bytes(N, K) / best / 1e3 / HBM_PEAK_GBS, 4)}
        dev.set_gemv_variant(0)
        dev.lib.tl_set_gemv_grid_waves_per_cu(0)
        out[f"{N}x{K}"] = rows
        del Ws
    return {"metric": "fp16 GEMV grid experiments (us per launch, best of 3 x 200 launches, W from HBM)", "results": out}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (every box of this build has one); got --gpus {args.gpus}",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from tensorlib_amd import HipDevice, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: tensorlib_amd has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    dev = HipDevice(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234)

    def randn(shape, std):
        return (torch.randn(shape, generator=gen, device="cuda", dtype=torch.float32) * std).to(torch.float16)

    if args.workload == "decode":
        from tensorlib_amd import llama2
        cfg = llama2.Llama2Config()
        m = llama2.Llama2Model(dev, cfg, max_tokens=128)
        m.random_init_on_device(seed=7)
        prompt = synth.token_ids(11, 128, cfg.vocab_size)
        m.generate(prompt, max(2, args.warmup), llama2.MODE_FUSED)
        _, tp, td = m.generate(prompt, args.steps + 1, llama2.MODE_FUSED)   # the first token comes out of the prefill
        tok_s = args.steps / td
        wbytes = cfg.weight_bytes_per_token()
        out = {
            "metric": "Llama2-7B decode tok/s (fused driver, batch 1)", "value": round(tok_s, 2), "unit": "tok/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(1e3 / tok_s, 5),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": f"Llama2-7B fp16 random-init, 128-token random prompt, {args.steps} greedy decode steps, "
                                   "batch 1, max_seq 2048", "weight_bytes_per_token": wbytes},
            "roofline": {"bound": "hbm", "achieved": round(wbytes * tok_s / 1e9, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(wbytes * tok_s / 1e9 / HBM_PEAK_GBS, 4), "traffic": None,
                         "kernel": "whole decode step (weight bytes per token x tok/s)"},
            "extra": {"prefill_tok_s": round(128 / tp, 1)},
        }
        m.close()
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline_llama2_decode()
        print(json.dumps(out))
        return

    if args.workload == "gemv_timeline":
        print(json.dumps(gemv_timeline(dev, randn, torch, args.steps)))
        return
    if args.workload == "hgemm_timeline":
        print(json.dumps(hgemm_timeline(dev, randn, torch, synth, args.steps)))
        return
    if args.workload == "gemv_grid":
        print(json.dumps(gemv_grid_experiments(dev, randn, torch, synth)))
        return

    if args.workload == "hgemm":
        rows = [int(r) for r in args.rows.split(",")]
        short_prompt = [(16, 12288, 4096), (16, 4096, 4096), (16, 22016, 4096), (16, 4096, 11008)]
        shapes = [s for s in HGEMM_SHAPES + short_prompt if s[0] in rows]
        if not shapes:
            print(f"--rows {args.rows}: no prefill shape has that many rows", file=sys.stderr)
            sys.exit(2)
        dev.lib.tl_set_hgemm_splitk_merge(args.splitk_merge)
        if args.hgemm_variant:
            dev.set_hgemm_variant(dev.hgemm_variants().index(args.hgemm_variant))
        mats = [(randn((M, K), 1.0), randn((N, K), 0.02), torch.empty((M, N), device="cuda", dtype=torch.float16))
                for (M, N, K) in shapes]
        step_flops = sum(synth.gemm_flops(*s) for s in shapes)

        def step():
            for A, B, C in mats:
                dev.matmul2d(A, B, C)
        for _ in range(args.warmup):
            step()
        wall, ev = time_region(step, args.steps, torch)
        value = step_flops / (wall / args.steps) / 1e12
        achieved = step_flops / (ev / args.steps) / 1e12
        sustained = mfma_sustained(dev)
        out = {
            "metric": f"fp16 HGEMM TFLOP/s (Llama2-7B prefill, M={args.rows} shapes)",
            "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(wall * 1e3 / args.steps, 5), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "prefill HGEMM X[M,K] . W[N,K]^T for (M,N,K) in " + ", ".join("x".join(map(str, s)) for s in shapes) +
                                   "; X~N(0,1), W~N(0,0.02); fp32 accumulate", "flops_per_step": step_flops,
                       "splitk_merge": args.splitk_merge, "variant": args.hgemm_variant or "dispatch"},
            "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(achieved / MFMA_FP16_PEAK_TFLOPS, 4), "traffic": None,
                         "kernel": "by shape: hgemm_f16_big_kernel / hgemm_f16_mid_kernel (a256x..), hgemm_f16_dlds_kernel (p..), "
                                   "hgemm_fewrows_kernel (fewrows); extra.hgemm_prefill names it per shape",
                         "flops_per_launch": step_flops / len(shapes),
                         "avg_launch_us": round(ev / args.steps / len(shapes) * 1e6, 2),
                         "sustained_mfma_tflops": sustained},
        }
        if not args.no_extra:
            out["extra"] = {"hgemm_prefill": hgemm_table(dev, randn, torch, synth, max(sustained["changing_operands"], sustained["changing_operands_16x16x32"]), shapes,
                                                         vendor=args.vendor_reference)}
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline_hgemm()
        print(json.dumps(out))
        return

    # ---- weights: NSETS rotating sets of the four matrices (3 x 476 MB) ------------------
    NSETS = 3
    sets = []
    for _ in range(NSETS):
        sets.append([(randn((N, K), 0.02), randn((1, K), 1.0), torch.empty((1, N), device="cuda", dtype=torch.float16))
                     for (N, K) in SWEEP])
    step_bytes = sum(synth.gemv_bytes(N, K) for N, K in SWEEP)
    counter = [0]

    def step():
        s = sets[counter[0] % NSETS]
        counter[0] += 1
        for W, x, y in s:
            dev.matmul2d(x, W, y)

    if args.copy_calibration:
        src = torch.zeros(1 << 27, device="cuda", dtype=torch.float16)   # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        for _ in range(5):
            dev.contiguous(src, (1 << 27,), (1,), 0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    wall, ev = time_region(step, args.steps, torch)
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (wall / args.steps) / 1e9
    launches = args.steps * len(SWEEP)
    avg_launch_s = ev / launches
    achieved = (step_bytes / len(SWEEP)) / avg_launch_s / 1e9

    out = {
        "metric": "fp16 GEMV GB/s (Llama2-7B decode sweep)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "Llama2-7B decode GEMV sweep, batch 1 fp16: 4096<-4096, 11008<-4096, 4096<-11008, "
                               "32000<-4096; W~N(0,0.02), x~N(0,1); fp32 accumulate; weights rotated over "
                               f"{NSETS} sets ({NSETS * step_bytes / 1e6:.0f} MB)",
                   "bytes_per_step": step_bytes},
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH,
            "traffic_source": GEMV_TRAFFIC_SOURCE,
            "kernel": "gemv_f16_stream_kernel",
            "bytes_per_launch": step_bytes / len(SWEEP),
            "avg_launch_us": round(avg_launch_s * 1e6, 3),
        },
    }
    del sets
    torch.cuda.empty_cache()

    extra = {}
    if not args.no_extra:
        # per-shape GEMV, each over >1 GB of rotating weights
        per_shape, cache_resident = {}, {}
        for (N, K) in SWEEP:
            nbuf = max(2, int(1.0e9 // (N * K * 2)) + 1)
            Ws = [randn((N, K), 0.02) for _ in range(nbuf)]
            x = randn((1, K), 1.0)
            y = torch.empty((1, N), device="cuda", dtype=torch.float16)
            idx = [0]

            def one():
                dev.matmul2d(x, Ws[idx[0] % nbuf], y)
                idx[0] += 1
            for _ in range(10):
                one()
            _, ev1 = time_region(one, 200, torch)
            us = ev1 / 200 * 1e6
            gbs = synth.gemv_bytes(N, K) / us / 1e3
            per_shape[f"{N}x{K}"] = {"us": round(us, 2), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
            # the same launch with ONE matrix used again and again: the three smaller ones then sit in the 256 MB
            # memory-side cache, so this is the cache-resident figure, not an HBM figure
            for _ in range(10):
                dev.matmul2d(x, Ws[0], y)
            _, ev2 = time_region(lambda: dev.matmul2d(x, Ws[0], y), 200, torch)
            us2 = ev2 / 200 * 1e6
            cache_resident[f"{N}x{K}"] = {"us": round(us2, 2), "GB/s": round(synth.gemv_bytes(N, K) / us2 / 1e3, 1)}
            del Ws
        extra["gemv_per_shape"] = per_shape
        extra["gemv_cache_resident"] = cache_resident
        # one decoded token launches 128 / 64 / 32 / 1 of the four shapes (wq wk wv wo / w1 w3 / w2 / classifier):
        # the sweep's equal weights flatter the mix, this figure does not
        mix = {(4096, 4096): 128, (11008, 4096): 64, (4096, 11008): 32, (32000, 4096): 1}
        mix_bytes = sum(n * synth.gemv_bytes(N, K) for (N, K), n in mix.items())
        mix_us = sum(n * per_shape[f"{N}x{K}"]["us"] for (N, K), n in mix.items())
        extra["gemv_decode_mix"] = {"launches_per_token": {f"{N}x{K}": n for (N, K), n in mix.items()},
                                    "bytes_per_token": mix_bytes, "us_per_token": round(mix_us, 1),
                                    "GB/s": round(mix_bytes / mix_us / 1e3, 1),
                                    "frac_hbm": round(mix_bytes / mix_us / 1e3 / HBM_PEAK_GBS, 4)}
        torch.cuda.empty_cache()

        sustained = mfma_sustained(dev)
        extra["mfma_sustained_tflops"] = sustained
        extra["hgemm_prefill"] = hgemm_table(dev, randn, torch, synth, max(sustained["changing_operands"], sustained["changing_operands_16x16x32"]))
        # a prompt of a few tokens (the reference's usual prefill): the projections of a 16-token prompt
        extra["hgemm_short_prompt"] = hgemm_table(dev, randn, torch, synth, max(sustained["changing_operands"], sustained["changing_operands_16x16x32"]),
                                                  [(16, 12288, 4096), (16, 4096, 4096), (16, 22016, 4096), (16, 4096, 11008)])
        torch.cuda.empty_cache()
        from tensorlib_amd import llama2
        extra["llama2_7b_decode"] = llama2.bench_decode(dev)
    out["extra"] = extra

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemv()
        if not args.no_extra:
            # the other two metrics' CPU figures, on the same host in the same run
            extra["hgemm_cpu_baseline"] = cpu_baseline_hgemm()
            extra["llama2_7b_decode"]["cpu"] = cpu_baseline_llama2_decode()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
