"""Benchmark of the per-batch planning path on one MI355X.

One step = one plan of the DeepSeek-V3-shaped EP8 cube configuration: histogram of
this GPU's [8192 x 8] routing indices, LP solve on the global per-expert counts,
logical->physical redirect.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is the p50 GPU time per plan in microseconds, from
HIP events recorded between plans on the stream the kernels run on.  The line also
carries
  roofline      redirect kernel at the sweep shape [262144 x 8] against the HBM peak;
                algorithmic traffic is 16 bytes per index (int64 in, int64 out);
  cpu_baseline  the scalar C restatement of the reference algorithm (oracle/), timed
                on this host on a bounded sample of the same plans;
  extras        p99, solve-only latency, batched plans/s, redirect tokens/s, ...
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
REDIRECT_BYTES_PER_INDEX = 16
HISTOGRAM_BYTES_PER_INDEX = 8
# HBM bytes one redirect launch moves at the sweep shape come from rocprofv3 counters (FETCH_SIZE and
# WRITE_SIZE, two runs, each scaled by what the same counter reads for the plain copy kernel of known
# size).  They cannot be measured from inside this script, so the figure is read from the tracked
# summary of that measurement, which also names the commit whose kernel it was taken from.
TRAFFIC_SUMMARY = ROOT / "profiles" / "redirect_sweep_262144x8_hbm_traffic.md"


def measured_redirect_traffic():
    """(bytes per launch, commit the kernel was measured at) from the profile summary, or (None, None)."""
    import re
    try:
        text = TRAFFIC_SUMMARY.read_text()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes_per_launch:\s*(\d+)", text)
    c = re.search(r"measured_at_commit:\s*([0-9a-f]+)", text)
    return (int(m.group(1)) if m else None), (c.group(1) if c else None)


def pct(a, q):
    return float(np.percentile(np.asarray(a, dtype=np.float64), q))


def event_times_us(fn, n, warmup, torch):
    """Runs fn() n times back to back; returns GPU microseconds between consecutive events."""
    for _ in range(warmup):
        fn()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
    for e in ev:
        e.record()
    torch.cuda.synchronize()
    ev[0].record()
    for i in range(n):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    return np.array([ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(n)])


class KernelTimer:
    """Times single kernels of the library by their own begin/end timestamps: the library
    records them into a pair of HIP events armed with lplb_time_next_launch()."""

    def __init__(self, lib, n):
        import ctypes
        self.ct = ctypes
        self.lib = lib
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.pairs = []
        for _ in range(n):
            a, b = ctypes.c_void_p(), ctypes.c_void_p()
            assert self.hip.hipEventCreate(ctypes.byref(a)) == 0 and self.hip.hipEventCreate(ctypes.byref(b)) == 0
            self.pairs.append((a, b))
        self.used = 0

    def arm(self):
        a, b = self.pairs[self.used]
        self.used += 1
        self.lib.lplb_time_next_launch(a, b)

    def take(self, n):
        """The next n pairs as two arrays of events, for the library's *_series calls."""
        pairs = self.pairs[self.used:self.used + n]
        assert len(pairs) == n
        self.used += n
        arr = self.ct.c_void_p * n
        return arr(*[a.value for a, _ in pairs]), arr(*[b.value for _, b in pairs])

    def times_us(self, torch):
        torch.cuda.synchronize()
        out = []
        for a, b in self.pairs[:self.used]:
            ms = self.ct.c_float()
            rc = self.hip.hipEventElapsedTime(self.ct.byref(ms), a, b)
            assert rc == 0, f"hipEventElapsedTime -> {rc}"
            out.append(ms.value * 1e3)
        self.used = 0
        return np.array(out)

    def close(self):
        for a, b in self.pairs:
            self.hip.hipEventDestroy(a)
            self.hip.hipEventDestroy(b)


def copy_sweep(lib, torch, dev) -> None:
    """The library's copy kernel (what the redirect is compared with) at a range of sizes.  Every launch is
    timed by its own begin/end timestamps; buffers rotate so that at least 512 MB of distinct lines pass
    between two uses of the same one (fewer pairs, still more than the 256 MB last-level cache, at 128 MiB)."""
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for n_bytes in (16, 1 << 18, 1 << 20, 1 << 21, 1 << 22, 1 << 23, 3 << 22, 1 << 24, 1 << 25, 1 << 26, 1 << 27):
        n_el = n_bytes // 8
        n_pairs = int(min(18, max(3, -(-(512 << 20) // (2 * n_bytes)))))
        src = [torch.randint(0, 256, (n_el,), dtype=torch.int64, device=dev) for _ in range(n_pairs)]
        dst = [torch.empty_like(t) for t in src]
        reps = 10
        n = n_pairs * reps
        arr = lambda ts: (ctypes.c_void_p * n)(*[ts[i % n_pairs].data_ptr() for i in range(n)])
        a_src, a_dst = arr(src), arr(dst)
        assert lib.lplb_copy_calibration_series(a_src, a_dst, n_el, n, None, None, stream) == 0   # warm-up pass
        torch.cuda.synchronize()
        timer = KernelTimer(lib, n)
        starts, stops = timer.take(n)
        assert lib.lplb_copy_calibration_series(a_src, a_dst, n_el, n, starts, stops, stream) == 0, lib.lplb_last_error()
        us = timer.times_us(torch)
        timer.close()
        assert torch.equal(dst[0], src[0])
        rows.append({"bytes_each_way": n_bytes, "buffer_pairs": n_pairs, "launches": n,
                     "avg_us": round(float(us.mean()), 2), "p50_us": round(pct(us, 50), 2),
                     "min_us": round(float(us.min()), 2),
                     "GBs_avg": round(2 * n_bytes / (float(us.mean()) * 1e-6) / 1e9, 1),
                     "frac_of_peak_avg": round(2 * n_bytes / (float(us.mean()) * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
        del src, dst
    # other shapes of the same copy at the sweep's size (16 MiB each way): what the library's choice rests on
    n_el, n_pairs, reps = (1 << 24) // 8, 16, 10
    src = [torch.randint(0, 256, (n_el,), dtype=torch.int64, device=dev) for _ in range(n_pairs)]
    dst = [torch.empty_like(t) for t in src]
    n = n_pairs * reps
    arr = lambda ts: (ctypes.c_void_p * n)(*[ts[i % n_pairs].data_ptr() for i in range(n)])
    a_src, a_dst = arr(src), arr(dst)
    shapes = []
    for loads in (1, 2, 4, 8):
        for threads in (256, 512, 1024):
            for barrier, streaming in ((1, 1), (0, 1), (1, 0)):
                if (barrier, streaming) != (1, 1) and threads != 1024:
                    continue
                args = (a_src, a_dst, n_el, n, loads, threads, barrier, streaming)
                assert lib.lplb_copy_shape_series(*args, None, None, stream) == 0, lib.lplb_last_error()
                timer = KernelTimer(lib, n)
                starts, stops = timer.take(n)
                assert lib.lplb_copy_shape_series(*args, starts, stops, stream) == 0
                us = timer.times_us(torch)
                timer.close()
                shapes.append({"loads_per_lane": loads, "threads": threads, "barrier": bool(barrier),
                               "streaming": bool(streaming), "workgroups": n_el // (2 * threads * loads),
                               "avg_us": round(float(us.mean()), 2), "p50_us": round(pct(us, 50), 2),
                               "min_us": round(float(us.min()), 2)})
    assert torch.equal(dst[0], src[0])
    del src, dst
    # time = fixed + bytes / rate, fitted over the sizes from 1 MiB up
    big = [r for r in rows if r["bytes_each_way"] >= 1 << 20]
    x = np.array([2.0 * r["bytes_each_way"] for r in big])
    y = np.array([r["avg_us"] for r in big])
    slope, fixed = np.polyfit(x, y, 1)
    print(json.dumps({"copy_sweep": rows, "shapes_at_16MiB": shapes, "fit_from_1MiB": {"fixed_us": round(float(fixed), 2),
                                                           "GBs": round(1e-3 / float(slope), 1)}}))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of the CPU baseline sample")
    ap.add_argument("--skip-extras", action="store_true")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the redirect and copy kernels at the sweep shape (for counter collection)")
    ap.add_argument("--roofline-reps", type=int, default=20, help="passes over the rotating buffers")
    ap.add_argument("--solver-only", action="store_true",
                    help="only 50 single and 10 batched (2048) LP solves at the plan's shape (for counter collection)")
    ap.add_argument("--copy-sweep", action="store_true",
                    help="only the copy kernel, from 16 bytes to 128 MiB per direction: the fixed cost of a launch "
                         "and what a streaming kernel of the sweep's size can reach on this box")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the plan; a run with --gpus > 1 is not supported "
                 "(every rank plans its own tokens; the only exchange between ranks is the sum of the count "
                 "vectors, which is not part of this measurement).")

    import torch

    from lplb_amd import synth
    from lplb_amd._native import CompiledSolver, load
    from oracle import oracle

    load()  # no fallback: raises if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    n_sms = props.multi_processor_count

    def to_dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    if args.copy_sweep:
        copy_sweep(load(), torch, dev)
        return

    # ------------------------------------------------------------------ inputs
    inp = synth.make_inputs("v3_ep8_cube")
    cfg = inp.cfg
    G, D = cfg.r2o.shape
    L, P = cfg.n_logical // cfg.ep_size, cfg.n_physical // cfg.ep_size
    C = (P - L) // D
    n_fixed = L - C * D
    o2r_host = np.argsort(cfg.r2o, axis=0, kind="stable").astype(np.int32)
    solver = CompiledSolver(1, G, D, P, C)
    r2o, o2r, phy2log = to_dev(cfg.r2o), to_dev(o2r_host), to_dev(inp.phy2log)
    idx = to_dev(inp.indices)
    counts = to_dev(inp.global_counts)
    avail = torch.zeros(1, dtype=torch.int32, device=dev)
    ws: dict = {}

    # Outputs are allocated once; the timed loop calls the C entry point directly with cached
    # pointers (the Python wrapper's argument checks cost more host time than the GPU needs).
    out0, o_w0, by0 = solver.plan(idx, r2o, o2r, phy2log, avail, n_sms, global_counts=counts)
    ws = {"out": out0, "o_weight": o_w0, "by_sm": by0,
          "global_workload": torch.empty(cfg.n_logical, dtype=torch.float32, device=dev)}
    lib = solver.lib
    stream = torch.cuda.current_stream().cuda_stream
    plan_args = (idx.data_ptr(), idx.numel(), counts.data_ptr(), r2o.data_ptr(), o2r.data_ptr(), phy2log.data_ptr(),
                 1, G, D, C, P, n_sms, by0.data_ptr(), ws["global_workload"].data_ptr(), o_w0.data_ptr(),
                 avail.data_ptr(), out0.data_ptr(), None, 0, 5)

    def plan(stream_handle=stream):
        rc = lib.lplb_plan(*plan_args, stream_handle)
        assert rc == 0, lib.lplb_last_error()

    plan()
    torch.cuda.synchronize()
    if args.roofline_only:
        args.steps, args.warmup, args.skip_extras, args.cpu_seconds = 1, 0, True, 0.0
    if args.solver_only:
        lib_ = solver.lib
        wl_ = counts.view(1, G, L)
        gw_ = torch.empty(1, G, L, dtype=torch.float32, device=dev)
        res_ = torch.empty(2048, 1, G, D, dtype=torch.float32, device=dev)
        sweep_ = to_dev(synth.sweep_counts(2048).reshape(2048, 1, G, L))
        st_ = torch.cuda.current_stream().cuda_stream
        for _ in range(50):
            assert lib_.lplb_solve(wl_.data_ptr(), gw_.data_ptr(), r2o.data_ptr(), phy2log.data_ptr(), 1, G, D, C,
                                   n_fixed, avail.data_ptr(), res_.data_ptr(), 0, 5, st_) == 0
        for _ in range(10):
            assert lib_.lplb_solve_batched(sweep_.data_ptr(), None, r2o.data_ptr(), phy2log.data_ptr(), 2048, 1, G, D,
                                           C, n_fixed, avail.data_ptr(), res_.data_ptr(), 0, 5, st_) == 0
        torch.cuda.synchronize()
        print(json.dumps({"solver_only": True, "feasible": int(avail[0])}))
        return

    # ----------------------------------------------------------- timed region
    for _ in range(args.warmup):
        plan()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    for e in ev:          # torch creates the HIP event at the first record: keep that out of the timed region
        e.record()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(args.steps):
        plan()
        ev[i + 1].record()
    t_enqueued = time.perf_counter()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per_plan_us = np.array([ev[i].elapsed_time(ev[i + 1]) * 1e3 for i in range(args.steps)])
    p50, p99 = pct(per_plan_us, 50), pct(per_plan_us, 99)
    assert int(avail[0]) == args.warmup + args.steps + 2, "an LP failed its feasibility test"

    extras: dict = {"p99_us_per_plan": round(p99, 2), "mean_us_per_plan": round(float(per_plan_us.mean()), 2),
                    "host_enqueue_us_per_plan": round((t_enqueued - t0) / args.steps * 1e6, 2),
                    "compute_units": n_sms, "device": props.name}

    # ------------------------------------------- roofline: redirect @ sweep shape
    sweep = synth.make_inputs("sweep_redirect")
    n_idx = sweep.indices.size
    n_buf = 18                                   # 18 x (16 + 16) MiB > 512 MB of distinct lines
    rng = np.random.default_rng(7)
    flat = sweep.indices.reshape(-1)
    bufs_in = [to_dev(np.roll(flat, int(rng.integers(0, n_idx)))) for _ in range(n_buf)]
    bufs_out = [torch.empty_like(b) for b in bufs_in]
    sweep_p2l = to_dev(sweep.phy2log)
    # Two slices per CU: at this size two 8-wave workgroups per CU beat one of 16 waves (one's ranking
    # overlaps the other's loads and stores); the figure with one slice per CU is in the extras.
    roof_blocks = 2 * n_sms
    tables = []
    for b in bufs_in:
        total, by = solver.count_idx(b, roof_blocks)
        tables.append(by)
    o_w, _ = solver.solve(tables[0][-1].view(1, G, L), r2o, sweep_p2l, avail)
    prepared = solver.prepare_mapping(o2r, sweep_p2l)        # once per mapping, as Planner does

    def redirect(i, n_blocks=roof_blocks, table=None):
        rc = lib.lplb_map_idx_prepared(bufs_in[i].data_ptr(), o_w.data_ptr(),
                                       (table if table is not None else tables[i]).data_ptr(), prepared.data_ptr(), n_idx,
                                       1, G, D, C, P, n_blocks, bufs_out[i].data_ptr(), None, stream)
        assert rc == 0, lib.lplb_last_error()

    reps = args.roofline_reps
    for i in range(n_buf):
        redirect(i)
        assert lib.lplb_copy_calibration(bufs_in[i].data_ptr(), bufs_out[i].data_ptr(), n_idx, stream) == 0
    torch.cuda.synchronize()
    # Each launch is timed by its kernel's own begin/end timestamps (what a kernel trace reports).  The launches
    # come from a loop inside the library: issued one by one from Python, one launch in ten reads about 4 us
    # longer, redirect and copy alike, which the same launches issued from compiled code do not show.  The same
    # bytes through a plain copy kernel are the practical ceiling on this box; the two kernels take turns, block
    # of n_buf launches by block, so that whatever drifts during the run treats them alike.
    n_series = n_buf
    timer = KernelTimer(lib, 3 * reps * n_series)
    ptrs = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    series_in, series_by, series_out = ptrs(bufs_in), ptrs(tables), ptrs(bufs_out)
    half = n_buf // 2
    copy_in, copy_out = ptrs(bufs_in[half:] + bufs_in[:half]), ptrs(bufs_out[half:] + bufs_out[:half])
    # (a third series: the copy in the redirect's own launch shape, two workgroups of 16 waves per CU and two
    # 16-byte loads per lane, which is 1 us slower than the copy's best shape)
    red_slots, copy_slots, twin_slots = [], [], []
    for _ in range(reps):
        for which, slots in (("redirect", red_slots), ("copy", copy_slots), ("twin", twin_slots)):
            starts, stops = timer.take(n_series)
            if which == "redirect":
                rc = lib.lplb_map_idx_prepared_series(series_in, o_w.data_ptr(), series_by, prepared.data_ptr(), n_idx, 1, G,
                                                      D, C, P, roof_blocks, series_out, n_series, starts, stops, stream)
            elif which == "copy":
                rc = lib.lplb_copy_calibration_series(copy_in, copy_out, n_idx, n_series, starts, stops, stream)
            else:
                rc = lib.lplb_copy_shape_series(copy_in, copy_out, n_idx, n_series, 2, 1024, 1, 1, starts, stops, stream)
            assert rc == 0, lib.lplb_last_error()
            slots.append(timer.used)
    both_us = timer.times_us(torch)
    red_us = np.concatenate([both_us[e - n_series:e] for e in red_slots])
    copy_us = np.concatenate([both_us[e - n_series:e] for e in copy_slots])
    twin_us = np.concatenate([both_us[e - n_series:e] for e in twin_slots])
    red_avg = float(red_us.mean())
    alg_bytes = n_idx * REDIRECT_BYTES_PER_INDEX
    achieved = alg_bytes / (red_avg * 1e-6) / 1e9
    copy_gbs = alg_bytes / (float(copy_us.mean()) * 1e-6) / 1e9
    # the same launches back to back with one event pair around each block: sustained rate, gaps between
    # kernels included
    burst = []
    for _ in range(max(4, reps // 2)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        assert lib.lplb_map_idx_prepared_series(series_in, o_w.data_ptr(), series_by, prepared.data_ptr(), n_idx, 1, G, D, C,
                                                P, roof_blocks, series_out, n_series, None, None, stream) == 0
        e1.record()
        torch.cuda.synchronize()
        burst.append(e0.elapsed_time(e1) * 1e3 / n_series)
    traffic, traffic_commit = measured_redirect_traffic()
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_measured_at_commit": traffic_commit,
                "kernel": "redirect_pairs",
                "workload": f"sweep_redirect [{sweep.indices.shape[0]} x {sweep.indices.shape[1]}] int64, {roof_blocks} slices, "
                            "mapping tables prepared once (lplb_map_idx_prepared)",
                "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_us": round(red_avg, 2),
                "p50_launch_us": round(pct(red_us, 50), 2), "p99_launch_us": round(pct(red_us, 99), 2),
                "launches_timed": int(red_us.size), "distinct_buffer_pairs": n_buf,
                # launches that read 2 us or more above the median: what separates avg from p50 (the copy has them too)
                "launches_2us_above_p50_frac": round(float(np.mean(red_us > pct(red_us, 50) + 2.0)), 4),
                "copy_launches_2us_above_p50_frac": round(float(np.mean(copy_us > pct(copy_us, 50) + 2.0)), 4),
                "back_to_back_us_per_launch": round(float(np.median(burst)), 2),
                "copy_kernel_GBs_same_bytes": round(copy_gbs, 1),
                "copy_kernel_avg_launch_us": round(float(copy_us.mean()), 2),
                "frac_of_copy_kernel": round(achieved / copy_gbs, 4),
                "copy_in_the_redirects_launch_shape_avg_us": round(float(twin_us.mean()), 2),
                "frac_of_copy_in_the_redirects_launch_shape": round(float(twin_us.mean()) / red_avg, 4)}
    extras["redirect_tokens_per_s"] = round(n_idx / (red_avg * 1e-6), 1)

    if not args.skip_extras:
        # the same redirect with one slice per CU (the reference's default n_sms = SM count)
        cu_tables = [solver.count_idx(b, n_sms)[1] for b in bufs_in]
        for i in range(n_buf):
            redirect(i, n_sms, cu_tables[i])
        cu_timer = KernelTimer(lib, 4 * n_buf)
        torch.cuda.synchronize()
        for _ in range(4):
            for i in range(n_buf):
                cu_timer.arm()
                redirect(i, n_sms, cu_tables[i])
        extras["redirect_sweep_us_one_slice_per_cu"] = round(float(cu_timer.times_us(torch).mean()), 2)
        cu_timer.close()
        # the reference's own call (o2r and phy2log instead of a prepared table: every workgroup builds the tables)
        up_timer = KernelTimer(lib, 4 * n_buf)
        for r in range(4 * n_buf):
            i = r % n_buf
            up_timer.arm()
            assert lib.lplb_map_idx(bufs_in[i].data_ptr(), o_w.data_ptr(), tables[i].data_ptr(), o2r.data_ptr(),
                                    sweep_p2l.data_ptr(), n_idx, 1, G, D, C, P, roof_blocks, bufs_out[i].data_ptr(), None,
                                    stream) == 0
        extras["redirect_sweep_us_without_prepared_table"] = round(float(up_timer.times_us(torch).mean()), 2)
        up_timer.close()

        # histogram at the sweep shape (8 B per index)
        def hist(i):
            rc = lib.lplb_count_idx(bufs_in[i].data_ptr(), n_idx, cfg.n_logical, n_sms, cu_tables[i].data_ptr(), stream)
            assert rc == 0
        k = [0]

        def hist_next():
            hist(k[0] % n_buf)
            k[0] += 1
        h_us = event_times_us(hist_next, 10 * n_buf, n_buf, torch)
        extras["histogram_sweep_us"] = round(float(h_us.mean()), 2)
        extras["histogram_sweep_GBs"] = round(n_idx * HISTOGRAM_BYTES_PER_INDEX / (float(h_us.mean()) * 1e-6) / 1e9, 1)
        extras["histogram_sweep_frac_of_peak"] = round(extras["histogram_sweep_GBs"] / HBM_PEAK_GBS, 4)
        # the histogram kernel alone (without the scan over slices that follows it), by its own timestamps
        h_timer = KernelTimer(lib, 4 * n_buf)
        for r in range(4 * n_buf):
            h_timer.arm()          # the first kernel of the call is the histogram
            hist(r % n_buf)
        hk_us = float(h_timer.times_us(torch).mean())
        h_timer.close()
        extras["histogram_kernel_sweep_us"] = round(hk_us, 2)
        extras["histogram_kernel_sweep_frac_of_peak"] = round(n_idx * HISTOGRAM_BYTES_PER_INDEX / (hk_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
        # the same kernel in a series of its own (every launch timed, no scan behind it): a timed kernel that is
        # followed at once by another kernel on the stream reads 1.3-1.6 us longer by its own events
        n_h = 10 * n_buf
        h_series = KernelTimer(lib, n_h)
        h_in = (ctypes.c_void_p * n_h)(*[bufs_in[r % n_buf].data_ptr() for r in range(n_h)])
        h_out = (ctypes.c_void_p * n_h)(*[cu_tables[r % n_buf].data_ptr() for r in range(n_h)])
        assert lib.lplb_slice_histogram_series(h_in, n_idx, cfg.n_logical, n_sms, h_out, n_h, None, None, stream) == 0
        starts, stops = h_series.take(n_h)
        assert lib.lplb_slice_histogram_series(h_in, n_idx, cfg.n_logical, n_sms, h_out, n_h, starts, stops, stream) == 0
        hs_us = float(h_series.times_us(torch).mean())
        h_series.close()
        extras["histogram_kernel_sweep_us_in_a_series_of_its_own"] = round(hs_us, 2)
        extras["histogram_kernel_sweep_frac_of_peak_in_a_series_of_its_own"] = round(
            n_idx * HISTOGRAM_BYTES_PER_INDEX / (hs_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)

        # the whole plan at the sweep shape: histogram of [262144 x 8], LP, redirect (16 B per index)
        sweep_counts_dev = to_dev(sweep.global_counts)
        sw_gw = torch.empty(cfg.n_logical, dtype=torch.float32, device=dev)
        sw_ow = torch.empty(1, G, D, dtype=torch.float32, device=dev)

        def plan_sweep(i, counts_ptr):
            rc = lib.lplb_plan(bufs_in[i].data_ptr(), n_idx, counts_ptr, r2o.data_ptr(), o2r.data_ptr(),
                               sweep_p2l.data_ptr(), 1, G, D, C, P, roof_blocks, tables[i].data_ptr(), sw_gw.data_ptr(),
                               sw_ow.data_ptr(), avail.data_ptr(), bufs_out[i].data_ptr(), None, 0, 5, stream)
            assert rc == 0, lib.lplb_last_error()
        for tag, ptr in (("", sweep_counts_dev.data_ptr()), ("_own_histogram", None)):
            turn_s = [0]

            def plan_sweep_next():
                plan_sweep(turn_s[0] % n_buf, ptr)
                turn_s[0] += 1
            ps_us = event_times_us(plan_sweep_next, 10 * n_buf, n_buf, torch)
            extras[f"plan_sweep_shape{tag}_us_p50"] = round(pct(ps_us, 50), 2)
            extras[f"plan_sweep_shape{tag}_us_p99"] = round(pct(ps_us, 99), 2)
        extras["plan_sweep_shape_frac_of_peak"] = round(
            n_idx * REDIRECT_BYTES_PER_INDEX / (extras["plan_sweep_shape_us_p50"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)

        # redirect on a batch 16x the sweep (512 MiB in, 512 MiB out): the fixed cost per launch fades
        big_n, big_slices = 16 * n_idx, 4 * n_sms
        big_in = [torch.cat([bufs_in[(j + s) % n_buf] for j in range(16)]) for s in (0, 7)]
        big_out = [torch.empty_like(b) for b in big_in]
        big_tables = [solver.count_idx(b, big_slices)[1] for b in big_in]

        def redirect_big(i):
            rc = lib.lplb_map_idx(big_in[i].data_ptr(), o_w.data_ptr(), big_tables[i].data_ptr(), o2r.data_ptr(),
                                  sweep_p2l.data_ptr(), big_n, 1, G, D, C, P, big_slices, big_out[i].data_ptr(), None, stream)
            assert rc == 0
        for i in (0, 1):
            redirect_big(i)
        big_timer = KernelTimer(lib, 12)
        torch.cuda.synchronize()
        for r in range(12):
            big_timer.arm()
            redirect_big(r % 2)
        big_us = float(big_timer.times_us(torch).mean())
        big_timer.close()
        extras["redirect_16x_sweep_us"] = round(big_us, 2)
        extras["redirect_16x_sweep_GBs"] = round(big_n * REDIRECT_BYTES_PER_INDEX / (big_us * 1e-6) / 1e9, 1)
        extras["redirect_16x_sweep_frac_of_peak"] = round(big_n * REDIRECT_BYTES_PER_INDEX / (big_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)
        del big_in, big_out, big_tables

        # kernels of the plan in isolation, at the plan's own shape
        wl = counts.view(1, G, L)
        gw = torch.empty(1, G, L, dtype=torch.float32, device=dev)
        res = torch.empty(1, G, D, dtype=torch.float32, device=dev)

        def solve_only():
            lib.lplb_solve(wl.data_ptr(), gw.data_ptr(), r2o.data_ptr(), phy2log.data_ptr(), 1, G, D, C, n_fixed,
                           avail.data_ptr(), res.data_ptr(), 0, 5, stream)
        s_us = event_times_us(solve_only, 1000, 100, torch)
        extras["solve_p50_us"] = round(pct(s_us, 50), 2)
        extras["solve_p99_us"] = round(pct(s_us, 99), 2)

        by_plan = ws["by_sm"]

        def count_only():
            lib.lplb_count_idx(idx.data_ptr(), idx.numel(), cfg.n_logical, n_sms, by_plan.data_ptr(), stream)

        def map_only():
            lib.lplb_map_idx(idx.data_ptr(), ws["o_weight"].data_ptr(), by_plan.data_ptr(), o2r.data_ptr(),
                             phy2log.data_ptr(), idx.numel(), 1, G, D, C, P, n_sms, ws["out"].data_ptr(), None, stream)
        extras["count_p50_us"] = round(pct(event_times_us(count_only, 1000, 100, torch), 50), 2)
        extras["redirect_p50_us"] = round(pct(event_times_us(map_only, 1000, 100, torch), 50), 2)

        # the plan kernel's own duration, the plan fed by this GPU's own histogram (what Planner.run
        # does without a process group), and the plan as the chain of the three entry points' kernels
        # the same plans without an event between them: wall clock of a run of 2000, one sync at the end
        torch.cuda.synchronize()
        t_run = time.perf_counter()
        for _ in range(2000):
            plan()
        torch.cuda.synchronize()
        extras["plan_back_to_back_wall_us"] = round((time.perf_counter() - t_run) / 2000 * 1e6, 2)
        plan_timer = KernelTimer(lib, 300)
        for _ in range(300):
            plan_timer.arm()
            plan()
        extras["plan_kernel_us_p50"] = round(pct(plan_timer.times_us(torch), 50), 2)
        plan_timer.close()
        local_args = plan_args[:2] + (None,) + plan_args[3:]

        def plan_local():
            assert lib.lplb_plan(*local_args, stream) == 0
        extras["plan_local_counts_us_p50"] = round(pct(event_times_us(plan_local, 1000, 100, torch), 50), 2)
        # the same plan on inputs that are not in any cache: 320 distinct index / output pairs
        # (1 MiB each, together more than the 256 MB the last-level cache holds), used in turn
        n_cold = 320
        cold_idx = torch.stack([torch.roll(idx.reshape(-1), 131 * i) for i in range(n_cold)])
        cold_out = torch.empty_like(cold_idx)
        cold_args = [(cold_idx[i].data_ptr(),) + plan_args[1:16] + (cold_out[i].data_ptr(),) + plan_args[17:]
                     for i in range(n_cold)]
        turn = [0]

        def plan_cold():
            turn[0] = (turn[0] + 1) % n_cold
            assert lib.lplb_plan(*cold_args[turn[0]], stream) == 0
        extras["plan_inputs_from_hbm_us_p50"] = round(pct(event_times_us(plan_cold, 1280, 320, torch), 50), 2)
        del cold_idx, cold_out
        assert lib.lplb_plan_set_cooperative(0) == 0
        extras["plan_as_chain_us_p50"] = round(pct(event_times_us(plan, 1000, 100, torch), 50), 2)
        extras["plan_local_counts_as_chain_us_p50"] = round(pct(event_times_us(plan_local, 1000, 100, torch), 50), 2)
        assert lib.lplb_plan_set_cooperative(1) == 0
        timeouts = ctypes.c_int(-1)
        assert lib.lplb_plan_sync_timeouts(ctypes.byref(timeouts)) == 0 and timeouts.value == 0, timeouts.value
        extras["plan_waits_that_ran_out"] = timeouts.value

        # the same plan replayed from a HIP graph (8 plans per graph): GPU-side cost without launch overhead
        per_graph = 8
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            plan(side.cuda_stream)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cap = torch.cuda.current_stream().cuda_stream
            for _ in range(per_graph):
                plan(cap)
        g_us = event_times_us(graph.replay, 300, 30, torch) / per_graph
        extras["graph_replay_us_per_plan_p50"] = round(pct(g_us, 50), 2)
        extras["graph_replay_us_per_plan_p99"] = round(pct(g_us, 99), 2)

        # 2048 independent LP instances in one launch
        sweep_wl = to_dev(synth.sweep_counts(2048).reshape(2048, 1, G, L))
        results = torch.empty(2048, 1, G, D, dtype=torch.float32, device=dev)

        def batched():
            lib.lplb_solve_batched(sweep_wl.data_ptr(), None, r2o.data_ptr(), phy2log.data_ptr(), 2048, 1, G, D, C,
                                   n_fixed, avail.data_ptr(), results.data_ptr(), 0, 5, stream)
        b_us = event_times_us(batched, 100, 10, torch)
        extras["batched_2048_solves_us"] = round(pct(b_us, 50), 2)
        extras["batched_plans_per_s"] = round(2048 / (pct(b_us, 50) * 1e-6), 1)
        # the timed launches' results, all 2048 of them, against the CPU checker (outside any timed region)
        avail.zero_()
        batched()
        torch.cuda.synchronize()
        b_flow, b_obj, b_ok = oracle.compare_batch(synth.sweep_counts(2048), results.cpu().numpy(), cfg.r2o, inp.phy2log,
                                                   1, C, n_fixed)
        assert b_flow <= 1e-4 and b_obj <= 1e-3 and int(avail[0]) == b_ok == 2048, (b_flow, b_obj, b_ok, int(avail[0]))
        extras["batched_2048_worst_flow_diff_vs_checker"] = float(f"{b_flow:.2e}")
        extras["batched_2048_worst_objective_diff_vs_checker"] = float(f"{b_obj:.2e}")

        # every other configuration of the benchmark suite: p50 / p99 per plan (global counts supplied, as
        # one launch and as the chain of kernels) and the LP kernel's own duration
        per_cfg = {}
        for name in ("cpu_ref_ep8", "v3_ep8_cube", "ep16_hypercube", "ep32_torus"):
            ci = synth.make_inputs(name)
            cc = ci.cfg
            g2, d2 = cc.r2o.shape
            l2, p2 = cc.n_logical // cc.ep_size, cc.n_physical // cc.ep_size
            c2 = (p2 - l2) // d2
            ng = cc.ep_size // g2
            t_r2o, t_o2r = to_dev(cc.r2o), to_dev(np.argsort(cc.r2o, axis=0, kind="stable").astype(np.int32))
            t_p2l, t_idx, t_cnt = to_dev(ci.phy2log), to_dev(ci.indices), to_dev(ci.global_counts)
            t_by = torch.empty(n_sms, cc.n_logical, dtype=torch.int32, device=dev)
            t_gw = torch.empty(cc.n_logical, dtype=torch.float32, device=dev)
            t_ow = torch.empty(ng, g2, d2, dtype=torch.float32, device=dev)
            t_out = torch.empty_like(t_idx)
            t_args = (t_idx.data_ptr(), t_idx.numel(), t_cnt.data_ptr(), t_r2o.data_ptr(), t_o2r.data_ptr(),
                      t_p2l.data_ptr(), ng, g2, d2, c2, p2, n_sms, t_by.data_ptr(), t_gw.data_ptr(), t_ow.data_ptr(),
                      avail.data_ptr(), t_out.data_ptr(), None, 0, 5, stream)

            def plan_cfg():
                assert lib.lplb_plan(*t_args) == 0
            row = {"indices": list(ci.indices.shape), "group_size": g2}
            us = event_times_us(plan_cfg, 500, 50, torch)
            row["one_launch_us_p50"], row["one_launch_us_p99"] = round(pct(us, 50), 2), round(pct(us, 99), 2)
            assert lib.lplb_plan_set_cooperative(0) == 0
            us = event_times_us(plan_cfg, 500, 50, torch)
            row["chain_us_p50"], row["chain_us_p99"] = round(pct(us, 50), 2), round(pct(us, 99), 2)
            assert lib.lplb_plan_set_cooperative(1) == 0
            lp_timer = KernelTimer(lib, 100)
            for _ in range(100):
                lp_timer.arm()
                assert lib.lplb_solve(t_cnt.data_ptr(), t_gw.data_ptr(), t_r2o.data_ptr(), t_p2l.data_ptr(), ng, g2, d2,
                                      c2, l2 - c2 * d2, avail.data_ptr(), t_ow.data_ptr(), 0, 5, stream) == 0
            row["lp_kernel_us_p50"] = round(pct(lp_timer.times_us(torch), 50), 2)
            lp_timer.close()
            per_cfg[name] = row
        extras["per_config"] = per_cfg

        # Planner.run through the Python API, wall clock with a device sync (host overhead included)
        from lplb_amd import Planner
        planner = Planner(torch.from_numpy(cfg.r2o), cfg.n_physical, cfg.n_logical, cfg.ep_size, device=dev)
        planner.phy2log = phy2log

        def wall_us_per_call(fn):
            """Median over five runs of 500 calls, each ended by a device sync (the first run after a pause
            reads up to twice the others)."""
            runs = []
            for _ in range(6):
                torch.cuda.synchronize()
                t = time.perf_counter()
                for _ in range(500):
                    fn()
                torch.cuda.synchronize()
                runs.append((time.perf_counter() - t) / 500 * 1e6)
            return round(float(np.median(runs[1:])), 2)
        extras["planner_run_wall_us"] = wall_us_per_call(lambda: planner.run(idx, avail, n_sms))
        extras["planner_run_us_p50"] = round(pct(event_times_us(lambda: planner.run(idx, avail, n_sms), 1000, 100, torch), 50), 2)

        # The same call on a Planner that was given a process group: this GPU's counts in one launch
        # (lplb_count_totals_add), all-reduce over the EP ranks, then LP and redirect as one plan on the summed
        # counts.  One GPU: the all-reduce itself is left out (the stand-in group below is never handed to
        # torch.distributed), everything around it runs as in a deployment.  The call is two library calls and
        # the host needs longer for them than the GPU: the wall figure is the sustained one, the event figure
        # adds what recording an event between calls costs.
        class OneRankGroup:
            def size(self):
                return cfg.ep_size
        grouped = Planner(torch.from_numpy(cfg.r2o), cfg.n_physical, cfg.n_logical, cfg.ep_size,
                          group=OneRankGroup(), device=dev)
        grouped.phy2log = phy2log
        grouped.deep_ep_initialized = True     # "the counts are already reduced": skips torch.distributed.all_reduce
        out_grouped = grouped.run(idx, avail, n_sms)
        assert torch.equal(out_grouped, planner.run(idx, avail, n_sms)), "group path and one-launch path disagree"
        extras["planner_run_with_group_us"] = round(
            pct(event_times_us(lambda: grouped.run(idx, avail, n_sms), 1000, 100, torch), 50), 2)
        extras["planner_run_with_group_wall_us"] = wall_us_per_call(lambda: grouped.run(idx, avail, n_sms))

    # ------------------------------------------------------------ CPU baseline
    torch.set_num_threads(1)
    idx_h, counts_h = inp.indices, inp.global_counts

    def cpu_plan():
        by = oracle.count_idx(idx_h, cfg.n_logical, n_sms)
        o_res, _, _ = oracle.solve(counts_h, cfg.r2o, inp.phy2log, 1, C, n_fixed)
        return oracle.map_idx(idx_h, o_res, by, o2r_host, inp.phy2log, 1, C, P)

    cpu_us = []
    t0c = time.perf_counter_ns()
    cpu_plan()
    cpu_us.append((time.perf_counter_ns() - t0c) / 1e3)
    t_end = time.perf_counter() + args.cpu_seconds
    while time.perf_counter() < t_end:
        t = time.perf_counter_ns()
        cpu_plan()
        cpu_us.append((time.perf_counter_ns() - t) / 1e3)
    cpu_baseline = {"value": round(pct(cpu_us, 50), 1), "unit": "us per plan (p50)", "cores": 1, "kind": "port",
                    "sample": f"{len(cpu_us)} plans of the same v3_ep8_cube inputs in {args.cpu_seconds:.0f} s, "
                              f"scalar C restatement of the reference algorithm, host has {os.cpu_count()} CPUs",
                    "p99": round(pct(cpu_us, 99), 1)}
    # The same plan on PyTorch CPU tensors (bincount / cumsum, dense fp32 LP, torch.linalg.cholesky, vectorised
    # redirect), once with one thread and once with every host core: 20 warm-up + up to 200 timed plans each.
    if args.cpu_seconds > 0:
        from oracle import torch_plan
        t_idx_h, t_counts_h = torch.from_numpy(idx_h), torch.from_numpy(counts_h)
        t_p2l_h, t_o2r_h = torch.from_numpy(inp.phy2log), torch.from_numpy(o2r_host)
        dense = torch_plan.DenseLp(cfg.r2o, C, n_fixed)

        def torch_cpu_plan():
            by = torch_plan.count_idx(t_idx_h, cfg.n_logical, n_sms)
            shares, _, _ = torch_plan.solve(t_counts_h, dense, t_p2l_h, 1)
            return torch_plan.map_idx(t_idx_h, shares, by, t_o2r_h, t_p2l_h, 1, C, P)
        torch_rows = {}
        for threads in (1, os.cpu_count() or 1):
            torch.set_num_threads(threads)
            for _ in range(20):
                torch_cpu_plan()
            samples = []
            t_stop = time.perf_counter() + args.cpu_seconds / 2
            while len(samples) < 200 and time.perf_counter() < t_stop:
                t = time.perf_counter_ns()
                torch_cpu_plan()
                samples.append((time.perf_counter_ns() - t) / 1e3)
            torch_rows[f"threads_{threads}"] = {"p50_us": round(pct(samples, 50), 1), "p99_us": round(pct(samples, 99), 1),
                                                "plans": len(samples), "torch_num_threads": torch.get_num_threads()}
        cpu_baseline["pytorch_cpu_restatement"] = torch_rows
        cpu_baseline["host_cpus"] = os.cpu_count()

    line = {
        "metric": "p50 us per plan (histogram + LP solve + redirect), EP8 cube V3 shape",
        "value": round(p50, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64 indices, f32 LP with f64 normal-equation solve",
        "data": "synthetic",
        "config": {"workload": "v3_ep8_cube: 256 logical + 16 redundant experts, EP8 cube r2o, int64 indices "
                               "[8192 x 8], global counts Zipf(1.0) x lognormal(0.3), n_blocks = CU count",
                   "n_blocks": n_sms},
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
