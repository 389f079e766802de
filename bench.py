#!/usr/bin/env python3
"""Benchmark of the placement-evaluation hot path on one MI355X.

A "step" is one pass of the approximate simulator over the whole batch of
candidate placements x arrival seeds of the workload (default: configuration 4,
16384 placements x 8 seeds x ~1M requests each), with request streams and
placement tables already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 4] [--placements N]

The CPU oracle is used here only for the `cpu_baseline` leg (a bounded sample of
the same workload, timed on the host cores) and to cross-check the GPU counts
of that sample; it is never part of what `value` measures.
"""
import argparse
import json
import os
import sys
import time
from concurrent.futures import ThreadPoolExecutor

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

FP64_VECTOR_PEAK_FMA_TFLOPS = 78.6   # MI355X published fp64 vector peak, FMA counted as 2
FP64_NON_FMA_PEAK_TOPS = 39.3        # the path has only add/max/compare: half of the above
LDS_PEAK_GBPS = 256 * 128 * 2.4      # 256 CUs x 128 B/clk x 2.4 GHz


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def kernel_sources_sha16():
    """First 16 hex digits of the SHA-256 over the library's kernel and host sources (mms_amd/csrc/*.hip, *.h,
    *.inc, in name order): what a recorded counter figure is tied to."""
    import glob
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "mms_amd", "csrc")
    for path in sorted(p for ext in ("*.hip", "*.h", "*.inc") for p in glob.glob(os.path.join(src, ext))):
        h.update(os.path.basename(path).encode() + b"\0")
        h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(kernel, workload):
    """HBM bytes per launch of `kernel` on `workload` from the committed counter summary
    (profiles/traffic.json: FETCH_SIZE / WRITE_SIZE of a rocprofv3 --pmc run, scaled by the same
    counters of a device copy of known size), and where the figure comes from.  The figure is a RECORDED one,
    not measured in this run (the counters need a profiler run of their own), so it is only given when the
    record is for this kernel instance, this workload and these very sources; otherwise None."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None, {"status": "no record"}
    sha = kernel_sources_sha16()
    for e in json.load(open(path)):
        if e["kernel"] == kernel and e["workload"] == workload:
            about = {"status": "recorded", "source": e.get("source"), "kernel_sources_sha16": e.get("kernel_sources_sha16"),
                     "measured_in_this_run": False}
            if e.get("kernel_sources_sha16") != sha:
                about["status"] = f"stale: the record is for other kernel sources (now {sha}); profile again"
                return None, about
            fetch = e["fetch_size_kib"] * e["copy_bytes"] / 1024.0 / e["copy_fetch_size_kib"]
            write = e["write_size_kib"] * e["copy_bytes"] / 1024.0 / e["copy_write_size_kib"]
            return (fetch + write) * 1024.0, about
    return None, {"status": "no record for this kernel and workload"}


def cpu_baseline(cfg, table, stream, sols, n_threads):
    """Times the C oracle (single thread, then n_threads threads over placement
    slices) on `sols` x one stream.  Returns (result dict of 1-thread run, evals/s 1T, evals/s MT)."""
    from mms_amd import engine as E
    from helpers import oracle_batch
    packed = E.pack_placements(sols, table)
    t0 = time.perf_counter()
    ref = oracle_batch(stream, table, packed, batching=cfg.batching)
    t1 = time.perf_counter() - t0
    evals = len(sols) * len(stream.tstamps)

    chunks = [sols[i::n_threads] for i in range(n_threads)]
    chunks = [c for c in chunks if c]
    packs = [E.pack_placements(c, table) for c in chunks]
    t0 = time.perf_counter()
    with ThreadPoolExecutor(len(chunks)) as pool:      # ctypes releases the GIL during the call
        list(pool.map(lambda p: oracle_batch(stream, table, p, batching=cfg.batching), packs))
    tm = time.perf_counter() - t0
    return ref, packed, evals / t1, evals / tm, t1


def model_stats_bench(args, cfg, streams):
    """One step = one mmsim_batch_model_stats call on the per-request outputs of B placements x the given
    streams (uploads of the window, kernel, copy of the [L][M] results).  Prints one JSON line."""
    from mms_amd import _lib, engine as E
    eng = E.Engine.default()
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    dws = [E.DeviceWorkload(eng, s.tstamps, s.model_ids, s.slos, cfg.num_models) for s in streams]
    flags = _lib.WANT_PER_REQUEST | (_lib.BATCHING if cfg.batching else 0)
    batch = E.Batch(eng, dws, table, E.pack_placements(cfg.placements, table), flags)
    batch.run()
    batch.sync()
    skip = [len(s.tstamps) // 50 for s in streams]
    for _ in range(args.warmup):
        batch.model_stats(skip)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        got = batch.model_stats(skip)
    sec = (time.perf_counter() - t0) / args.steps
    B, L = len(cfg.placements), len(cfg.placements) * len(streams)
    pairs = B * sum(len(s.tstamps) for s in streams)
    result = {
        "metric": "per-request outputs reduced to serving statistics, (simulation x request) pairs/sec",
        "value": pairs / sec, "unit": "pairs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": f"config {cfg.index} ({cfg.name}): statistics of {B} placements x {len(streams)} seeds, "
                               f"{len(streams[0].tstamps)} requests/seed, {cfg.num_models} models",
                   "kernel": "model_stats_kernel", "lanes": L},
        # finish (8 B) and good (1 B) of every (simulation, request) once: what one pass over the outputs reads;
        # the radix selection reads them eight times
        "roofline": {"bound": "hbm", "achieved": 9.0 * pairs / sec / 1e9, "peak": 8000.0, "unit": "GB/s",
                     "frac": 9.0 * pairs / sec / 8e12, "traffic": None,
                     "note": "achieved = 9 algorithmic bytes per (simulation, request) over the whole call"},
    }
    if not args.no_cpu:     # the same statistics with numpy on the fetched outputs, first placement of the first stream
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        from oracle_backend import model_stats_numpy
        out = batch.fetch()
        st = streams[0]
        R = len(st.tstamps)
        t0 = time.perf_counter()
        want = model_stats_numpy(st.tstamps, st.model_ids, out["finish"][0, 0, :R], out["good"][0, 0, :R], skip[0],
                                 cfg.num_models)
        t1 = time.perf_counter() - t0
        same = all(np.array_equal(got[k][0, 0], want[k]) for k in
                   ("model_num_requests", "model_num_good", "first_start", "last_start", "latency_p90", "latency_p99"))
        close = all(np.allclose(got[k][0, 0], want[k], rtol=1e-12, atol=0) for k in ("latency_sum", "latency_mean", "latency_std"))
        result["cpu_baseline"] = {"value": R / t1, "unit": "pairs/s", "cores": 1, "kind": "port",
                                  "sample": f"placement 0 x seed 0 ({R} requests, {t1:.2f}s), numpy sort per model on the copied outputs",
                                  "gpu_equals_cpu_on_sample": bool(same and close)}
    batch.close()
    print(json.dumps(result), flush=True)


class _StopSearch(Exception):
    """Raised by the bench's evaluator hook to end a search after a given number of evaluator calls."""


class _CallLog:
    """Counts and times the evaluator's library calls of one search (whatever backend is installed in
    mms_amd.engine), keeps a digest of what every call returned, and can end the search after `max_calls`
    calls or once the calls have used `budget_s` seconds."""

    def __init__(self, engine_module, max_calls=None, budget_s=None):
        self.E = engine_module
        self.max_calls, self.budget_s = max_calls, budget_s
        self.calls, self.placements, self.in_calls = 0, 0, 0.0
        self.stamps, self.digests = [], []

    def __enter__(self):
        import hashlib
        self._saved = (self.E.evaluate, self.E.evaluate_successors)
        self.t0 = time.perf_counter()

        def wrap(fn, count):
            def hooked(*a, **k):
                if (self.max_calls is not None and self.calls >= self.max_calls) or \
                        (self.budget_s is not None and self.in_calls >= self.budget_s):
                    raise _StopSearch()
                t = time.perf_counter()
                out = fn(*a, **k)
                self.in_calls += time.perf_counter() - t
                self.calls += 1
                self.placements += count(a)
                self.stamps.append(time.perf_counter() - self.t0)
                h = hashlib.sha256(np.ascontiguousarray(out["n_good"]).tobytes())
                h.update(np.ascontiguousarray(out["latency_sum"]).tobytes())
                self.digests.append(h.hexdigest()[:12])
                return out
            return hooked
        self.E.evaluate = wrap(self._saved[0], lambda a: len(a[3]))
        self.E.evaluate_successors = wrap(self._saved[1], lambda a: len(a[3]) + len(a[4]))
        return self

    def __exit__(self, *exc):
        self.E.evaluate, self.E.evaluate_successors = self._saved
        self.seconds = time.perf_counter() - self.t0
        return exc[0] is _StopSearch


def search_bench(args):
    """Wall clock of whole placement searches (the callers of the hot path) on the GPU, each with the SAME search
    code timed beside it on one host core (`cpu_baseline`: the C oracle behind the evaluator, one placement after
    another as the reference's loop does, plain greedy loop).  Greedy searches are sequential (one placement per
    step): the GPU runs them with the one-step look-ahead; beam, layout-enumeration and evolutionary searches send
    hundreds to thousands of placements per call.  A CPU leg that would take minutes is cut after about
    `--cpu-budget` seconds of evaluator calls and compared with the GPU's time for the same calls (the calls must
    have returned the same numbers).  Also measured: how long one evaluator call takes against its number of
    placements on both sides, i.e. from how many placements per call the GPU pays.  Prints one JSON line; `value`
    is placements scored per second over the batch-shaped searches."""
    import pytest
    import oracle_backend
    from mms_amd import engine as E
    from mms_amd.placement_policy import (ClusterEnv, ModelData, ModelParallelismGreedy, ModelParallelismSearch,
                                          ModelPlacement, PlacementEvaluator, SelectiveReplicationGreedy,
                                          SelectiveReplicationSearch)
    from mms_amd.placement_policy import base_policy
    from mms_amd.placement_policy.base_policy import evolutionary_search, replica_placement_beam_search
    from mms_amd.profiling import ParallelConfig, synthetic_profile
    from mms_amd.simulator.workload import GammaProcess, Workload
    from mms_amd.synthetic import power_law_rates
    GB = 1 << 30

    def problem(num_models, num_devices, total_rate, duration, configs):
        rates = power_law_rates(num_models, total_rate, 0.6)
        model_datas = []
        for i in range(num_models):
            base = [0.15, 0.25, 0.5][i % 3]
            prof = synthetic_profile(f"p{i % 3}", base, configs, weight_bytes=[2.6, 5.2, 13.4][i % 3] * GB)
            model_datas.append(ModelData(f"m{i}", base * 5, float(rates[i]), 4.0, prof))
        workload = Workload.merge(*[GammaProcess(md.rate, md.cv).generate_workload(md.name, 0, duration, slo=md.slo, seed=100 + i)
                                    for i, md in enumerate(model_datas)])
        return model_datas, ClusterEnv(num_devices, 13 * GB), workload

    # (profiles up to 32 stages: the evolutionary search merges groups into deeper pipelines)
    pipe = [ParallelConfig(1, 1, pp) for pp in (1, 2, 4, 8, 16, 32)]
    md32, env32, wl32 = problem(32, 32, 60.0, 1800.0 * args.search_scale, pipe)
    wide = sorted({ParallelConfig(1, op, pp) for op in (1, 2, 4) for pp in (1, 2, 4, 8, 16, 32)})
    md64, env64, wl64 = problem(64, 64, 120.0, 900.0 * args.search_scale, wide)
    log(f"[bench] search problems: 32 models / 32 devices / {len(wl32)} requests; 64 models / 64 devices / {len(wl64)} requests")

    def evo(model_datas, env, wl, iters):
        def run():
            np.random.seed(0)
            ev = PlacementEvaluator(model_datas, env, wl, "fast_simulator", False)
            # start: every device its own group with one of the small models; the search does the rest
            init = ModelPlacement([ParallelConfig(1, 1, 1)] * env.num_devices,
                                  [[(3 * g) % len(model_datas)] for g in range(env.num_devices)])
            return evolutionary_search([init], model_datas, env, ev, iters, 0)
        return run

    def beam_pp4(model_datas, env, wl):
        def run():
            ev = PlacementEvaluator(model_datas, env, wl, "fast_simulator", False)
            n = env.num_devices // 4
            init = ModelPlacement([ParallelConfig(1, 1, 4)] * n, [[] for _ in range(n)])
            return replica_placement_beam_search(init, model_datas, env, wl, ev, 3, 0)
        return run

    # name -> (search, kind).  "sequential": one placement per step; "batch": many placements per call
    searches = [
        ("ModelParallelismSearch, 32 models / 32 devices (3 layouts, greedy)",
         lambda: ModelParallelismSearch(verbose=0).solve_placement(md32, env32, wl32)[0], "sequential"),
        ("SelectiveReplicationGreedy, 32 / 32",
         lambda: SelectiveReplicationGreedy(verbose=0).solve_placement(md32, env32, wl32)[0], "sequential"),
        ("ModelParallelismGreedy(group_size=4), 32 / 32",
         lambda: ModelParallelismGreedy(group_size=4).solve_placement(md32, env32, wl32)[0], "sequential"),
        ("ModelParallelismSearch, 64 models / 64 devices (12 layouts in lockstep, greedy)",
         lambda: ModelParallelismSearch(verbose=0).solve_placement(md64, env64, wl64)[0], "sequential"),
        ("SelectiveReplicationSearch (beam 3), 32 / 32",
         lambda: SelectiveReplicationSearch(verbose=0).solve_placement(md32, env32, wl32)[0], "batch"),
        ("replica_placement_beam_search (beam 3) on 8 groups of 4 stages, 32 / 32", beam_pp4(md32, env32, wl32), "batch"),
        ("evolutionary_search (population 1024, 8 iterations), 32 / 32", evo(md32, env32, wl32, 8), "batch"),
        ("evolutionary_search (population 1024, 4 iterations), 64 / 64", evo(md64, env64, wl64, 4), "batch"),
    ]

    # warm-up: library, context, first launches
    ModelParallelismSearch(verbose=0).solve_placement(md32[:4], ClusterEnv(4, 13 * GB), wl32)

    rows = {}
    batch_placements, batch_seconds = 0, 0.0
    all_same = True
    for name, run, kind in searches:
        row = {"kind": kind}
        base_policy.FAST_GREEDY_LOOKAHEAD = True
        with _CallLog(E) as gpu:
            sol = run()
        row["gpu"] = {"seconds": gpu.seconds, "evaluator_calls": gpu.calls, "placements_scored": gpu.placements,
                      "seconds_inside_calls": gpu.in_calls}
        if kind == "sequential":    # the same search without the look-ahead, for the record
            base_policy.FAST_GREEDY_LOOKAHEAD = False
            with _CallLog(E) as plain:
                sol_plain = run()
            row["gpu_without_lookahead"] = {"seconds": plain.seconds, "evaluator_calls": plain.calls}
            row["same_placement_with_and_without_lookahead"] = str(sol) == str(sol_plain)
            all_same = all_same and row["same_placement_with_and_without_lookahead"]
        if not args.no_cpu:
            # the same search code on one host core: the C oracle behind the evaluator, plain greedy loop
            mp = pytest.MonkeyPatch()
            oracle_backend.install(mp)
            base_policy.FAST_GREEDY_LOOKAHEAD = False
            try:
                with _CallLog(E, budget_s=args.cpu_budget if kind == "batch" else None) as cpu:
                    sol_cpu = run()
                    cpu.finished = True
            finally:
                mp.undo()
                base_policy.FAST_GREEDY_LOOKAHEAD = True
            finished = getattr(cpu, "finished", False)
            if finished:
                gpu_same_work = gpu.seconds
                same = str(sol) == str(sol_cpu)
            else:           # cut short: compare with the GPU's time up to the same call, the calls must agree
                k = cpu.calls
                gpu_same_work = gpu.stamps[k - 1] if 0 < k <= len(gpu.stamps) else float("nan")
                same = k > 0 and cpu.digests[:k] == gpu.digests[:k]
                cpu.seconds = cpu.stamps[k - 1] if k else float("nan")
            row["cpu_baseline"] = {
                "seconds": cpu.seconds, "cores": 1, "kind": "port", "evaluator_calls": cpu.calls,
                "placements_scored": cpu.placements, "complete_search": finished,
                "sample": "the whole search" if finished else f"the first {cpu.calls} evaluator calls of the search "
                          f"({cpu.placements} placements; cut after {args.cpu_budget:.0f} s inside the calls)",
                "gpu_seconds_for_the_same_work": gpu_same_work,
                "gpu_speedup_over_one_core": cpu.seconds / gpu_same_work,
                "same_result_as_gpu": bool(same)}
            all_same = all_same and bool(same)
        if kind == "batch":
            batch_placements += gpu.placements
            batch_seconds += gpu.seconds
        rows[name] = row
        cb = row.get("cpu_baseline", {})
        log(f"[bench] {name}: GPU {gpu.seconds:.2f} s / {gpu.calls} calls / {gpu.placements} placements"
            + (f"; one core {cb['seconds']:.2f} s ({'whole search' if cb['complete_search'] else str(cb['evaluator_calls']) + ' calls'}), "
               f"GPU for the same work {cb['gpu_seconds_for_the_same_work']:.2f} s -> {cb['gpu_speedup_over_one_core']:.2f}x, "
               f"same result {cb['same_result_as_gpu']}" if cb else ""))

    # One evaluator call against its number of placements (counts level, what get_stats asks for), on both sides:
    # the GPU's call time is flat until the chip fills, one core's grows linearly; they cross where the GPU pays.
    crossover = {"placements_per_call": [], "gpu_ms": [], "cpu_ms": []}
    ev = PlacementEvaluator(md32, env32, wl32, "fast_simulator", False)
    final, _ = SelectiveReplicationGreedy(verbose=0).solve_placement(md32, env32, wl32)
    rng = np.random.default_rng(0)
    pool = []
    for _ in range(4096):      # placements like the ones the searches score: the greedy result with a few replicas dropped
        rows_ = [list(ms) for ms in final.group_models]
        for _ in range(4):
            g = int(rng.integers(len(rows_)))
            if len(rows_[g]) > 1:
                rows_[g].pop(int(rng.integers(len(rows_[g]))))
        pool.append(ModelPlacement(final.group_configs, rows_))
    ev.get_stats(pool[:2])
    cpu_ms_per_placement = None
    if not args.no_cpu:
        mp = pytest.MonkeyPatch()
        oracle_backend.install(mp)
        try:
            ev_cpu = PlacementEvaluator(md32, env32, wl32, "fast_simulator", False)
            t0 = time.perf_counter()
            ev_cpu.get_stats(pool[:64])
            cpu_ms_per_placement = (time.perf_counter() - t0) * 1e3 / 64
        finally:
            mp.undo()
    for n in (1, 8, 64, 256, 1024, 4096):
        t0 = time.perf_counter()
        for _ in range(3):
            ev.get_stats(pool[:n])
        crossover["placements_per_call"].append(n)
        crossover["gpu_ms"].append((time.perf_counter() - t0) * 1e3 / 3)
        crossover["cpu_ms"].append(None if cpu_ms_per_placement is None else cpu_ms_per_placement * n)
    if cpu_ms_per_placement is not None:
        crossover["cpu_ms_per_placement"] = cpu_ms_per_placement
        crossover["gpu_pays_from_placements_per_call"] = crossover["gpu_ms"][0] / cpu_ms_per_placement
    log(f"[bench] one get_stats call: {crossover}")

    print(json.dumps({
        "metric": "placements scored per second inside whole batch-shaped placement searches (beam, evolutionary)",
        "value": batch_placements / batch_seconds, "unit": "placements/s", "n_gpus": 1, "steps": 1, "warmup": 1,
        "ms_per_step": batch_seconds * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": f"placement searches: 32 models / 32 devices / {len(wl32)} training requests and "
                               f"64 models / 64 devices / {len(wl64)} training requests, 13 GB per device"},
        "searches": rows, "one_evaluator_call": crossover, "every_search_gave_the_same_result_on_both_sides": bool(all_same)}),
        flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", type=int, default=4,
                    help="synthetic configuration 1..5 (4 is the headline; 5 runs the batching simulator)")
    ap.add_argument("--placements", type=int, default=None, help="truncate the candidate list")
    ap.add_argument("--seeds", type=int, default=None, help="use only the first N arrival seeds")
    ap.add_argument("--cpu-sample", type=int, default=2048, help="placements timed on the CPU oracle")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="also launch one plain device copy of BYTES (read BYTES, write BYTES) so that "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiled run can be scaled")
    ap.add_argument("--flags", type=str, default="scores", choices=["scores", "model", "stats"],
                    help="scores: goodput+latency only; model: + per-model counts; stats: + per-group counts")
    ap.add_argument("--model-stats", action="store_true",
                    help="time mmsim_batch_model_stats (serving statistics of the per-request outputs, on the device) "
                         "instead of the simulation; the per-request outputs of every simulation stay on the device, so "
                         "it defaults to --placements 64 --seeds 1")
    ap.add_argument("--search", action="store_true",
                    help="time whole placement searches (the callers of the hot path: greedy, layout enumeration, beam, "
                         "evolutionary) on the GPU and, the same search code, on one host core, instead of the simulation")
    ap.add_argument("--search-scale", type=float, default=1.0,
                    help="--search: scales the length of the training workloads (for a quick run)")
    ap.add_argument("--cpu-budget", type=float, default=15.0,
                    help="--search: seconds of evaluator calls after which the one-core leg of a batch-shaped search is cut")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="a field of the library's options (mmsim_options in include/mmsim.h), e.g. batching_lds_tables=2; "
                         "repeatable; the default run sets none")
    args = ap.parse_args()
    if args.model_stats:    # 9 bytes per (simulation, request): the full batch would not fit
        args.placements = 64 if args.placements is None else args.placements
        args.seeds = 1 if args.seeds is None else args.seeds

    if args.gpus != 1:
        print("bench.py: this build evaluates placements on ONE GPU; --gpus must be 1 "
              "(lanes are independent, a multi-GPU run would only split the batch).", file=sys.stderr)
        sys.exit(2)

    if args.search:
        return search_bench(args)

    from mms_amd import _lib, engine as E
    from mms_amd.synthetic import make_config

    t0 = time.perf_counter()
    cfg = make_config(args.config, args.placements)
    seeds = list(cfg.base_seeds if args.seeds is None else cfg.base_seeds[:args.seeds])
    streams = [cfg.stream(s) for s in seeds]
    B = len(cfg.placements)
    R_total = sum(len(s.tstamps) for s in streams)
    log(f"[bench] {cfg.name}: {B} placements x {len(seeds)} seeds, {R_total} requests over seeds, "
        f"inputs generated in {time.perf_counter() - t0:.1f}s")

    if args.copy_calibration:
        import torch
        src = torch.ones(args.copy_calibration // 4, dtype=torch.int32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)                      # the calibration launch (the fill above is a write-only kernel)
        torch.cuda.synchronize()
        log(f"[bench] copy calibration: one device copy of {args.copy_calibration} bytes")
        del src, dst

    if args.model_stats:
        return model_stats_bench(args, cfg, streams)

    eng = E.Engine.default()
    dev = eng.device_info()
    log(f"[bench] device: {dev}")
    if args.option:
        eng.set_options(**{k: int(v) for k, v in (kv.split("=", 1) for kv in args.option)})
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    t0 = time.perf_counter()
    packed = E.pack_placements(cfg.placements, table)
    t_pack = time.perf_counter() - t0
    flags = {"scores": 0, "model": _lib.WANT_MODEL_COUNTS,
             "stats": _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS}[args.flags]
    if cfg.batching:
        flags |= _lib.BATCHING
    t0 = time.perf_counter()
    dws = [E.DeviceWorkload(eng, s.tstamps, s.model_ids, s.slos, cfg.num_models) for s in streams]
    batch = E.Batch(eng, dws, table, packed, flags)
    t_upload = time.perf_counter() - t0
    info = batch.info()
    batch_kernel = batch.kernel_name()
    log(f"[bench] kernel: {batch_kernel}")
    log(f"[bench] batch: {info}; python pack {t_pack:.2f}s, library pack+upload {t_upload:.2f}s")

    for _ in range(args.warmup):
        batch.run()
        batch.sync()
    kernel_ms = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        batch.run()
        kernel_ms.append(batch.sync())          # HIP events around the kernel, on its stream
    wall = time.perf_counter() - t0
    out = batch.fetch()
    batch.close()

    evals_per_step = R_total * B
    lanes = B * len(seeds)
    sec_per_step = wall / args.steps
    kernel_s = float(np.mean(kernel_ms)) / 1e3
    value = evals_per_step / sec_per_step

    kernel = batch_kernel
    workload = (f"config {cfg.index} ({cfg.name}): {cfg.num_models} models, {cfg.num_devices} devices, "
                f"{B} candidate placements x {len(seeds)} seeds, {R_total // len(seeds)} requests/seed")
    # Operations of the reference loop on these inputs.  Plain simulator: 2*stages + replicas + 3 per dispatched
    # request, counted exactly by one untimed pass of the kernel itself (and cross-checked against the oracle on
    # the CPU sample below).  Batching simulator: 2*stages + 2 per check_slo call (+1 for a head's deadline) and
    # 2*stages + 1 per committed batch, counted by the oracle on the CPU sample and scaled to the batch.
    total_ops = None
    achieved_tops = None
    ops_note = "achieved counts 2*stages+replicas+3 per dispatched request of the reference loop (what the " \
               "reference executes on these inputs, not what this kernel executes: it keeps choices and skips requests)"
    if not cfg.batching:
        ops_batch = E.Batch(eng, dws, table, packed, _lib.WANT_OP_COUNT)
        ops_batch.run()
        ops_batch.sync()
        ops_out = ops_batch.fetch()
        ops_batch.close()
        total_ops = int(ops_out["fp_ops"].sum())
        assert np.array_equal(ops_out["n_good"], out["n_good"])
        achieved_tops = total_ops / kernel_s / 1e12
    else:
        assert np.all(out["status"] == 0), "a lane ran out of idle-event slots"
        ops_note = "achieved counts 2*stages+2 per check_slo call (+1 per head deadline) and 2*stages+1 per committed " \
                   "batch of the reference loop, counted by the oracle on the CPU sample and scaled to the batch"

    traffic, traffic_record = measured_traffic(kernel, workload) if args.flags == "scores" else (None, {"status": "not recorded for this output level"})

    hbm_bytes = info["stream_bytes"] + info["table_bytes"] + 12 * lanes
    # dispatched requests = evaluations whose model has a replica: every one costs 3 operations beyond clocks
    dispatched = None
    if total_ops is not None:
        hosted = np.zeros((B, cfg.num_models), bool)
        for p, pl in enumerate(cfg.placements):
            for ms in pl.group_models:
                hosted[p, list(ms)] = True
        per_model = np.zeros(cfg.num_models)
        for st in streams:
            ids = st.model_ids[st.model_ids >= 0]
            per_model += np.bincount(ids, minlength=cfg.num_models)
        dispatched = float((hosted * per_model[None, :]).sum())

    result = {
        "metric": "simulated request x placement evals/sec",
        "value": value,
        "unit": "evals/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": workload, "kernel": kernel,
                   "workgroups": info["workgroups"], "wavefronts_per_workgroup": info["waves_per_group"],
                   "lds_bytes_per_workgroup": info["lds_bytes"], "stream_segments": info["segments"],
                   "placements": B, "seeds": len(seeds), "requests_per_seed": R_total // len(seeds),
                   "lanes": lanes, "outputs": args.flags, "inputs_resident_in_hbm": True,
                   **({"options": args.option} if args.option else {})},
        "placements_per_sec": lanes / sec_per_step,
        "kernel_ms": kernel_s * 1e3,
        "goodput_mean": float(out["n_good"].sum() / evals_per_step),
        "roofline": {
            "bound": "valu_fp64",
            "achieved": achieved_tops,
            "peak": FP64_NON_FMA_PEAK_TOPS,
            "unit": "TFLOP/s",
            "frac": None if achieved_tops is None else achieved_tops / FP64_NON_FMA_PEAK_TOPS,
            "frac_of_published_fma_peak": None if achieved_tops is None else achieved_tops / FP64_VECTOR_PEAK_FMA_TFLOPS,
            "ops_per_launch": total_ops,
            "ops_per_eval": None if total_ops is None else total_ops / evals_per_step,
            "traffic": traffic,
            "traffic_record": traffic_record,
            "note": "fp64 add/max/compare only (no FMA): peak = published 78.6 TFLOP/s / 2; " + ops_note,
            # the two other ceilings of this path, for the record: compulsory HBM bytes (streams once per
            # wavefront group + tables + results) and algorithmic LDS bytes (8 per clock read or written:
            # 2*stages + replicas per dispatched request) against 8 TB/s and 256 CUs x 128 B/clk x 2.4 GHz
            "hbm": {"achieved_GBps": hbm_bytes / kernel_s / 1e9, "peak_GBps": 8000.0,
                    "frac": hbm_bytes / kernel_s / 8e12, "bytes_per_launch": hbm_bytes},
            "lds": None if total_ops is None else {
                "achieved_GBps": 8.0 * (total_ops - 3 * dispatched) / kernel_s / 1e9, "peak_GBps": LDS_PEAK_GBPS,
                "frac": 8.0 * (total_ops - 3 * dispatched) / kernel_s / 1e9 / LDS_PEAK_GBPS},
        },
    }

    if not args.no_cpu:
        n_threads = min(16, os.cpu_count() or 1)
        sample = cfg.placements[:min(args.cpu_sample, B)]
        ref, spacked, c1, cm, t1 = cpu_baseline(cfg, table, streams[0], sample, n_threads)
        same = np.array_equal(out["n_good"][0, :len(sample)], ref["n_good"])
        if cfg.batching:        # scale the sample's operation count to the whole batch
            sample_evals = len(sample) * len(streams[0].tstamps)
            total_ops = int(round(ref["fp_ops"] / sample_evals * evals_per_step))
            rf = result["roofline"]
            rf["achieved"] = total_ops / kernel_s / 1e12
            rf["frac"] = rf["achieved"] / FP64_NON_FMA_PEAK_TOPS
            rf["frac_of_published_fma_peak"] = rf["achieved"] / FP64_VECTOR_PEAK_FMA_TFLOPS
            rf["ops_per_launch"] = total_ops
            rf["ops_per_eval"] = total_ops / evals_per_step
        result["cpu_baseline"] = {
            "value": c1, "unit": "evals/s", "cores": 1, "kind": "port",
            "sample": f"first {len(sample)} placements x seed {seeds[0]} "
                      f"({len(sample) * len(streams[0].tstamps)} evals, {t1:.1f}s), C oracle -O2, request loop only",
            "value_all_cores": cm, "cores_all": n_threads,
            "gpu_over_cpu_1core": value / c1, "gpu_over_cpu_all_cores": value / cm,
            "gpu_counts_match_cpu_on_sample": bool(same),
        }
        if not same:
            log("[bench] WARNING: GPU and CPU goodput counts differ on the CPU sample")
    print(json.dumps(result))


if __name__ == "__main__":
    main()
