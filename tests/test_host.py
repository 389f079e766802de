"""Host-side logic that needs no GPU: the C ABI surface, table packing,
workload generation and statistics, helpers."""
import ctypes
import os
import re

import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.placement_policy import ClusterEnv, ModelData, ModelPlacement
from mms_amd.profiling import (LatencyMemData, ParallelConfig, ProfilingResult, load_test_prof_result,
                               synthetic_profile)
from mms_amd.simulator.workload import (DeterministicProcess, GammaProcess, PoissonProcess, Request,
                                        Workload)
from mms_amd.synthetic import gamma_arrivals_fast, make_config, power_law_rates
from mms_amd.util import (GB, decompose2tok, get2tok, get_factors, get_partitions, is_valid_size,
                          to_str_round)
from oracle import oracle_py

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI ------------------------------------------------------------------------------

def test_library_loads_and_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mmsim.h")).read()
    declared = set(re.findall(r"\b(mmsim_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in mmsim.h but not exported"
    assert declared == set(_lib.SIGNATURES), "ctypes signatures and header disagree"
    assert lib.mmsim_abi_version() == int(re.search(r"#define MMSIM_ABI_VERSION (\d+)", header).group(1))


def test_no_device_means_a_loud_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(_lib.MmsimError) as e:
        E.Engine(0)
    assert e.value.code == _lib.E_HIP and "HIP device" in str(e.value)


def test_struct_layouts_match_the_header():
    assert ctypes.sizeof(_lib.Tables) == 48
    assert ctypes.sizeof(_lib.Placements) == 40
    assert ctypes.sizeof(_lib.Result) == 10 * 8
    assert ctypes.sizeof(_lib.BatchInfo) == 8 * 4 + 3 * 8 + 6 * 4
    assert ctypes.sizeof(_lib.ModelStats) == 9 * 8
    # field order of mmsim_model_stats as the header declares it
    header = open(os.path.join(ROOT, "include", "mmsim.h")).read()
    body = re.search(r"typedef struct \{([^}]*)\} mmsim_model_stats;", header).group(1)
    assert re.findall(r"\*(\w+);", body) == [f[0] for f in _lib.ModelStats._fields_]
    # mmsim_options: field order and size, and the defaults the library fills in (no GPU needed)
    body = re.search(r"typedef struct \{([^}]*)\} mmsim_options;", header).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    assert re.findall(r"int(?:32|64)_t (\w+);", body) == [f[0] for f in _lib.Options._fields_]
    assert ctypes.sizeof(_lib.Options) == 14 * 4 + 8
    opt = _lib.Options()
    _lib.load().mmsim_options_default(ctypes.byref(opt))
    assert opt.struct_size == ctypes.sizeof(_lib.Options)
    assert (opt.request_loop, opt.counts_in_lds, opt.skip_ahead, opt.sched_spin_limit, opt.batching_lds_tables) == (-1,) * 5
    assert (opt.waves_per_cu, opt.sched_groups, opt.segment_requests, opt.batching_lanes, opt.stats_scratch_bytes) == (0,) * 5


def test_weighted_choice_is_numpys_choice():
    """The evolutionary search draws parents and models with np.random.choice(n, p=...) in the reference
    (base_policy.py:662, 679); the drop-in's shortcut must consume the same draw and return the same index."""
    from mms_amd.placement_policy.base_policy import _choice_cdf, _weighted_choice
    rng = np.random.default_rng(0)
    for trial in range(300):
        n = int(rng.integers(1, 40))
        p = rng.random(n) ** 3
        p[rng.random(n) < 0.2] = 0.0
        if p.sum() == 0:
            p[0] = 1.0
        p = p / np.sum(p)
        cdf = _choice_cdf(p)
        np.random.seed(trial)
        want = [np.random.choice(n, p=p) for _ in range(5)] + [np.random.uniform()]
        np.random.seed(trial)
        got = [_weighted_choice(cdf) for _ in range(5)] + [np.random.uniform()]
        assert got == want


def test_a_failed_simulation_is_an_error_not_a_score(monkeypatch):
    """A batching simulation whose status is not 0 ran out of event slots (or met an unsupported input); its
    counts and per-request outputs are partly unwritten.  Whatever turns results into scores or statistics must
    raise instead of using them: the evaluator, the replacement path and the device statistics."""
    import oracle_backend
    from mms_amd.placement_policy import ModelPlacementWithReplacement, PlacementEvaluator, gen_train_workload
    from mms_amd.simulator import controller as sim
    oracle_backend.install(monkeypatch)
    ok = E.check_status(np.zeros((2, 3), np.int32))
    assert ok is None
    with pytest.raises(_lib.MmsimError) as err:
        E.check_status(np.array([[0, 0, 0], [0, _lib.E_OVERFLOW, 0]], np.int32))
    assert err.value.code == _lib.E_OVERFLOW and "(1, 1)" in str(err.value)

    model_datas = [ModelData(f"m{i}", 1.0, 4, 1, load_test_prof_result("test-2GB-100ms")) for i in range(3)]
    cluster_env = ClusterEnv(4, 64 * GB)
    sol = ModelPlacement([ParallelConfig(1, 1, 2), ParallelConfig(1, 1, 2)], [[0, 1, 2], [0, 1, 2]])
    wl = gen_train_workload(model_datas, simulation_min_samples=2000)
    forced = {"code": _lib.E_OVERFLOW}

    def failing(fn):
        def wrapped(*a, **k):
            out = fn(*a, **k)
            out["status"] = np.full_like(out["status"], forced["code"])
            if not k.get("allow_failed", False):
                E.check_status(out["status"])
            return out
        return wrapped
    monkeypatch.setattr(E, "evaluate", failing(E.evaluate))
    monkeypatch.setattr(E, "eval_pairs", failing(E.eval_pairs))
    ev = PlacementEvaluator(model_datas, cluster_env, wl, "fast_simulator", False)
    for call in (lambda: ev.get_scores([sol]), lambda: ev.get_stats([sol]),
                 lambda: ev.get_scores([ModelPlacementWithReplacement([0, 50], [sol, sol])])):
        with pytest.raises(_lib.MmsimError) as err:
            call()
        assert err.value.code == _lib.E_OVERFLOW

    class FailingBatch(oracle_backend._HostBatch):
        def fetch(self, per_request=True, allow_failed=False):
            out = super().fetch(per_request)
            out["status"] = np.full_like(out["status"], _lib.E_UNSUPPORTED)
            if not allow_failed:
                E.check_status(out["status"])
            return out
    monkeypatch.setattr(E, "Batch", FailingBatch)
    ev._prepare()
    model_ids, slos, names, profs = wl.cached_data
    with pytest.raises(_lib.MmsimError) as err:
        sim.device_compute_stats(wl, [sol], names, profs, model_ids, slos, 10)
    assert err.value.code == _lib.E_UNSUPPORTED


# ---- table build (controller.py:412-476) --------------------------------------------------

def test_latency_table_values_follow_the_reference_formula():
    profs = [load_test_prof_result("alpa/bert-1.3b"), load_test_prof_result("test-2GB-100ms"),
             load_test_prof_result("alpa/bert-2.6b")]
    table = E.LatencyTable(profs)
    cfgs = [ParallelConfig(1, 1, 4), ParallelConfig(1, 1, 1), ParallelConfig(1, 1, 8), ParallelConfig(1, 1, 2)]
    ids = [table.config_id(c) for c in cfgs]
    assert ids == [0, 1, 2, 3] and table.config_id(cfgs[2]) == 2
    lat, pp = table.arrays()
    assert lat.shape == (3, 4, 8, 1) and pp.tolist() == [4, 1, 8, 2]
    # the independent restatement builds the per-placement table; compare column by column
    m2g, g2m, ns, ref = oracle_py.build_tables(cfgs, [[0, 1, 2]] * 4, profs)
    for c, cfg in enumerate(cfgs):
        assert np.array_equal(lat[:, c, :cfg.pp, 0], ref[:, c, :cfg.pp, 0])
    assert np.float32(0.028 * (1 + 0.009 * 4)) == lat[0, 0, 0, 0]
    assert np.isinf(lat[2, 0]).all() and np.isinf(lat[1, 2]).all()      # configs without a profile
    # batch sizes: the penalty still comes from the batch-1 stage list
    prof = synthetic_profile("x", 0.2, [ParallelConfig(1, 1, 2)], batch_sizes=(1, 2, 4), batch_slope=0.15)
    t2 = E.LatencyTable([prof], [1, 2, 4])
    t2.config_id(ParallelConfig(1, 1, 2))
    lat2, _ = t2.arrays()
    want = [np.float32(prof.para_dict[ParallelConfig(1, 1, 2)].latency[b][0] * (1 + 0.009 * 2)) for b in (1, 2, 4)]
    assert lat2[0, 0, 0].tolist() == want and lat2[0, 0, 1].tolist() == want


def test_pack_placements_layout():
    table = E.LatencyTable([load_test_prof_result("test-2GB-100ms")] * 5)
    sols = [ModelPlacement([ParallelConfig(1, 1, 2)] * 2, [[0, 1, 2, 3], (0, 1)]),
            ModelPlacement([ParallelConfig(1, 1, 4)], [np.array([3, 2])]),
            ModelPlacement([], []),
            ModelPlacement([ParallelConfig(1, 1, 1), ParallelConfig(1, 1, 2), ParallelConfig(1, 1, 1)], [[], [4], []])]
    ng, gc, off, idx = E.pack_placements(sols, table)
    assert ng.tolist() == [2, 1, 0, 3]
    assert gc.tolist() == [[0, 0, 0], [1, 0, 0], [0, 0, 0], [2, 0, 2]]
    assert off.tolist() == [[0, 4, 6, 6], [6, 8, 8, 8], [8, 8, 8, 8], [8, 8, 9, 9]]
    assert idx.tolist() == [0, 1, 2, 3, 0, 1, 3, 2, 4]


def test_placement_helpers():
    p = ModelPlacement([ParallelConfig(1, 1, 2), ParallelConfig(1, 1, 1), ParallelConfig(1, 1, 4)], [[3, 1], [0], [2, 0]])
    q = p.add_model(1, 5)
    assert p.group_models[1] == [0] and q.group_models[1] == [0, 5] and q.group_configs is p.group_configs
    n = q.normalize()
    assert n.group_models == ((0, 2), (0, 5), (1, 3))
    assert n.group_configs == (ParallelConfig(1, 1, 4), ParallelConfig(1, 1, 1), ParallelConfig(1, 1, 2))
    c = p.copy()
    c.group_models[0].append(9)
    assert p.group_models[0] == [3, 1]
    md = [ModelData(f"m{i}", 1, 1, 1, load_test_prof_result("test-2GB-100ms")) for i in range(4)]
    ModelPlacement([ParallelConfig(1, 1, 1)], [[0, 1]]).verify(md, ClusterEnv(1, 4.5 * GB))
    with pytest.raises(AssertionError):
        ModelPlacement([ParallelConfig(1, 1, 1)], [[0, 1, 2]]).verify(md, ClusterEnv(1, 4.5 * GB))
    with pytest.raises(AssertionError):
        ModelPlacement([ParallelConfig(1, 1, 2)], [[0, 0]]).verify(md, ClusterEnv(2, 4.5 * GB))
    with pytest.raises(AssertionError):      # no profile for this config -> infinite memory
        ModelPlacement([ParallelConfig(1, 2, 1)], [[0]]).verify(md, ClusterEnv(2, 4.5 * GB))


# ---- workloads (workload.py) ------------------------------------------------------------------

def test_gamma_arrivals_fast_equals_the_sequential_loop():
    for rate, cv, dur, seed in [(2.5, 1, 60, 0), (1, 4, 300, 7), (0.05, 8, 1000, 3), (30, 8, 100, 5),
                                (0.3, 6, 50, 11), (0.01, 2, 400, 2), (0.02, 1, 90, 4), (0.011, 3, 95, 8)]:
        slow = np.array(GammaProcess(rate, cv).generate_arrivals(0, dur, seed))
        fast = gamma_arrivals_fast(rate, cv, 0, dur, seed)
        assert slow.shape == fast.shape and np.array_equal(slow, fast)
    # tiny blocks force the "draw another block" branch many times
    refills = 0
    for seed in range(40):
        slow = np.array(GammaProcess(0.011, 1).generate_arrivals(5.0, 95, seed))
        fast = gamma_arrivals_fast(0.011, 1, 5.0, 95, seed)
        assert np.array_equal(slow, fast)
        refills += len(slow) > 1          # block size is 1 here, so more than one arrival means a refill
    assert refills > 5


def test_workload_generation_statistics_and_merge():
    w = GammaProcess(10, 3).generate_workload("m", 0, 2000, slo=0.5, seed=1)
    assert abs(w.rate - 10) / 10 < 0.1 and abs(w.cv - 3) / 3 < 0.15
    assert np.all(np.diff(w.arrivals) >= 0) and [r.idx for r in w.requests] == list(range(len(w)))
    p = PoissonProcess(5).generate_workload("p", 0, 1000, seed=2)
    assert abs(p.cv - 1) < 0.1
    d = DeterministicProcess(4).generate_workload("d", 1.0, 10)
    assert len(d) == 40 and d.arrivals[0] == 1.0 and abs(d.arrivals[1] - 1.25) < 1e-12 and d.cv < 1e-9
    merged = w + p
    assert len(merged) == len(w) + len(p)
    assert np.all(np.diff(merged.arrivals) >= 0)
    assert [r.idx for r in merged.requests] == list(range(len(merged)))
    assert {r.model_name for r in merged.requests} == {"m", "p"}
    assert Workload.merge(w) is w
    parts = merged.split_time_interval(500)
    assert sum(len(x) for x in parts) == len(merged) and len(parts) in (4, 5)
    rr = merged.split_round_robin(3)
    assert [len(x) for x in rr] == [len(merged[i::3]) for i in range(3)]
    assert len(Workload.empty()) == 0 and Workload.empty().split_time_interval(1) == []
    with pytest.raises(NotImplementedError):
        merged[3]
    assert str(merged).startswith("Workload(len=")


def test_compute_stats_conventions():
    arrivals = np.arange(100, dtype=float)
    reqs = [Request("a" if i % 4 else "b", None, 1.0, i, {}) for i in range(100)]
    w = Workload(arrivals, reqs)
    good = np.ones(100, bool)
    good[::10] = False
    finish = arrivals + np.where(good, 0.5 + 0.001 * np.arange(100), 0.0)
    st = w.compute_stats(arrivals, finish, good, warmup=10)
    # skip = int(10/99*100) = 10 -> requests 10..89 are counted
    assert st.num_requests == 80
    assert [s.name for s in st.per_model_stats] == ["b", "a"]          # ascending request count
    a = st.per_model_stats[1]
    idx = np.array([i for i in range(10, 90) if i % 4])
    ok = good[idx]
    lat = (finish - arrivals)[idx][ok]
    assert a.num_requests == len(idx) and a.goodput == np.mean(ok)
    assert a.latency_p90 == np.sort(lat)[int(0.9 * len(lat))] and a.latency_p99 == np.sort(lat)[int(0.99 * len(lat))]
    assert st.goodput == np.mean(good[10:90]) and st.latency_mean == np.mean((finish - arrivals)[10:90])
    none_good = w.compute_stats(arrivals, arrivals.copy(), np.zeros(100, bool), warmup=10)
    assert all(s.goodput == 0 and s.throughput == 0 and s.latency_mean == 0 for s in none_good.per_model_stats)
    Workload.print_stats(st)


# ---- profiles ---------------------------------------------------------------------------------

def test_profiles():
    p = load_test_prof_result("alpa/bert-1.3b")
    assert p.para_dict[ParallelConfig(1, 1, 8)].latency[1][-1] == 0.016
    assert p.para_dict[ParallelConfig(1, 1, 2)].weight_mem == [1.3 * GB, 1.3 * GB]
    with pytest.raises(ValueError):
        load_test_prof_result("nope")
    r = ProfilingResult("x", {}, 0, 0)
    r.add_result(ParallelConfig(1, 1, 2), 1, [0.2, 0.3], [1, 1], [5, 5])
    r.add_result(ParallelConfig(1, 1, 2), 1, [0.25, 0.25], [2, 2], [6, 6], "better")    # smaller bottleneck wins
    r.add_result(ParallelConfig(1, 1, 2), 1, [0.1, 0.4], [3, 3], [7, 7])                # larger bottleneck ignored
    r.add_result(ParallelConfig(1, 1, 2), 2, [0.3, 0.3], [4, 4], [8, 8])
    e = r.para_dict[ParallelConfig(1, 1, 2)]
    assert e.latency == {1: [0.25, 0.25], 2: [0.3, 0.3]} and e.weight_mem == [6, 6] and e.metadata == "better"
    s = synthetic_profile("s", 0.2, [ParallelConfig(1, 2, 4), ParallelConfig(1, 1, 1)], (1, 2), 0.15, stage_comm=0.002)
    assert s.para_dict[ParallelConfig(1, 2, 4)].latency[2] == [0.2 * 1.15 / 4 * 1.05 + 0.002] * 4
    assert s.para_dict[ParallelConfig(1, 1, 1)].latency[1] == [0.2]


# ---- helpers (util.py) ------------------------------------------------------------------------

def test_partition_helpers():
    assert get_factors(12) == [1, 2, 3, 4, 6, 12] and get_factors(1) == [1] and get_factors(49) == [1, 7, 49]
    assert get2tok(34) == [1, 2, 4, 8, 16, 32] and get2tok(1) == [1]
    assert decompose2tok(13) == [1, 4, 8] and decompose2tok(0) == [] and decompose2tok(64) == [64]
    assert get_partitions(5, 1) == [[5]]
    assert get_partitions(4, 2) == [[3, 1], [2, 2], [1, 3]]
    for n, k in [(16, 3), (24, 3), (12, 4)]:
        parts = get_partitions(n, k)
        assert all(sum(p) == n and len(p) == k and min(p) >= 1 for p in parts)
        assert len({tuple(p) for p in parts}) == len(parts)
    # n = 12: a trailing part must be <= 12 % 8 or leave a multiple of 8
    assert [p[-1] for p in get_partitions(12, 2)] == [1, 2, 3, 4]
    assert is_valid_size(16, 5) and not is_valid_size(12, 5)
    assert to_str_round([1, 2.5, "x", None, {"a": 0.1234567}], 2) == "[1, 2.50, x, None, {'a': '0.12'}]"


def test_synthetic_configs_are_deterministic_and_as_specified():
    c1 = make_config(1)
    s = c1.stream(0)
    assert 1000 < len(s.tstamps) < 1500 and s.slos.dtype == np.float32 and np.all(s.slos == np.float32(0.5))
    assert c1.placements[0].group_configs == [ParallelConfig(1, 1, 4)] * 2
    c2a, c2b = make_config(2), make_config(2, 10)
    assert len(c2a.placements) == 64
    assert [p.group_models for p in c2a.placements[:10]] == [p.group_models for p in c2b.placements]
    for p in c2a.placements:
        assert sum(c.pp for c in p.group_configs) == 16 and all(2 <= len(ms) <= 6 for ms in p.group_models)
    assert np.array_equal(c2a.stream(3).tstamps, c2b.stream(3).tstamps)
    c3 = make_config(3, 130)
    assert c3.placements[0].group_models[0] == [0, 32, 1, 0] and len(c3.placements[129].group_configs) == 32
    assert abs(power_law_rates(64, 200.0, 0.5).sum() - 200.0) < 1e-9
    c4 = make_config(4, 8)
    for p in c4.placements:
        assert sum(c.op * c.pp for c in p.group_configs) == 64
        assert all(c.op in (1, 2, 4) and 8 <= len(ms) <= 24 for c, ms in zip(p.group_configs, p.group_models))
    c5 = make_config(5, 4)
    assert c5.batching and c5.batch_sizes == [1, 2, 4, 8] and set(np.round(c5.latencies, 2)) == {0.06, 0.12, 0.25, 0.5}
    w = c2a.workload(1)
    st = c2a.stream(1)
    assert np.array_equal(w.arrivals, st.tstamps)
    assert [r.model_name for r in w.requests] == [f"m{m}" for m in st.model_ids]


def test_alpa_serve_import_names_resolve_to_this_package():
    import importlib
    import sys
    import mms_amd.compat as compat
    compat.install()
    try:
        pp = importlib.import_module("alpa_serve.placement_policy")
        ctl = importlib.import_module("alpa_serve.simulator.controller")
        wl = importlib.import_module("alpa_serve.simulator.workload")
        for name in ("ModelData", "ClusterEnv", "ModelParallelismGreedy", "ModelParallelismSearch",
                     "SelectiveReplicationGreedy", "SelectiveReplicationSearch", "ModelParallelismILP"):
            assert hasattr(pp, name), name
        assert ctl.approximate_one_case.__module__ == "mms_amd.simulator.controller"
        assert wl.Workload.__module__ == "mms_amd.simulator.workload"
        from alpa_serve.placement_policy.base_policy import ModelPlacement, PlacementEvaluator  # noqa: F401
        from alpa_serve.profiling import ParallelConfig, ProfilingResult  # noqa: F401
        from alpa_serve.util import ServingCase, GB  # noqa: F401
    finally:
        for k in [k for k in sys.modules if k == "alpa_serve" or k.startswith("alpa_serve.")]:
            del sys.modules[k]


def test_add_model_normalized_is_add_model_then_normalize():
    """The greedy look-ahead builds its successor placements with add_model_normalized; it must give what
    add_model followed by normalize gives (base_policy.py:19-35 of the reference), ties between equal groups
    included, whether the placement it starts from is in canonical form or not."""
    import random
    from mms_amd.placement_policy.base_policy import ModelPlacement
    from mms_amd.profiling import ParallelConfig
    rnd = random.Random(5)
    for _ in range(1500):
        G = rnd.randint(1, 8)
        cfgs = [ParallelConfig(1, 1, rnd.choice([1, 2, 4])) for _ in range(G)]
        rows = [rnd.sample(range(10), rnd.randint(0, 4)) for _ in range(G)]
        sol = ModelPlacement(cfgs, rows)
        if rnd.random() < 0.7:
            sol = sol.normalize()
        g = rnd.randrange(G)
        m = rnd.choice([x for x in range(12) if x not in sol.group_models[g]])
        want = sol.add_model(g, m).normalize()
        got = sol.add_model_normalized(g, m)
        assert got == want
        assert type(got.group_models) is tuple and all(type(r) is tuple for r in got.group_models)
        assert got.add_model_normalized(0, 99) == got.add_model(0, 99).normalize()
