"""GPU parity of the plain (non-batching) simulator against the CPU oracle.

Everything goes through the C ABI of libmmsim (ctypes).  Bars: served/dropped
flags, all counts and finish times bit-exact (the tolerance the task states
for latencies is 1e-12 relative; the same fp64 operation sequence gives
identical bits, so identical bits are asserted).
"""
import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.synthetic import make_config
from oracle import oracle_c
from randcase import random_case
from helpers import assert_batch_matches, oracle_batch

pytestmark = pytest.mark.gpu

ALL = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS | _lib.WANT_PER_REQUEST | _lib.WANT_OP_COUNT


@pytest.fixture(scope="module")
def eng():
    return E.Engine.default()


def test_library_reports_the_device(eng):
    info = eng.device_info()
    print(info, flush=True)
    assert info["arch"].startswith("gfx950")
    assert info["compute_units"] >= 1


def test_single_placement_call_matches_oracle_on_random_cases(eng):
    for seed in range(300):
        c = random_case(seed, max_m=5, max_g=4, max_s=4, max_r=120)
        lat = c["lat"][..., 0]
        fin, good, cnt, _ = oracle_c.simulate_requests_mixed(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["num_stages"], lat)
        f2 = np.empty(c["R"])
        g2 = np.empty(c["R"], bool)
        cnt2 = E.simulate_requests_mixed(eng, f2, g2, c["tstamps"], c["model_ids"], c["slos"], c["m2g"],
                                         c["num_stages"], lat)
        assert np.array_equal(g2, good), seed
        assert np.array_equal(f2.view(np.uint64), fin.view(np.uint64)), seed
        for a, b in zip(cnt, cnt2):
            assert np.array_equal(a, b), seed


def test_single_placement_call_keeps_the_listing_order_of_replicas(eng):
    # m_id2g_id lists group 1 before group 0: ties must go to group 1
    lat = np.full((1, 2, 1), 0.1, np.float32)
    m2g = np.array([[1, 0]], np.int32)
    f, g = np.empty(3), np.empty(3, bool)
    cnt = E.simulate_requests_mixed(eng, f, g, np.zeros(3), np.zeros(3, np.int32),
                                    np.full(3, np.inf, np.float32), m2g, np.array([1, 1], np.int32), lat)
    assert cnt[2].tolist() == [1, 2]


def _run_config(eng, cfg, sols, seeds, flags):
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(sols, table)
    streams = [cfg.stream(s) for s in seeds]
    dws = [E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models) for st in streams]
    batch = E.Batch(eng, dws, table, packed, flags)
    batch.run()
    batch.sync()
    out = batch.fetch()
    info = batch.info()
    batch.close()
    return out, table, packed, streams, info


def test_scalar_clock_variant_matches_oracle(eng):
    """simulate_requests (alpa_serve/simulator/controller.py:506-558), the mixed=False loop: finish bits,
    flags and all four count arrays against the oracle; closed form for a single group."""
    F32 = np.float32
    gsum, gmax = np.full((1, 1), 0.3, F32), np.full((1, 1), 0.1, F32)
    R = 10
    fin, good = np.empty(R), np.empty(R, bool)
    E.simulate_requests(eng, fin, good, np.zeros(R), np.zeros(R, np.int32), np.full(R, np.inf, F32),
                        np.zeros((1, 1), np.int32), gmax, gsum)
    start, want = 0.0, []
    for _ in range(R):                       # the next request may start 0.1 after the previous start
        want.append(start + float(F32(0.3)) + 0.011)
        start = start + float(F32(0.1))
    assert fin.tolist() == want and good.all()
    for seed in range(300):
        c = random_case(5_000_000 + seed, max_m=6, max_g=5, max_s=4, max_r=300, load=1.0 + seed % 5)
        gmax = c["lat"][..., 0].max(axis=2)
        gsum = c["lat"][..., 0].sum(axis=2, dtype=np.float32)
        f0, g0, c0 = oracle_c.simulate_requests(c["tstamps"], c["model_ids"], c["slos"], c["m2g"], gmax, gsum)
        R = len(c["tstamps"])
        fin, good = np.empty(R), np.empty(R, bool)
        cnt = E.simulate_requests(eng, fin, good, c["tstamps"], c["model_ids"], c["slos"], c["m2g"], gmax, gsum)
        assert np.array_equal(good, g0), seed
        assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64)), seed
        for a, b in zip(cnt, c0):
            assert np.array_equal(a, b), seed


def test_config1_sanity_case(eng):
    cfg = make_config(1)
    out, table, packed, streams, _ = _run_config(eng, cfg, cfg.placements, [0], ALL)
    ref = oracle_batch(streams[0], table, packed, want_per_request=True)
    assert_batch_matches(out, ref, 0, packed[0], per_request=True, where="cfg1")
    assert out["fp_ops"][0, 0] == ref["fp_ops"]
    assert 0 < ref["n_good"][0] <= len(streams[0].tstamps)


def test_config2_all_placements_all_seeds_per_request(eng):
    cfg = make_config(2)
    out, table, packed, streams, info = _run_config(eng, cfg, cfg.placements, cfg.base_seeds, ALL)
    assert info["lanes"] == 256
    total_ops = 0
    for s, st in enumerate(streams):
        ref = oracle_batch(st, table, packed, want_per_request=True)
        assert_batch_matches(out, ref, s, packed[0], per_request=True, where=f"cfg2 seed {s}")
        total_ops += ref["fp_ops"]
    assert out["fp_ops"].sum() == total_ops


def test_config2_ragged_batch_sizes(eng):
    # batch sizes that do not fill a wavefront, and one that spills into a second tile
    cfg = make_config(2, 70)
    for n in (1, 3, 63, 65, 70):
        out, table, packed, streams, _ = _run_config(eng, cfg, cfg.placements[:n], [1], ALL)
        ref = oracle_batch(streams[0], table, packed, want_per_request=True)
        assert_batch_matches(out, ref, 0, packed[0], per_request=True, where=f"cfg2 B={n}")


@pytest.mark.parametrize("flags", [0, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS])
def test_config3_every_candidate_of_the_greedy_step(eng, flags):
    """All 4096 candidates of configuration 3 (both base placements, every (group, model) move) against
    the oracle: goodput and latency sums, and with counts every per-model and per-group counter."""
    cfg = make_config(3)
    assert len(cfg.placements) == 4096
    out, table, packed, streams, info = _run_config(eng, cfg, cfg.placements, [0], flags)
    assert info["lanes"] == 4096
    ref = oracle_batch(streams[0], table, packed)
    assert_batch_matches(out, ref, 0, packed[0], where="cfg3")


def test_config4_subsample_counts_and_a_few_full_traces(eng):
    cfg = make_config(4, 96)
    out, table, packed, streams, info = _run_config(
        eng, cfg, cfg.placements, [0], _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS | _lib.WANT_OP_COUNT)
    print(info, flush=True)
    ref = oracle_batch(streams[0], table, packed)
    assert_batch_matches(out, ref, 0, packed[0], where="cfg4")
    assert out["fp_ops"].sum() == ref["fp_ops"]
    # full per-request traces (1M requests each) for 4 placements
    out, table, packed, streams, _ = _run_config(eng, cfg, cfg.placements[:4], [0], ALL)
    ref = oracle_batch(streams[0], table, packed, want_per_request=True)
    assert_batch_matches(out, ref, 0, packed[0], per_request=True, where="cfg4 traces")
    # traces and model counts without group / operation counts, a full wavefront of placements
    some_flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_PER_REQUEST
    out, table, packed, streams, _ = _run_config(eng, cfg, cfg.placements[:64], [0], some_flags)
    ref = oracle_batch(streams[0], table, packed, want_per_request=True)
    assert_batch_matches(out, ref, 0, packed[0], per_request=True, where="cfg4 traces, 64 placements")
    assert (~ref["good"]).all(axis=0).mean() > 0.2      # many requests are rejected by all 64 placements


def test_config4_every_seed_against_the_oracle(eng):
    """The headline batch runs eight arrival seeds; here 64 placements spread over the candidate list are
    compared with the oracle on every one of them at full stream length (8 x 64 x ~1M evaluations), at the
    scores level (the kernel the benchmark times) and at the counts level."""
    from concurrent.futures import ThreadPoolExecutor
    cfg = make_config(4)
    assert len(cfg.base_seeds) == 8
    sols = cfg.placements[37::256][:64]
    assert len(sols) == 64
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(sols, table)
    streams = [cfg.stream(s) for s in cfg.base_seeds]
    dws = [E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models) for st in streams]
    with ThreadPoolExecutor(8) as pool:             # the oracle call releases the GIL
        refs = list(pool.map(lambda st: oracle_batch(st, table, packed), streams))
    for flags in (0, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS):
        batch = E.Batch(eng, dws, table, packed, flags)
        batch.run()
        batch.sync()
        out = batch.fetch()
        name = batch.kernel_name()
        batch.close()
        assert name.endswith("true>"), name         # the loop over runs, as in the benchmark
        for s, ref in enumerate(refs):
            assert_batch_matches(out, ref, s, packed[0], where=f"cfg4 seed {cfg.base_seeds[s]}, flags {flags}")
    assert len({int(r["n_good"].sum()) for r in refs}) == 8      # the seeds are different streams
    for dw in dws:
        dw.close()


@pytest.mark.parametrize("depths", [(1, 2, 4), (1, 2, 4, 8, 16), (1, 2, 3, 4), (1, 3, 5, 8, 11, 16)])
@pytest.mark.parametrize("uniform", [True, False])
def test_stage_walk_variants(eng, depths, uniform):
    """Every hand-scheduled stage walk: depths that are all powers of two or not,
    one latency per configuration or one per stage, 4- and 16-stage buckets;
    130 placements of mixed depth so that lanes leave the walk at different levels."""
    from types import SimpleNamespace
    from mms_amd.profiling import LatencyMemData, ParallelConfig, ProfilingResult
    from mms_amd.placement_policy.base_policy import ModelPlacement
    rng = np.random.default_rng(1000 * len(depths) + 2 * sum(depths) + int(uniform))
    M, R = 12, 4000
    pcs = [ParallelConfig(1, 1, d) for d in depths]
    profiles = []
    for m in range(M):
        para = {}
        for pc in pcs:
            total = rng.uniform(0.05, 0.3)
            stages = np.full(pc.pp, total / pc.pp) if uniform else rng.dirichlet(np.ones(pc.pp)) * total
            para[pc] = LatencyMemData(latency={1: [float(x) for x in stages]}, act_mem={1: [0.0] * pc.pp},
                                      weight_mem=[1.0] * pc.pp)
        profiles.append(ProfilingResult(f"m{m}", para_dict=para, preprocess_cpu=0, postprocess_cpu=0))
    sols = []
    for _ in range(130):
        left, cfgs, models = 40, [], []
        while left > 0:
            d = int(rng.choice([x for x in depths if x <= left]))
            left -= d
            cfgs.append(ParallelConfig(1, 1, d))
            models.append([int(x) for x in rng.choice(M, size=int(rng.integers(1, 6)), replace=False)])
        sols.append(ModelPlacement(cfgs, models))
    gaps = rng.exponential(0.02, size=R)
    gaps[rng.random(R) < 0.1] = 0.0
    st = SimpleNamespace(tstamps=np.cumsum(gaps), model_ids=rng.integers(0, M, R).astype(np.int32),
                         slos=rng.uniform(0.2, 1.0, R).astype(np.float32))
    table = E.LatencyTable(profiles, [1])
    packed = E.pack_placements(sols, table)
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, M)
    batch = E.Batch(eng, [dw], table, packed, ALL)
    batch.run()
    batch.sync()
    out = batch.fetch()
    assert batch.info()["smax_bucket"] == (4 if max(depths) <= 4 else 16)
    batch.close()
    ref = oracle_batch(st, table, packed, want_per_request=True)
    assert_batch_matches(out, ref, 0, packed[0], per_request=True, where=f"depths {depths} uniform {uniform}")
    assert 0.05 * R * 130 < ref["n_good"].sum() < 0.98 * R * 130    # both accepts and rejects are exercised


COUNTS_IN_REGISTERS = -1    # per-model and per-group counts, the latter in registers with adds to global rows


COUNTS_IN_LDS = -2          # the same counts, per-group counters in LDS


@pytest.mark.parametrize("flags", [0, COUNTS_IN_REGISTERS, COUNTS_IN_LDS, ALL])
@pytest.mark.parametrize("groups,regions,segment,spin", [(1, 1, 64, None), (3, 2, 256, None), (5, 8, 512, None),
                                                        (64, 8, 16384, None), (1, 8, 64, 0), (2, 5, 128, 1),
                                                        (2, 8, 512, None)])
def test_scheduled_launch_with_items_taking_turns(eng, opts, flags, groups, regions, segment, spin):
    """The loop over runs is launched as a schedule: a workgroup owns several (tile, stream) items, its
    LDS is cut into regions sized by the items' clock slots, and its wavefronts simulate the items a
    segment at a time, clocks parked in device memory in between.  Forced here on a small batch with
    few workgroups, few regions and short segments: 420 placements using 4..56 devices (7 tiles of
    different sizes x 2 streams of odd, unequal lengths), every output level.  With ``spin`` 0 or 1 a
    wavefront that finds all the items it could take in other wavefronts' hands leaves at once instead
    of waiting (normally it would look again for about 70 ms): the holders then finish the items alone,
    and every item must still be completed.  Two workgroups with eight regions give each of the seven items of a
    workgroup a wavefront of its own for the whole stream (one segment), large items sharing a SIMD with small ones."""
    from types import SimpleNamespace
    from mms_amd.profiling import ParallelConfig
    from mms_amd.placement_policy.base_policy import ModelPlacement
    from mms_amd.profiling import synthetic_profile
    opts(request_loop=1)
    opts(sched_groups=groups)
    opts(waves_per_cu=regions)
    opts(segment_requests=segment)
    if spin is not None:
        opts(sched_spin_limit=spin)
    if flags in (COUNTS_IN_REGISTERS, COUNTS_IN_LDS):
        opts(counts_in_lds=0 if flags == COUNTS_IN_REGISTERS else 1)
        flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    traces = bool(flags & _lib.WANT_PER_REQUEST)
    rng = np.random.default_rng(77)
    M, R = 24, 3001
    pcs = [ParallelConfig(1, 1, d) for d in (1, 2, 4, 8)]
    profiles = [synthetic_profile(f"m{m}", float(rng.uniform(0.05, 0.3)), pcs) for m in range(M)]
    sols = []
    for i in range(420):
        left, cfgs, models = int(rng.choice([4, 8, 12, 20, 28, 36, 44, 56])), [], []
        while left > 0:
            d = int(rng.choice([x for x in (1, 2, 4, 8) if x <= left]))
            left -= d
            cfgs.append(ParallelConfig(1, 1, d))
            models.append([int(x) for x in rng.choice(M, size=int(rng.integers(1, 6)), replace=False)])
        sols.append(ModelPlacement(cfgs, models))
    streams = []
    for seed in range(2):
        gaps = rng.exponential(0.01, size=R + seed * 70)
        ids = np.repeat(rng.integers(-1, M, len(gaps)), rng.integers(1, 9, len(gaps)))[:len(gaps)]   # bursts of 1..8
        streams.append(SimpleNamespace(tstamps=np.cumsum(gaps), model_ids=ids.astype(np.int32),
                                       slos=rng.uniform(0.2, 1.0, len(gaps)).astype(np.float32)))
    table = E.LatencyTable(profiles, [1])
    packed = E.pack_placements(sols, table)
    dws = [E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, M) for st in streams]
    batch = E.Batch(eng, dws, table, packed, flags)
    info = batch.info()
    print(info, flush=True)
    assert info["workgroups"] == min(groups, 14) and info["waves_per_group"] <= regions and info["launches"] == 1
    assert info["segments"] == (-(-(R + 70) // segment) if 14 > info["workgroups"] * info["waves_per_group"] else 1)
    for _ in range(2):                      # a re-run starts from scratch again
        batch.run()
        batch.sync()
    out = batch.fetch()
    batch.close()
    for s, st in enumerate(streams):
        ref = oracle_batch(st, table, packed, want_per_request=traces)
        assert_batch_matches(out, ref, s, packed[0], per_request=traces, where=f"seed {s}")
        if traces:
            assert out["fp_ops"][s].sum() == ref["fp_ops"]


@pytest.mark.parametrize("mode", ["chunks", "runs", "batching"])
def test_paired_placements_and_streams(eng, opts, mode):
    """mmsim_eval_pairs simulates placement b on stream stream_of[b] only (the segments of placements that
    replace one another).  Every result must equal the [stream][placement] entry of the full cross product
    that mmsim_eval_batch computes: 150 placements over 3 streams of different lengths, tiles ragged at the
    stream boundaries, both request loops of the plain simulator and the batching simulator."""
    cfg = make_config(5 if mode == "batching" else 2, 150)
    if mode != "batching":
        opts(request_loop=1 if mode == "runs" else 0)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(cfg.placements, table)
    lens = (2500, 1700, 3001)
    streams = [cfg.stream(s) for s in cfg.base_seeds[:3]]
    dws = [E.DeviceWorkload(eng, st.tstamps[:n], st.model_ids[:n], st.slos[:n], cfg.num_models)
           for st, n in zip(streams, lens)]
    stream_of = np.random.default_rng(3).integers(0, 3, len(cfg.placements)).astype(np.int32)
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS | _lib.WANT_PER_REQUEST
    if mode == "batching":
        flags |= _lib.BATCHING
    full = E.eval_batch(eng, dws, table, packed, flags)
    for fl in (flags, flags & ~_lib.WANT_PER_REQUEST, flags & _lib.BATCHING):
        got = E.eval_pairs(eng, dws, table, packed, stream_of, fl)
        for b, sidx in enumerate(stream_of):
            for k in got:
                if k == "status":
                    continue
                want = full[k][sidx, b]
                if k in ("finish", "good"):
                    assert np.array_equal(got[k][b][:lens[sidx]], want[:lens[sidx]]), (k, b)
                else:
                    assert np.array_equal(got[k][b], want), (k, b)


@pytest.mark.parametrize("config", [2, 5])
@pytest.mark.parametrize("normalize", [True, False])
def test_successors_built_by_the_library(eng, config, normalize):
    """mmsim_eval_successors builds "placement + one more replica" candidates itself; every output must equal
    what the same candidates give when they are built as Python objects (add_model / normalize) and sent through
    mmsim_eval_batch -- including the order of the per-group counts, which is the order normalize() puts the
    groups in.  Bases: placements as generated (rows unsorted, groups in no particular order), placements with
    empty groups, and normalized ones; both simulators."""
    from mms_amd.placement_policy.base_policy import ModelPlacement
    cfg = make_config(config, 40)
    rng = np.random.default_rng(11 + config)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    bases = list(cfg.placements[:30]) + [p.normalize() for p in cfg.placements[30:40]]
    emptied = cfg.placements[3]
    bases.append(ModelPlacement(list(emptied.group_configs), [[] for _ in emptied.group_models]))
    parent, group, model = [], [], []
    for b, sol in enumerate(bases):
        for _ in range(5):
            g = int(rng.integers(len(sol.group_configs)))
            free = [m for m in range(cfg.num_models) if m not in sol.group_models[g]]
            parent.append(b)
            group.append(g)
            model.append(int(rng.choice(free)))
    kids = [bases[p].add_model(g, m) for p, g, m in zip(parent, group, model)]
    if normalize:
        kids = [k.normalize() for k in kids]
    st = cfg.stream(cfg.base_seeds[0])
    n = 6000
    dw = E.DeviceWorkload(eng, st.tstamps[:n], st.model_ids[:n], st.slos[:n], cfg.num_models)
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS | (_lib.BATCHING if cfg.batching else 0)
    want = E.evaluate(eng, [dw], table, bases + kids, flags)
    got = E.evaluate_successors(eng, [dw], table, bases, parent, group, model, flags, normalize=normalize)
    for k in ("n_good", "latency_sum", "model_num_requests", "model_num_good", "group_num_requests", "group_num_good"):
        assert np.array_equal(got[k], want[k]), k
    assert len({tuple(r) for r in want["group_num_requests"][0].tolist()}) > len(bases)     # the counts tell groups apart
    # nothing to add: the bases alone
    alone = E.evaluate_successors(eng, [dw], table, bases, [], [], [], flags)
    assert np.array_equal(alone["n_good"][0], want["n_good"][0][:len(bases)])
    for bad in (([len(bases)], [0], [0]), ([0], [99], [0]), ([0], [0], [cfg.num_models])):
        with pytest.raises(_lib.MmsimError) as err:
            E.evaluate_successors(eng, [dw], table, bases, *bad, flags)
        assert err.value.code == _lib.E_INVALID
    dw.close()


def test_eight_wavefronts_per_workgroup(eng, opts):
    """Large batches of small placements run 8 wavefronts per workgroup (two per SIMD); forced here on
    520 placements of configuration 2 (16 clock slots)."""
    opts(waves_per_cu=8)
    cfg = make_config(2, 520)
    for flags in (0, ALL):
        out, table, packed, streams, info = _run_config(eng, cfg, cfg.placements, [0, 3], flags)
        assert info["waves"] == 18
        for s, st in enumerate(streams):
            ref = oracle_batch(st, table, packed, want_per_request=bool(flags))
            assert_batch_matches(out, ref, s, packed[0], per_request=bool(flags), where=f"8 waves, seed {s}")


def test_scores_only_mode_equals_full_mode(eng):
    cfg = make_config(2)
    a, *_ = _run_config(eng, cfg, cfg.placements, [0, 1], 0)
    b, *_ = _run_config(eng, cfg, cfg.placements, [0, 1], ALL)
    assert np.array_equal(a["n_good"], b["n_good"])
    assert np.array_equal(a["latency_sum"], b["latency_sum"])


@pytest.mark.parametrize("n_placements", [200, 640])
def test_scores_only_on_bursty_streams_matches_oracle(eng, opts, n_placements):
    """A scores-only run keeps the chosen group from request to request while no lane accepts, and does
    not simulate requests that every lane of a wavefront must reject.  Configuration 4's bursts (nine in
    ten requests repeat the model of the one before) exercise both: goodput and latency sums equal the
    oracle's bit for bit, in full and ragged tiles, with the skipping and without it."""
    cfg = make_config(4, n_placements)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(cfg.placements, table)
    st = cfg.stream(0)
    assert np.mean(st.model_ids[1:] == st.model_ids[:-1]) > 0.8
    ref = oracle_batch(st, table, packed)
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models)
    for runs, skip in (("1", "1"), ("1", "0"), ("0", "1")):   # loop over runs (with / without skipping), chunked loop
        opts(request_loop=int(runs))
        opts(skip_ahead=int(skip))
        batch = E.Batch(eng, [dw], table, packed, 0)
        batch.run()
        batch.sync()
        out = batch.fetch()
        batch.close()
        assert np.array_equal(out["n_good"][0], ref["n_good"]), f"n_good differs (runs {runs}, skip {skip})"
        assert np.array_equal(out["latency_sum"][0], ref["latency_sum"]), f"latency_sum differs (runs {runs}, skip {skip})"
    # per-model and per-group counts: requests that are not simulated still count for the group they would have chosen
    # (group counters in LDS, or in registers with adds to global rows when a lane's group changes)
    for runs, lds in (("1", "1"), ("1", "0"), ("0", "0")):
        opts(request_loop=int(runs))
        opts(counts_in_lds=int(lds))
        batch = E.Batch(eng, [dw], table, packed, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS)
        for _ in range(2):      # a second run starts from zeroed counters again
            batch.run()
            batch.sync()
        out = batch.fetch()
        batch.close()
        assert_batch_matches(out, ref, 0, packed[0], where=f"counts, runs {runs}, group counters in LDS {lds}")
    dw.close()


@pytest.mark.parametrize("loop", ["runs", "chunks"])
@pytest.mark.parametrize("flags", [0, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS, _lib.WANT_GROUP_COUNTS + 1000, ALL])
def test_runs_of_one_model_with_odd_requests(eng, opts, loop, flags):
    """Runs of equal models with tied arrival times, SLOs that change inside a run (also inf and NaN),
    unknown models, streams that end inside a block of 64, several seeds: results equal the oracle's for
    every placement of configuration 2, with either request loop, scores only and with every output."""
    opts(request_loop=1 if loop == "runs" else 0)
    if flags >= 1000:       # per-group counts alone, kept in registers and added to global rows
        flags -= 1000
        opts(counts_in_lds=0)
    cfg = make_config(2)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(cfg.placements, table)
    base_slo = np.asarray(cfg.slos, np.float32)
    M = cfg.num_models
    streams = []
    for seed, R in enumerate([1, 63, 64, 65, 5000, 20011]):
        rng = np.random.default_rng(100 + seed)
        runs = rng.geometric(0.12, size=R)
        models = np.repeat(rng.integers(0, M, size=R), runs)[:R].astype(np.int32)
        models[rng.random(R) < 0.02] = -1
        gaps = rng.exponential(0.004, size=R)
        gaps[rng.random(R) < 0.25] = 0.0
        gaps[rng.random(R) < 0.01] += 2.0                      # pauses that let the queues drain
        ts = np.cumsum(gaps)
        slos = base_slo[np.maximum(models, 0)] * rng.choice([1.0, 1.0, 1.0, 0.5, 3.0], size=R).astype(np.float32)
        slos[rng.random(R) < 0.01] = np.inf
        slos[rng.random(R) < 0.01] = np.nan
        streams.append((ts, models, slos.astype(np.float32)))
    dws = [E.DeviceWorkload(eng, t, m, s, M) for t, m, s in streams]
    batch = E.Batch(eng, dws, table, packed, flags)
    batch.run()
    batch.sync()
    out = batch.fetch()
    batch.close()
    from mms_amd.synthetic import Stream
    for k, (t, m, s) in enumerate(streams):
        traces = bool(flags & _lib.WANT_PER_REQUEST)
        ref = oracle_batch(Stream(t, m, s), table, packed, want_per_request=traces)
        assert_batch_matches(out, ref, k, packed[0], per_request=traces, where=f"stream {k}, {loop}")
        assert 0 < ref["n_good"].sum() < len(t) * len(cfg.placements) or len(t) < 64


@pytest.mark.parametrize("n_configs", [12, 63, 70])
@pytest.mark.parametrize("flags", [0, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS, ALL])
def test_loop_over_runs_with_many_configurations_and_unhosted_models(eng, opts, n_configs, flags):
    """With one latency per (model, configuration) and outputs beyond the scores, the loop over runs keeps a model's row
    of the latency table in a register, one entry per lane, and gathers the latencies of a run's listed replicas from
    it: rows of 13 and of 64 entries (the most that fit) take that path, 71 entries send the batch to the chunked loop
    although the loop over runs is asked for.  Models with up to six replicas (more than the four of the usual scan),
    models that no placement of a tile hosts (their runs are passed over) and unknown models are in the stream."""
    from types import SimpleNamespace
    from mms_amd.profiling import ParallelConfig, synthetic_profile
    from mms_amd.placement_policy.base_policy import ModelPlacement
    opts(request_loop=1)
    rng = np.random.default_rng(7000 + n_configs)
    M, R, B = 10, 6000, 130
    pcs = [ParallelConfig(1 + k // 16, 1 + (k // 4) % 4, (1, 2, 4, 8)[k % 4]) for k in range(n_configs)]
    assert len(set(pcs)) == n_configs
    profiles = [synthetic_profile(f"m{m}", float(rng.uniform(0.05, 0.3)), pcs) for m in range(M)]
    sols = []
    for _ in range(B):
        cfgs, models = [], []
        for _g in range(int(rng.integers(3, 9))):
            cfgs.append(pcs[int(rng.integers(0, n_configs))])
            # models 0-1 are everywhere (up to eight replicas), 2-7 here and there, 8-9 hosted by nobody
            models.append([0, 1][: int(rng.integers(0, 3))] + [int(x) for x in rng.choice(np.arange(2, 8), size=int(rng.integers(0, 3)), replace=False)])
        sols.append(ModelPlacement(cfgs, models))
    runs = rng.geometric(0.1, size=R)
    model_ids = np.repeat(rng.integers(0, M, size=R), runs)[:R].astype(np.int32)
    model_ids[rng.random(R) < 0.01] = -1
    gaps = rng.exponential(0.01, size=R)
    gaps[rng.random(R) < 0.2] = 0.0
    st = SimpleNamespace(tstamps=np.cumsum(gaps), model_ids=model_ids, slos=rng.uniform(0.2, 1.5, R).astype(np.float32))
    table = E.LatencyTable(profiles, [1])
    packed = E.pack_placements(sols, table)
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, M)
    batch = E.Batch(eng, [dw], table, packed, flags)
    batch.run()
    batch.sync()
    out = batch.fetch()
    name = batch.kernel_name()
    assert batch.info()["max_replicas"] > 4
    batch.close()
    assert name.endswith(", true>") == (n_configs < 64), name       # the last template argument: loop over runs
    traces = bool(flags & _lib.WANT_PER_REQUEST)
    ref = oracle_batch(st, table, packed, want_per_request=traces)
    assert_batch_matches(out, ref, 0, packed[0], per_request=traces, where=f"{n_configs} configurations, flags {flags}")
    assert 0.02 * R * B < ref["n_good"].sum() < 0.9 * R * B


def test_rerunning_a_batch_gives_the_same_answer(eng):
    cfg = make_config(2)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(cfg.placements, table)
    st = cfg.stream(0)
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models)
    batch = E.Batch(eng, [dw], table, packed, _lib.WANT_MODEL_COUNTS)
    res = []
    for _ in range(3):
        batch.run()
        batch.sync()
        res.append(batch.fetch())
    for r in res[1:]:
        assert np.array_equal(r["n_good"], res[0]["n_good"])
        assert np.array_equal(r["model_num_good"], res[0]["model_num_good"])


def test_edge_inputs(eng):
    cfg = make_config(2, 8)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(cfg.placements, table)
    # empty stream
    dw = E.DeviceWorkload(eng, np.zeros(0), np.zeros(0, np.int32), np.zeros(0, np.float32), cfg.num_models)
    out = E.evaluate(eng, [dw], table, cfg.placements, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS)
    assert out["n_good"].sum() == 0 and out["model_num_requests"].sum() == 0
    # unknown models, NaN / inf SLOs, a placement with an empty group and one with no model at all
    from mms_amd.placement_policy.base_policy import ModelPlacement
    from mms_amd.profiling import ParallelConfig
    st = cfg.stream(0)
    mids = st.model_ids.copy()
    mids[::7] = -1
    slos = st.slos.copy()
    slos[::11] = np.nan
    slos[::13] = np.inf
    sols = list(cfg.placements) + [ModelPlacement([ParallelConfig(1, 1, 2), ParallelConfig(1, 1, 1)], [[], [3, 4]]),
                                   ModelPlacement([ParallelConfig(1, 1, 4)], [[]])]
    packed = E.pack_placements(sols, table)
    dw = E.DeviceWorkload(eng, st.tstamps, mids, slos, cfg.num_models)
    batch = E.Batch(eng, [dw], table, packed, ALL)
    batch.run(); batch.sync()
    out = batch.fetch()
    batch.close()
    from mms_amd.synthetic import Stream
    ref = oracle_batch(Stream(st.tstamps, mids, slos), table, packed, want_per_request=True)
    assert_batch_matches(out, ref, 0, packed[0], per_request=True, where="edge")


def test_error_codes(eng):
    cfg = make_config(2, 4)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    st = cfg.stream(0)
    with pytest.raises(_lib.MmsimError) as e:
        E.DeviceWorkload(eng, st.tstamps, st.model_ids + 1000, st.slos, cfg.num_models)
    assert e.value.code == _lib.E_INVALID
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models)
    num_groups, group_cfg, gm_off, gm_idx = E.pack_placements(cfg.placements, table)
    bad = gm_idx.copy()
    bad[0] = cfg.num_models + 5
    with pytest.raises(_lib.MmsimError) as e:
        E.Batch(eng, [dw], table, (num_groups, group_cfg, gm_off, bad), 0)
    assert e.value.code == _lib.E_INVALID
    bad_cfg = group_cfg.copy()
    bad_cfg[0, 0] = 99
    with pytest.raises(_lib.MmsimError) as e:
        E.Batch(eng, [dw], table, (num_groups, bad_cfg, gm_off, gm_idx), 0)
    assert e.value.code == _lib.E_INVALID
    with pytest.raises(_lib.MmsimError) as e:
        E.Engine(device=99)
    assert e.value.code == _lib.E_INVALID
