"""GPU parity of the statistics kernel (mmsim_batch_model_stats) with
Workload.compute_stats' conventions (workload.py:308-354).

The kernel (one workgroup per simulation and model) reduces the per-request
outputs that the simulation kernels left in device memory; the check fetches those same outputs and reduces them with
numpy (``model_stats_numpy``: sort, ``sorted[int(q * n)]``, ``np.mean``,
``np.std``).  Bars: counts, first / last accepted arrival and both percentiles
bit-exact; sum and mean within 1e-12 relative, the deviation within 1e-12 of
itself plus 1e-12 of the mean (compensated sums on the device, pairwise sums in
numpy).
"""
import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.synthetic import make_config
from oracle_backend import model_stats_numpy

pytestmark = pytest.mark.gpu

EXACT = ("model_num_requests", "model_num_good", "first_start", "last_start", "latency_p90", "latency_p99")
CLOSE = ("latency_sum", "latency_mean", "latency_std")


@pytest.fixture(scope="module")
def eng():
    return E.Engine.default()


def _check(eng, cfg, sols, seeds, skips, flags=0):
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    streams = [cfg.stream(s) for s in seeds]
    dws = [E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models) for st in streams]
    batch = E.Batch(eng, dws, table, E.pack_placements(sols, table), flags | _lib.WANT_PER_REQUEST)
    batch.run()
    batch.sync()
    out = batch.fetch()
    for skip in skips:
        got = batch.model_stats(skip)
        for s, st in enumerate(streams):
            for b in range(len(sols)):
                R = len(st.tstamps)
                want = model_stats_numpy(st.tstamps, st.model_ids, out["finish"][s, b, :R], out["good"][s, b, :R],
                                         skip[s], cfg.num_models)
                for k in EXACT:
                    assert np.array_equal(got[k][s, b], want[k]), (k, s, b, skip)
                for k in CLOSE:
                    # (a deviation far below the mean is the difference of nearly equal numbers on both sides:
                    # it is held to 1e-12 of the mean, not of itself)
                    atol = 1e-12 * np.abs(want["latency_mean"]) if k == "latency_std" else 1e-300
                    assert np.all(np.abs(got[k][s, b] - want[k]) <= 1e-12 * np.abs(want[k]) + atol), (k, s, b, skip)
    batch.close()
    return out


def test_plain_simulator_two_streams_every_window(eng):
    cfg = make_config(2, 64)
    R = min(len(cfg.stream(s).tstamps) for s in (0, 1))
    out = _check(eng, cfg, cfg.placements, (0, 1),
                 [(0, 0), (1, 7), (R // 10, R // 7), (R // 2 - 1, R // 2 - 1), (R // 2 + 5, R), (3 * R, 0)])
    assert 0 < out["good"].mean() < 1       # both accepted and rejected requests took part


def test_more_simulations_than_scratch_rows_take_several_launches(eng, opts):
    cfg = make_config(2, 11)
    R = len(cfg.stream(0).tstamps)
    opts(stats_scratch_bytes=3 * 8 * R + 100)   # three simulations per launch, 22 in all
    _check(eng, cfg, cfg.placements, (0, 1), [(0, 0), (R // 9, R // 8)])


def test_more_placements_than_one_wavefront_and_deep_pipelines(eng):
    cfg = make_config(4, 96)
    cfg.duration *= 0.02        # about 20000 requests
    R = len(cfg.stream(3).tstamps)
    _check(eng, cfg, cfg.placements, (3,), [(0,), (R // 20,)])


def test_batching_simulator(eng):
    cfg = make_config(5, 24)
    cfg.duration *= 0.05
    R = len(cfg.stream(0).tstamps)
    _check(eng, cfg, cfg.placements, (0,), [(0,), (R // 9,)], flags=_lib.BATCHING)


def test_statistics_of_a_batching_run_that_needs_more_event_slots(eng, opts):
    """device_compute_stats (approximate_one_case without fast_stats) takes the statistics from what the run left on
    the device; a simulation that runs out of idle-event slots (forced here: eight slots) makes it run the batch
    again with twice the slots until every simulation fits.  The result is that of a run with the default slots."""
    import types
    from mms_amd.simulator import controller as sim
    cfg = make_config(5, 6)
    cfg.duration *= 0.05
    st = cfg.stream(0)
    wl = types.SimpleNamespace(arrivals=st.tstamps, requests=None)
    names = [f"m{i}" for i in range(cfg.num_models)]
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)

    def stats():
        return sim.device_compute_stats(wl, cfg.placements, names, cfg.profiles, st.model_ids, st.slos, 10,
                                        enable_batching=True, table=table)
    want = stats()
    opts(batching_event_slots=8)
    got = stats()
    assert len(got) == len(want) == 6
    for g, w in zip(got, want):
        assert g.goodput == w.goodput and g.latency_mean == w.latency_mean and g.num_requests == w.num_requests
        assert list(g.group_num_requests) == list(w.group_num_requests)
        for pg, pw in zip(g.per_model_stats, w.per_model_stats):
            assert (pg.name, pg.num_requests, pg.goodput, pg.latency_p99) == (pw.name, pw.num_requests, pw.goodput, pw.latency_p99)


@pytest.mark.parametrize("config, placements, seeds, shrink, flags", [
    (2, 5, (0, 1), 1.0, 0), (4, 1, (2,), 0.05, 0), (4, 16, (1,), 0.02, 0), (5, 3, (0,), 0.05, _lib.BATCHING)],
    ids=["cfg2-5x2", "cfg4-1", "cfg4-16", "cfg5-3-batching"])
def test_a_handful_of_simulations(eng, config, placements, seeds, shrink, flags):
    """One placement on one stream is what approximate_one_case(fast_stats=False) sends."""
    cfg = make_config(config, placements)
    cfg.duration *= shrink
    R = min(len(cfg.stream(s).tstamps) for s in seeds)
    _check(eng, cfg, cfg.placements, seeds, [tuple(0 for _ in seeds), tuple(R // 11 for _ in seeds),
                                             tuple(R // 2 + 3 for _ in seeds)], flags=flags)


def test_equal_latencies_by_the_thousand_and_few_distinct_ones(eng):
    """The selection ranks the last candidates directly once at most 1024 still match the digits fixed so far.  An idle
    system gives thousands of requests the very same latency, so the candidates never thin out and all eight
    passes run; two latency values with a few thousand requests each thin out only at the last differing digit; a
    short stream is small from the start.  All three against numpy."""
    from types import SimpleNamespace
    from mms_amd.placement_policy.base_policy import ModelPlacement
    from mms_amd.profiling import ParallelConfig, synthetic_profile
    pcs = [ParallelConfig(1, 1, 1), ParallelConfig(1, 1, 2)]
    profiles = [synthetic_profile("a", 0.1, pcs), synthetic_profile("b", 0.1000001, pcs)]
    sols = [ModelPlacement([pcs[0], pcs[0]], [[0], [1]]), ModelPlacement([pcs[1]], [[0, 1]])]
    for R, gap in ((20000, 1.0), (6000, 0.12), (300, 1.0), (1025, 1.0), (2049, 1.0)):
        t = np.arange(R) * gap                                   # gap 1.0: every request finds its group idle
        m = (np.arange(R) % 2).astype(np.int32)
        cfg = SimpleNamespace(profiles=profiles, batch_sizes=[1], num_models=2,
                              stream=lambda s, t=t, m=m: SimpleNamespace(tstamps=t, model_ids=m, slos=np.full(len(t), 5.0, np.float32)))
        out = _check(eng, cfg, sols, (0,), [(0,), (R // 7,)])
        lat = out["finish"][0, 0, :R] - t
        assert out["good"][0, 0].all()
        if R == 20000:      # (the latency only changes in its last bits from one binade of the arrival time to the next)
            for model in (0, 1):
                assert np.unique(lat[m == model], return_counts=True)[1].max() > 2 * 1024


def test_negative_latencies_of_the_batching_simulator(eng):
    """A group that became idle earlier can pick a request up with its old idle time and finish it before it arrived
    (controller.py:739-744, :715-720; the oracle does the same): the selection must order negative latencies below
    the positive ones.  Placement 104 on stream 29 has one such request (found by a randomized comparison)."""
    cfg = make_config(5, 105)
    cfg.duration = 40.0
    st = cfg.stream(29)
    R = len(st.tstamps)
    out = _check(eng, cfg, cfg.placements[100:105], (29,), [(0,), (R // 50,)], flags=_lib.BATCHING)
    latency = out["finish"][0, :, :R] - st.tstamps[None, :]
    assert ((latency < 0) & out["good"][0, :, :R]).any()


def test_requires_per_request_outputs_and_the_same_streams(eng):
    cfg = make_config(2, 4)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    st = cfg.stream(0)
    dw = E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models)
    batch = E.Batch(eng, [dw], table, E.pack_placements(cfg.placements, table), 0)
    batch.run()
    batch.sync()
    with pytest.raises(_lib.MmsimError, match="MMSIM_WANT_PER_REQUEST"):
        batch.model_stats([0])
    batch.close()
    batch = E.Batch(eng, [dw], table, E.pack_placements(cfg.placements, table), _lib.WANT_PER_REQUEST)
    with pytest.raises(_lib.MmsimError, match="never run"):
        batch.model_stats([0])
    batch.run()
    batch.sync()
    other = E.DeviceWorkload(eng, st.tstamps[:-1], st.model_ids[:-1], st.slos[:-1], cfg.num_models)
    batch.workloads = [other]
    with pytest.raises(_lib.MmsimError, match="streams the batch was created with"):
        batch.model_stats([0])
    # another stream of the same length and model count is refused too: the batch knows its workloads
    twin = E.DeviceWorkload(eng, st.tstamps, np.roll(st.model_ids, 1), st.slos, cfg.num_models)
    batch.workloads = [twin]
    with pytest.raises(_lib.MmsimError, match="streams the batch was created with"):
        batch.model_stats([0])
    batch.workloads = [dw]
    batch.model_stats([0])
    batch.close()
