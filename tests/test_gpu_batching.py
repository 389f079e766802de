"""GPU parity of the batching simulator.

Bars: served/dropped flags, finish times and all counts bit-exact against
(a) the golden vectors written by the reference's own function and (b) the CPU
oracle on the seeded benchmark configuration.  The per-lane latency sum is
accumulated in service order on the GPU and in arrival order by the oracle, so
it is compared to 1e-12 relative.
"""
import os

import numpy as np
import pytest

from mms_amd import _lib, engine as E
from mms_amd.synthetic import make_config
from oracle import oracle_c
from randcase import random_case
from helpers import oracle_batch

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "batching_vectors.npz")
BSS = [1, 2, 4, 8, 16]


@pytest.fixture(scope="module")
def eng():
    return E.Engine.default()


def _single(eng, c, bss):
    R = len(c["tstamps"])
    fin, good = np.empty(R), np.empty(R, bool)
    cnt = E.simulate_requests_mixed_batching(eng, fin, good, c["tstamps"], c["model_ids"], c["slos"], c["m2g"],
                                             c["g2m"], c["num_stages"], c["lat"], bss)
    return fin, good, cnt


def test_reference_golden_vectors(eng):
    z = np.load(GOLDEN)
    n = int(z["num_cases"])
    for i in range(n):
        g = lambda k: z[f"c{i}_{k}"]
        c = {k: g(k) for k in ("tstamps", "model_ids", "slos", "m2g", "g2m", "num_stages", "lat")}
        fin, good, cnt = _single(eng, c, BSS[:int(g("nb"))])
        assert np.array_equal(good, g("good")), i
        assert np.array_equal(fin.view(np.uint64), g("finish").view(np.uint64)), i
        for a, k in zip(cnt, ("mreq", "mgood", "greq", "ggood")):
            assert np.array_equal(a, g(k)), (i, k)


def test_random_cases_match_oracle(eng):
    for seed in range(200):
        nb = 1 + seed % 5
        c = random_case(3_000_000 + seed, max_m=6, max_g=4, max_s=4, max_r=200, nb=nb, load=1.0 + seed % 9,
                        inf_slo=False)
        bss = BSS[:nb]
        f0, g0, c0, _ = oracle_c.simulate_requests_mixed_batching(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
        fin, good, cnt = _single(eng, c, bss)
        assert np.array_equal(good, g0), seed
        assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64)), seed
        for a, b in zip(cnt, c0):
            assert np.array_equal(a, b), seed


def test_batches_of_sixteen_and_more(eng):
    """Batches larger than the sixteen queue entries that an octet fetches at once: the arrival behind the batch
    and the members past the fetched ones come from memory.  (Seeds found by a randomized comparison.)"""
    biggest = 0
    for seed in (137, 160, 179, 215, 226, 304, 311, 412, 497, 592, 593, 647, 664, 773, 857, 1000, 1006, 1091):
        nb = 1 + seed % 6
        assert nb >= 5
        c = random_case(9_000_000 + seed, max_m=2 + seed % 12, max_g=1 + seed % 14, max_s=1 + seed % 8, max_r=300,
                        nb=nb, load=0.5 + (seed % 23), inf_slo=False, tie_prob=0.05 * (seed % 8),
                        p_member=0.2 + 0.1 * (seed % 7))
        bss = [1 << k for k in range(nb)]
        f0, g0, c0, _ = oracle_c.simulate_requests_mixed_batching(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
        fin, good, cnt = _single(eng, c, bss)
        assert np.array_equal(good, g0), seed
        assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64)), seed
        for a, b in zip(cnt, c0):
            assert np.array_equal(a, b), seed
        if g0.any():
            biggest = max(biggest, int(np.unique(f0[g0], return_counts=True)[1].max()))
    assert biggest >= 16


@pytest.mark.parametrize("lanes", [8, 64])
def test_batch_sizes_that_are_not_powers_of_two(eng, opts, lanes):
    """The latency column of a batch size is floor(log2(size)) (controller.py:668, :716), so sizes such as 3 and 5
    share columns with 2 and 4; the kernel's shortcut for sizes 1, 2, 4, ... must not be taken then."""
    opts(batching_lanes=lanes)
    odd = [1, 2, 3, 5, 8, 9, 17]        # floor(log2) = 0, 1, 1, 2, 3, 3, 4
    grown = 0
    for seed in range(60):
        nb = 2 + seed % 6
        c = random_case(5_000_000 + 1000 * lanes + seed, max_m=6, max_g=4, max_s=5, max_r=250, nb=nb,
                        load=3.0 + seed % 9, inf_slo=False)
        bss = odd[:nb]
        f0, g0, c0, _ = oracle_c.simulate_requests_mixed_batching(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
        fin, good, cnt = _single(eng, c, bss)
        assert np.array_equal(good, g0), seed
        assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64)), seed
        for a, b in zip(cnt, c0):
            assert np.array_equal(a, b), seed
        served = f0[g0]
        grown += int(len(served) - len(np.unique(served)))     # requests that shared a batch finish together
    assert grown > 100


@pytest.mark.parametrize("lanes", [8, 16, 32, 64])
@pytest.mark.parametrize("lds_tables", [0, 1, 2, 3])
def test_every_kernel_variant(eng, opts, lanes, lds_tables):
    """Tile width (simulating lanes per wavefront), which tables are read from LDS, and the number of latency
    columns held in registers (4, 8 or 16) are picked from the input's size; here each is forced."""
    opts(batching_lanes=lanes)
    opts(batching_lds_tables=lds_tables)
    all_bss = [1 << k for k in range(16)]
    for seed, nb in enumerate([1, 3, 4, 5, 8, 9, 16] * 4):
        c = random_case(4_000_000 + 100 * lanes + 10 * lds_tables + seed, max_m=7, max_g=5, max_s=6, max_r=150,
                        nb=nb, load=2.0 + seed % 7, inf_slo=False)
        bss = all_bss[:nb]
        f0, g0, c0, _ = oracle_c.simulate_requests_mixed_batching(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
        fin, good, cnt = _single(eng, c, bss)
        assert np.array_equal(good, g0), (seed, nb)
        assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64)), (seed, nb)
        for a, b in zip(cnt, c0):
            assert np.array_equal(a, b), (seed, nb)


@pytest.mark.parametrize("lanes", [8, 16])
def test_many_groups_many_pending_events(eng, opts, lanes):
    """More than 64 groups busy at once: the idle events fill more than eight chunks of the event list, so
    the scan of the chunk minima takes several rounds."""
    opts(batching_lanes=lanes)
    for seed in (12, 19, 22, 44, 50, 70):      # 74 to 90 groups each, up to 23 replicas per model
        c = random_case(6_000_000 + seed, max_m=40, max_g=90, max_s=2, max_r=1500, nb=3, load=60.0,
                        inf_slo=False, tie_prob=0.1, p_member=0.15)
        assert c["m2g"].shape[1] >= 70
        bss = BSS[:3]
        f0, g0, c0, max_heap = oracle_c.simulate_requests_mixed_batching(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
        assert max_heap > 64, max_heap
        fin, good, cnt = _single(eng, c, bss)
        assert np.array_equal(good, g0), seed
        assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64)), seed
        for a, b in zip(cnt, c0):
            assert np.array_equal(a, b), seed


@pytest.mark.parametrize("lanes", [8, 16])
def test_a_simulation_that_runs_out_of_event_slots(eng, opts, lanes):
    """With fewer event slots than the reference's heap holds entries a simulation stops with MMSIM_E_OVERFLOW (the
    slots are provisioned from the group count; here they are forced down to eight).  A batch reports that in
    status[] instead of returning numbers; the one-call entry points simulate such a simulation again with twice the
    slots until it fits, so their results are the reference's."""
    opts(batching_lanes=lanes)
    opts(batching_event_slots=8)
    c = random_case(6_000_012, max_m=40, max_g=90, max_s=2, max_r=1500, nb=3, load=60.0,
                    inf_slo=False, tie_prob=0.1, p_member=0.15)
    f0, g0, c0, max_heap = oracle_c.simulate_requests_mixed_batching(
        c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], BSS[:3])
    assert max_heap > 32
    fin, good, cnt = _single(eng, c, BSS[:3])      # 8 -> 16 -> 32 -> ... slots inside the call
    assert np.array_equal(good, g0)
    assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64))
    for a, b in zip(cnt, c0):
        assert np.array_equal(a, b)

    cfg = make_config(5, 24)
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(cfg.placements, table)
    st = cfg.stream(0)
    n = 30000
    dw = E.DeviceWorkload(eng, st.tstamps[:n], st.model_ids[:n], st.slos[:n], cfg.num_models)
    flags = _lib.BATCHING | _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    batch = E.Batch(eng, [dw], table, packed, flags)
    batch.run()
    batch.sync()
    with pytest.raises(_lib.MmsimError) as err:
        batch.fetch()
    assert err.value.code == _lib.E_OVERFLOW
    assert (batch.fetch(allow_failed=True)["status"] == _lib.E_OVERFLOW).any()
    batch.close()
    out = E.evaluate(eng, [dw], table, cfg.placements, flags)
    lat, pp = table.arrays()
    ref = oracle_c.eval_placements(st.tstamps[:n], st.model_ids[:n], st.slos[:n], lat, pp, cfg.batch_sizes, *packed,
                                   batching=True, want_counts=True)
    assert not out["status"].any()
    assert np.array_equal(out["n_good"][0], ref["n_good"])
    np.testing.assert_allclose(out["latency_sum"][0], ref["latency_sum"], rtol=1e-12)
    for k in ("model_num_requests", "model_num_good", "group_num_requests", "group_num_good"):
        assert np.array_equal(out[k][0][:, :ref[k].shape[1]], ref[k]), k
    # ... and so does the paired entry point (placement b on stream b mod 2)
    n2 = 20000
    dw2 = E.DeviceWorkload(eng, st.tstamps[:n2], st.model_ids[:n2], st.slos[:n2], cfg.num_models)
    stream_of = np.arange(len(cfg.placements), dtype=np.int32) % 2
    got = E.eval_pairs(eng, [dw, dw2], table, packed, stream_of, flags)
    ref2 = oracle_c.eval_placements(st.tstamps[:n2], st.model_ids[:n2], st.slos[:n2], lat, pp, cfg.batch_sizes, *packed,
                                    batching=True, want_counts=True)
    for b in range(len(cfg.placements)):
        r = ref2 if stream_of[b] else ref
        assert got["n_good"][b] == r["n_good"][b], b
        assert np.array_equal(got["model_num_good"][b], r["model_num_good"][b]), b
    dw2.close()
    dw.close()
    opts(batching_event_slots=0)
    _single(eng, c, BSS[:3])                 # and the context is fine afterwards


def test_groups_that_become_idle_at_the_same_instant(eng):
    """Idle events with equal times are popped in group order (the reference's heap holds (time, group)
    tuples, alpa_serve/simulator/controller.py:728-740).  Twelve identical one-stage groups all start a
    request at the same arrival time, so twelve events share one time and span two chunks of the kernel's
    event list; the queued requests they pick up afterwards keep the times equal."""
    G = M = 12
    rng = np.random.default_rng(7)
    waves = 6
    tst = np.repeat(np.arange(waves) * 0.05, M)          # M arrivals at each instant, one per model
    mids = np.concatenate([rng.permutation(M) for _ in range(waves)]).astype(np.int32)
    slos = np.full(tst.size, 5.0, np.float32)
    m2g = np.full((M, G), -1, np.int32)                   # [M][G] and [G][M], unused entries -1
    g2m = np.full((G, M), -1, np.int32)
    for m in range(M):
        m2g[m, 0] = (m * 5) % G                           # a permutation of the groups
        g2m[(m * 5) % G, 0] = m
    lat = np.full((M, G, 1, 2), 0.125, np.float32)        # same latency everywhere, both batch sizes
    c = {"tstamps": tst, "model_ids": mids, "slos": slos, "m2g": m2g, "g2m": g2m,
         "num_stages": np.ones(G, np.int32), "lat": lat}
    bss = [1, 2]
    f0, g0, c0, _ = oracle_c.simulate_requests_mixed_batching(
        c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
    assert g0.sum() > M                                   # queued requests were served from idle events
    fin, good, cnt = _single(eng, c, bss)
    assert np.array_equal(good, g0)
    assert np.array_equal(fin.view(np.uint64), f0.view(np.uint64))
    for a, b in zip(cnt, c0):
        assert np.array_equal(a, b)


def _run(eng, cfg, sols, seeds, flags):
    table = E.LatencyTable(cfg.profiles, cfg.batch_sizes)
    packed = E.pack_placements(sols, table)
    streams = [cfg.stream(s) for s in seeds]
    dws = [E.DeviceWorkload(eng, st.tstamps, st.model_ids, st.slos, cfg.num_models) for st in streams]
    batch = E.Batch(eng, dws, table, packed, flags | _lib.BATCHING)
    batch.run()
    ms = batch.sync()
    out = batch.fetch()
    info = batch.info()
    batch.close()
    return out, table, packed, streams, info, ms


def _check(out, ref, s, per_request=False):
    assert np.all(out["status"][s] == 0)
    assert np.array_equal(out["n_good"][s], ref["n_good"])
    assert np.array_equal(out["model_num_requests"][s], ref["model_num_requests"])
    assert np.array_equal(out["model_num_good"][s], ref["model_num_good"])
    assert np.array_equal(out["group_num_requests"][s], ref["group_num_requests"])
    assert np.array_equal(out["group_num_good"][s], ref["group_num_good"])
    np.testing.assert_allclose(out["latency_sum"][s], ref["latency_sum"], rtol=1e-12, atol=0)
    if per_request:
        R = ref["finish"].shape[1]
        assert np.array_equal(out["good"][s][:, :R], ref["good"])
        assert np.array_equal(out["finish"][s][:, :R].view(np.uint64), ref["finish"].view(np.uint64))


def test_config5_subsample_counts(eng):
    cfg = make_config(5, 96)
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    out, table, packed, streams, info, ms = _run(eng, cfg, cfg.placements, cfg.base_seeds, flags)
    assert len(streams) == 4
    print(info, f"kernel {ms:.1f} ms", flush=True)
    for s, st in enumerate(streams):
        ref = oracle_batch(st, table, packed, batching=True)
        _check(out, ref, s)


def test_config5_full_size_properties(eng):
    """Configuration 5 at full size (8192 candidates x 4 arrival seeds): no simulation runs out of event
    slots, a placement's results do not depend on where it sits in the batch or on what shares its
    wavefront, and the counts are consistent with each other and with the streams."""
    cfg = make_config(5)
    B = len(cfg.placements)
    assert B == 8192
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
    base, table, packed, streams, info, ms = _run(eng, cfg, cfg.placements, cfg.base_seeds, flags)
    print(info, f"kernel {ms:.1f} ms", flush=True)
    assert info["lanes"] == 4 * B and np.all(base["status"] == 0)
    # a permutation of the candidate list permutes the results
    perm = np.random.default_rng(11).permutation(B)
    shuffled, *_ = _run(eng, cfg, [cfg.placements[i] for i in perm], cfg.base_seeds, 0)
    assert np.all(shuffled["status"] == 0)
    assert np.array_equal(shuffled["n_good"], base["n_good"][:, perm])
    assert np.array_equal(shuffled["latency_sum"], base["latency_sum"][:, perm])
    # a small batch (other tile width, other LDS layout) agrees, and agrees with the oracle
    pick = perm[:40]
    small, t2, p2, *_ = _run(eng, cfg, [cfg.placements[i] for i in pick], cfg.base_seeds[:1], flags)
    for k in ("n_good", "model_num_good"):
        assert np.array_equal(small[k][0], base[k][0][pick]), k
    for k in ("group_num_requests", "group_num_good"):      # the group axis is as wide as the batch's largest placement
        g = small[k][0].shape[1]
        assert np.array_equal(small[k][0], base[k][0][pick][:, :g]) and not base[k][0][pick][:, g:].any(), k
    # batch members are summed in another order by tiles of another width: 1e-12 relative
    np.testing.assert_allclose(small["latency_sum"][0], base["latency_sum"][0][pick], rtol=1e-12, atol=0)
    ref = oracle_batch(streams[0], t2, p2, batching=True)
    _check(small, ref, 0)
    # counts: goodput = sum of per-model goods = sum of per-group goods; every request of a hosted model is
    # served or dropped on exactly one group; models without a replica are not counted at all
    assert np.array_equal(base["model_num_good"].sum(axis=2), base["n_good"])
    assert np.array_equal(base["group_num_good"].sum(axis=2), base["n_good"])
    assert np.array_equal(base["group_num_requests"].sum(axis=2), base["model_num_requests"].sum(axis=2))
    hosted = np.zeros((B, cfg.num_models), bool)
    for b, pl in enumerate(cfg.placements):
        for ms_ in pl.group_models:
            hosted[b, list(ms_)] = True
    for s, st in enumerate(streams):
        per_model = np.bincount(st.model_ids[st.model_ids >= 0], minlength=cfg.num_models)
        assert np.array_equal(base["model_num_requests"][s], hosted * per_model[None, :])
        assert np.all(base["n_good"][s] <= len(st.tstamps))


def test_config5_full_traces_for_a_few_placements(eng):
    cfg = make_config(5, 3)
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS | _lib.WANT_PER_REQUEST
    out, table, packed, streams, _, _ = _run(eng, cfg, cfg.placements, [2], flags)
    ref = oracle_batch(streams[0], table, packed, batching=True, want_per_request=True)
    _check(out, ref, 0, per_request=True)


def test_batching_on_the_small_configs_too(eng):
    # configuration 2's placements with a batch-size axis added to the profiles
    from mms_amd.profiling import synthetic_profile
    cfg = make_config(2, 70)
    pcs = sorted({c for s in cfg.placements for c in s.group_configs})
    cfg.batch_sizes = [1, 2, 4]
    cfg.profiles = [synthetic_profile(f"m{m}", float(cfg.latencies[m]), pcs, batch_sizes=cfg.batch_sizes,
                                      batch_slope=0.2) for m in range(cfg.num_models)]
    flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS | _lib.WANT_PER_REQUEST
    out, table, packed, streams, _, _ = _run(eng, cfg, cfg.placements, [0, 3], flags)
    for s, st in enumerate(streams):
        ref = oracle_batch(st, table, packed, batching=True, want_per_request=True)
        _check(out, ref, s, per_request=True)
