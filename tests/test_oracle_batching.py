"""Pins for the CPU oracle of the batching simulator.

No reference test covers simulate_requests_mixed_batching
(alpa_serve/simulator/controller.py:631-798).  The golden vectors in
tests/golden/batching_vectors.npz were written by that very function
(tests/golden/make_batching_vectors.py); both restatements must reproduce
them bit for bit.  On top: behaviour probes and invariants.
"""
import os

import numpy as np
import pytest

from oracle import oracle_c, oracle_py
from randcase import random_case

F32 = np.float32
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "batching_vectors.npz")
BSS = [1, 2, 4, 8, 16]


def _same(a, fin, good, counts):
    assert np.array_equal(a[0].view(np.uint64), fin.view(np.uint64))
    assert np.array_equal(a[1], good)
    for x, y in zip(a[2], counts):
        assert np.array_equal(x, y)


def test_both_restatements_reproduce_the_reference_vectors():
    z = np.load(GOLDEN)
    n = int(z["num_cases"])
    assert n >= 200
    shared = 0
    for i in range(n):
        g = lambda k: z[f"c{i}_{k}"]
        bss = BSS[:int(g("nb"))]
        args = (g("tstamps"), g("model_ids"), g("slos"), g("m2g"), g("g2m"), g("num_stages"), g("lat"), bss)
        want = (g("finish"), g("good"), [g(k) for k in ("mreq", "mgood", "greq", "ggood")])
        _same(oracle_c.simulate_requests_mixed_batching(*args), *want)
        _same(oracle_py.simulate_mixed_batching(*args), *want)
        fin = g("finish")[g("good")]
        shared += len(fin) - len(np.unique(fin))
    assert shared > 1000          # the vectors do exercise batches larger than one


def _one_group_one_model(S, lat_by_bs):
    """lat_by_bs[b] = per-stage latency for batch_sizes[b]."""
    nb = len(lat_by_bs)
    lat = np.zeros((1, 1, S, nb), F32)
    for b, v in enumerate(lat_by_bs):
        lat[0, 0, :, b] = v
    return (np.zeros((1, 1), np.int32), np.zeros((1, 1), np.int32), np.array([S], np.int32), lat)


def test_overhead_is_added_before_the_stages_when_a_batch_runs():
    rng = np.random.default_rng(5)
    probes = 0
    for _ in range(200):
        s = float(F32(rng.uniform(0.05, 0.3)))
        t0 = float(rng.uniform(0.1, 50.0))
        first, last = ((t0 + 0.011) + s) + s, ((t0 + s) + s) + 0.011
        m2g, g2m, ns, lat = _one_group_one_model(2, [s])
        fin, good, _, _ = oracle_c.simulate_requests_mixed_batching(
            np.array([t0]), np.zeros(1, np.int32), np.array([1.0], F32), m2g, g2m, ns, lat, [1])
        assert good[0] and fin[0] == first
        probes += first != last
    assert probes >= 5            # the two orders do round differently on these inputs


def test_waiting_requests_are_batched_when_the_group_frees_up():
    # one model, latencies 0.1 (bs1) / 0.12 (bs2) / 0.16 (bs4); requests at 0, .01, .02, .03, .04
    m2g, g2m, ns, lat = _one_group_one_model(1, [0.1, 0.12, 0.16])
    ts = np.array([0.0, 0.01, 0.02, 0.03, 0.04])
    fin, good, cnt, _ = oracle_c.simulate_requests_mixed_batching(
        ts, np.zeros(5, np.int32), np.full(5, 5.0, F32), m2g, g2m, ns, lat, [1, 2, 4])
    first = (0.0 + 0.011) + float(F32(0.1))
    assert fin[0] == first
    # the other four wait; when the drain loop pops the idle event they run as one batch of 4
    second = max(first + 0.011, first) + float(F32(0.16))
    assert fin[1:].tolist() == [second] * 4 and good.all()
    assert cnt[2].tolist() == [5] and cnt[3].tolist() == [5] and cnt[1].tolist() == [5]
    a = oracle_py.simulate_mixed_batching(ts, np.zeros(5, np.int32), np.full(5, 5.0, F32), m2g, g2m, ns, lat, [1, 2, 4])
    assert np.array_equal(a[0], fin)


def test_batch_does_not_grow_without_enough_waiting_requests():
    m2g, g2m, ns, lat = _one_group_one_model(1, [0.1, 0.12, 0.16])
    ts = np.array([0.0, 0.01, 0.02, 0.03])       # 3 waiting -> batch of 2 (4 needs 3 more besides the head)
    fin, good, _, _ = oracle_c.simulate_requests_mixed_batching(
        ts, np.zeros(4, np.int32), np.full(4, 5.0, F32), m2g, g2m, ns, lat, [1, 2, 4])
    assert fin[1] == fin[2] and fin[3] != fin[2]     # (1,2) batched, 3 alone... or with nothing left
    first = (0.0 + 0.011) + float(F32(0.1))
    assert fin[1] == (first + 0.011) + float(F32(0.12))


def test_head_request_that_cannot_make_its_deadline_is_dropped_and_counted():
    m2g, g2m, ns, lat = _one_group_one_model(1, [0.1])
    ts = np.array([0.0, 0.01, 0.02])
    slos = np.array([1.0, 0.12, 1.0], F32)      # the 2nd can start only at .111 -> .232 > .01+.12
    fin, good, cnt, _ = oracle_c.simulate_requests_mixed_batching(
        ts, np.zeros(3, np.int32), slos, m2g, g2m, ns, lat, [1])
    assert good.tolist() == [True, False, True] and fin[1] == ts[1]
    assert cnt[0].tolist() == [3] and cnt[1].tolist() == [2]
    assert cnt[2].tolist() == [3] and cnt[3].tolist() == [2]


def test_unplaced_model_is_not_counted_in_the_batching_variant():
    m2g = np.array([[0], [-1]], np.int32)
    g2m = np.array([[0, -1]], np.int32)
    lat = np.full((2, 1, 1, 1), 0.1, F32)
    fin, good, cnt, _ = oracle_c.simulate_requests_mixed_batching(
        np.array([0.0, 1.0]), np.array([1, -1], np.int32), np.full(2, 1.0, F32), m2g, g2m,
        np.array([1], np.int32), lat, [1])
    assert not good.any() and cnt[0].tolist() == [0, 0]


@pytest.mark.parametrize("nb", [1, 2, 3, 4, 5])
def test_restatements_agree_and_invariants_hold(nb):
    bss = BSS[:nb]
    for seed in range(400):
        c = random_case(2_000_000 + 1000 * nb + seed, nb=nb, max_r=120, load=1.0 + seed % 7, inf_slo=False)
        args = (c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"], c["num_stages"], c["lat"], bss)
        fin, good, (mreq, mgood, greq, ggood), h = oracle_c.simulate_requests_mixed_batching(*args)
        b = oracle_py.simulate_mixed_batching(*args)
        _same(b, fin, good, (mreq, mgood, greq, ggood))
        assert b[3] == h
        ts = c["tstamps"]
        assert np.all(fin >= ts)
        assert np.array_equal(fin[~good], ts[~good])
        # every enqueued request is served or dropped on exactly one group
        assert greq.sum() == mreq.sum()
        assert ggood.sum() == mgood.sum() == good.sum()
        # requests that share a finish time form batches of an allowed size, all of one model
        for f in np.unique(fin[good]):
            members = np.flatnonzero(good & (fin == f))
            by_model = {}
            for r in members:
                by_model.setdefault(int(c["model_ids"][r]), []).append(r)
            for rs in by_model.values():
                assert len(rs) <= bss[-1]
