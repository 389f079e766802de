"""Pins for the CPU oracle of the non-batched request loops.

The oracle restates alpa_serve/simulator/controller.py:561-628 (stage clocks)
and :506-558 (scalar clock).  The reference holds no per-request vectors for
them, so they are pinned by what the arithmetic fixes: closed forms, a worked
example derived by hand from the source, a textbook Lindley recursion,
behaviour probes that a plausible slip (tie-break, overhead placement,
counting of rejected requests, form of the SLO compare) would fail, and
bit-for-bit agreement of two separately written restatements.
"""
import numpy as np
import pytest

from oracle import oracle_c, oracle_py
from randcase import random_case

F32 = np.float32


def one_group(S, lat_rows):
    """M models on a single group with S stages; lat_rows[m] = S stage latencies."""
    M = len(lat_rows)
    m2g = np.zeros((M, 1), np.int32)
    lat = np.array(lat_rows, F32).reshape(M, 1, S)
    return m2g, np.array([S], np.int32), lat


def run_both(ts, mids, slos, m2g, ns, lat):
    a = oracle_c.simulate_requests_mixed(ts, mids, slos, m2g, ns, lat)
    b = oracle_py.simulate_mixed(ts, mids, slos, m2g, ns, lat)
    assert np.array_equal(a[0].view(np.uint64), b[0].view(np.uint64))
    assert np.array_equal(a[1], b[1])
    for x, y in zip(a[2], b[2]):
        assert np.array_equal(x, y)
    return a


def test_worked_example_pp2_exact_bits():
    # test-2GB-100ms at pp=2: stage latency float32(0.051 * (1 + 0.009*2)); three
    # arrivals 10 ms apart, SLO 0.5 s.  Expected finishes derived by hand:
    # (l+l)+0.011, (3 additions of l)+0.011, (4 additions of l)+0.011.
    l32 = F32(0.051 * (1 + 0.009 * 2))
    assert float(l32).hex() == "0x1.a94ff00000000p-5"
    m2g, ns, lat = one_group(2, [[l32, l32]])
    ts = np.array([0.0, 0.01, 0.02])
    fin, good, cnt, _ = run_both(ts, np.zeros(3, np.int32), np.full(3, 0.5, F32), m2g, ns, lat)
    assert [x.hex() for x in fin.tolist()] == [
        "0x1.d65e460418937p-4", "0x1.55831f020c49cp-3", "0x1.bfd71b020c49cp-3"]
    assert good.all() and cnt[0][0] == 3 and cnt[3][0] == 3


def test_table_values_of_canned_profile():
    # float32(latency * (1 + 0.009*pp)) for the canned 100 ms profile
    assert float(F32(0.100 * 1.009)).hex() == "0x1.9d49520000000p-4"
    assert float(F32(0.026 * (1 + 0.009 * 4))).hex() == "0x1.b951c60000000p-6"


@pytest.mark.parametrize("S", [1, 2, 3, 5, 8])
def test_burst_at_time_zero_is_a_running_sum(S):
    # All arrivals at t=0, one group, equal stage latency s, SLO=+inf:
    # request n leaves after S+n sequential additions of s, then +0.011.
    s = float(F32(0.0371))
    m2g, ns, lat = one_group(S, [[s] * S])
    R = 40
    fin, good, _, _ = run_both(np.zeros(R), np.zeros(R, np.int32), np.full(R, np.inf, F32), m2g, ns, lat)
    acc, sums = 0.0, []
    for _ in range(S + R):
        acc += s
        sums.append(acc)
    assert good.all()
    assert fin.tolist() == [sums[S + n - 1] + 0.011 for n in range(R)]


def test_idle_pipeline_adds_stage_latencies_left_to_right():
    lats = [float(F32(x)) for x in (0.013, 0.029, 0.007, 0.031)]
    m2g, ns, lat = one_group(4, [lats])
    ts = np.array([0.5, 3.25, 9.125, 20.0625])
    fin, good, _, _ = run_both(ts, np.zeros(4, np.int32), np.full(4, 10, F32), m2g, ns, lat)
    assert fin.tolist() == [((((t + lats[0]) + lats[1]) + lats[2]) + lats[3]) + 0.011 for t in ts]
    assert good.all()


def test_single_stage_single_server_is_lindley():
    # S=1, one group, no balking: D_n = max(A_n, D_{n-1}) + s  (G/D/1 FIFO queue)
    rng = np.random.default_rng(7)
    ts = np.cumsum(rng.exponential(0.05, 500))
    s = float(F32(0.06))
    m2g, ns, lat = one_group(1, [[s]])
    fin, good, _, _ = run_both(ts, np.zeros(500, np.int32), np.full(500, np.inf, F32), m2g, ns, lat)
    dep, want = 0.0, []
    for a in ts.tolist():
        dep = max(a, dep) + s
        want.append(dep + 0.011)
    assert good.all() and fin.tolist() == want


def test_ties_go_to_the_first_listed_group():
    # two identical single-stage groups, three arrivals at t=0: g0, g1, then the tie -> g0
    s = F32(0.1)
    m2g = np.array([[0, 1]], np.int32)
    lat = np.full((1, 2, 1), s, F32)
    _, good, cnt, _ = run_both(np.zeros(3), np.zeros(3, np.int32), np.full(3, np.inf, F32),
                               m2g, np.array([1, 1], np.int32), lat)
    assert good.all() and cnt[2].tolist() == [2, 1]
    # listing order, not group index, decides: list group 1 first
    m2g = np.array([[1, 0]], np.int32)
    _, _, cnt, _ = run_both(np.zeros(3), np.zeros(3, np.int32), np.full(3, np.inf, F32),
                            m2g, np.array([1, 1], np.int32), lat)
    assert cnt[2].tolist() == [1, 2]


def test_selection_reads_the_last_stage_clock():
    # g0 has pp=2 (last stage frees late), g1 has pp=1.  After one request on each,
    # the next goes to whichever LAST-stage clock is smaller.
    lat = np.zeros((1, 2, 2), F32)
    lat[0, 0] = [0.05, 0.30]     # last-stage clock of g0 after 1st request: 0.35
    lat[0, 1] = [0.20, 0.0]      # g1: 0.20
    m2g = np.array([[0, 1]], np.int32)
    ns = np.array([2, 1], np.int32)
    _, _, cnt, _ = run_both(np.zeros(3), np.zeros(3, np.int32), np.full(3, np.inf, F32), m2g, ns, lat)
    assert cnt[2].tolist() == [1, 2]


def test_rejected_requests_count_for_the_group_but_not_as_good_and_leave_clocks_alone():
    s = float(F32(0.1))
    m2g, ns, lat = one_group(1, [[s]])
    ts = np.array([0.0, 0.0, 0.0, 1.0])
    slos = np.array([1.0, 0.15, 0.25, 0.05], F32)   # 2nd would finish at .211 (>0.15): reject; 3rd .211 ok
    fin, good, cnt, _ = run_both(ts, np.zeros(4, np.int32), slos, m2g, ns, lat)
    assert good.tolist() == [True, False, True, False]
    assert fin[1] == ts[1] and fin[3] == ts[3]
    assert fin[2] == (s + s) + 0.011          # clock untouched by the rejected one
    assert cnt[0].tolist() == [4] and cnt[1].tolist() == [2]
    assert cnt[2].tolist() == [4] and cnt[3].tolist() == [2]


def test_unknown_model_and_unplaced_model():
    m2g = np.array([[0], [-1]], np.int32)
    lat = np.full((2, 1, 1), 0.1, F32)
    ts = np.array([0.0, 1.0, 2.0])
    fin, good, cnt, _ = run_both(ts, np.array([-1, 1, 0], np.int32), np.full(3, 1, F32),
                                 m2g, np.array([1], np.int32), lat)
    assert good.tolist() == [False, False, True]
    assert fin[0] == 0.0 and fin[1] == 1.0
    assert cnt[0].tolist() == [1, 1]      # unplaced model still counted, unknown id not
    assert cnt[2].tolist() == [1]


def test_missing_config_and_odd_slos():
    lat = np.full((1, 1, 1), np.inf, F32)
    m2g = np.zeros((1, 1), np.int32)
    ns = np.array([1], np.int32)
    ts = np.array([0.0, 1.0])
    _, good, cnt, _ = run_both(ts, np.zeros(2, np.int32), np.array([5.0, np.nan], F32), m2g, ns, lat)
    assert not good.any() and cnt[2].tolist() == [2]     # dispatched and counted, never served
    lat = np.full((1, 1, 1), 0.1, F32)
    _, good, _, _ = run_both(ts, np.zeros(2, np.int32), np.array([np.nan, np.inf], F32), m2g, ns, lat)
    assert good.tolist() == [False, True]


def test_slo_compare_is_on_the_latency_not_on_the_deadline():
    # (t + 0.011) - tstamp <= slo   versus   t + 0.011 <= tstamp + slo   round differently
    # when the arrival time is small next to the latency.  A first request keeps the
    # group busy until c; the second arrives so that its latency is within an ulp of its SLO.
    rng = np.random.default_rng(11)
    n = 400000
    c = rng.uniform(0.3, 3.0, n).astype(F32).astype(np.float64)
    s = rng.uniform(0.01, 0.4, n).astype(F32).astype(np.float64)
    slo = rng.uniform(0.2, 3.0, n).astype(F32).astype(np.float64)
    fin = (c + s) + 0.011
    ts = fin - slo
    ts = ts - rng.integers(0, 5, n) * np.spacing(ts)     # latency a few ulps(ts) above the SLO
    ok = (ts > 0) & (ts < c)
    by_latency = (fin - ts) <= slo
    by_deadline = fin <= ts + slo
    picks = np.flatnonzero(ok & (by_latency != by_deadline))[:40]
    assert len(picks) >= 20
    for i in picks:
        m2g = np.zeros((2, 1), np.int32)
        lat = np.array([c[i], s[i]], F32).reshape(2, 1, 1)
        f, good, _, _ = run_both(np.array([0.0, ts[i]]), np.array([0, 1], np.int32),
                                 np.array([np.inf, slo[i]], F32), m2g, np.array([1], np.int32), lat)
        assert bool(good[1]) == bool(by_latency[i])
        assert f[1] == (fin[i] if by_latency[i] else ts[i])


def test_slo_is_single_precision():
    # slo given as the float32 nearest to 0.111 (latency 0.1 + 0.011 overhead ~ 0.111)
    s = float(F32(0.1))
    lat_total = (0.0 + s) + 0.011
    slo32 = F32(lat_total)
    m2g, ns, lat = one_group(1, [[s]])
    _, good, _, _ = run_both(np.array([0.0]), np.zeros(1, np.int32), np.array([slo32], F32), m2g, ns, lat)
    assert bool(good[0]) == (lat_total <= float(slo32))


def test_two_restatements_agree_and_invariants_hold_on_random_cases():
    for seed in range(1500):
        c = random_case(seed)
        lat = c["lat"][..., 0]
        fin, good, (mreq, mgood, greq, ggood), ops = run_both(
            c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["num_stages"], lat)
        ts, mids = c["tstamps"], c["model_ids"]
        with np.errstate(invalid="ignore"):
            assert np.all((fin - ts)[good] <= c["slos"].astype(np.float64)[good])
        assert np.array_equal(fin[~good], ts[~good])
        assert mreq.sum() == (mids >= 0).sum()
        placed = np.array([m >= 0 and c["m2g"][m, 0] >= 0 for m in mids], bool)
        # a model whose replicas all run at +inf can leave every clock at +inf;
        # such a request is counted for the model but reaches no group
        assert greq.sum() <= placed.sum()
        if np.isfinite(lat).all():
            assert greq.sum() == placed.sum()
        assert ggood.sum() == mgood.sum() == good.sum()
        assert np.all(mgood <= mreq) and np.all(ggood <= greq)
        assert ops >= 0


def test_infinite_slo_with_finite_latency_drops_nothing():
    for seed in range(200):
        c = random_case(900000 + seed, p_inf_row=0.0, p_unknown=0.0)
        slos = np.full(c["R"], np.inf, F32)
        _, good, _, _ = run_both(c["tstamps"], c["model_ids"], slos, c["m2g"], c["num_stages"], c["lat"][..., 0])
        placed = np.array([c["m2g"][m, 0] >= 0 for m in c["model_ids"]], bool)
        assert np.array_equal(good, placed)


def test_relabelling_groups_keeps_per_request_results():
    rng = np.random.default_rng(3)
    for seed in range(200):
        c = random_case(700000 + seed)
        G = c["G"]
        perm = rng.permutation(G)              # new index of old group g is perm[g]
        inv = np.argsort(perm)
        m2g = c["m2g"].copy()
        m2g[m2g >= 0] = perm[m2g[m2g >= 0]]    # same listing order, new labels
        lat = c["lat"][..., 0][:, inv]
        ns = c["num_stages"][inv]
        a = run_both(c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["num_stages"], c["lat"][..., 0])
        b = run_both(c["tstamps"], c["model_ids"], c["slos"], m2g, ns, lat)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        assert np.array_equal(a[2][2], b[2][2][perm])


# ---- scalar-clock variant (controller.py:506-558) ---------------------------------

def test_scalar_clock_variant_closed_form_and_agreement():
    # one group, latency sum 0.3 / max 0.1: next request may start 0.1 after the previous start
    gsum, gmax = np.full((1, 1), 0.3, F32), np.full((1, 1), 0.1, F32)
    m2g = np.zeros((1, 1), np.int32)
    R = 10
    fin, good, cnt = oracle_c.simulate_requests(np.zeros(R), np.zeros(R, np.int32), np.full(R, np.inf, F32),
                                                m2g, gmax, gsum)
    start, want = 0.0, []
    for _ in range(R):
        want.append(start + float(F32(0.3)) + 0.011)
        start = start + float(F32(0.1))
    assert fin.tolist() == want and good.all()
    for seed in range(500):
        c = random_case(300000 + seed)
        gmax = c["lat"][..., 0].max(axis=2)
        gsum = c["lat"][..., 0].sum(axis=2, dtype=np.float32)
        a = oracle_c.simulate_requests(c["tstamps"], c["model_ids"], c["slos"], c["m2g"], gmax, gsum)
        b = oracle_py.simulate_scalar_clock(c["tstamps"], c["model_ids"], c["slos"], c["m2g"], gmax, gsum)
        assert np.array_equal(a[0].view(np.uint64), b[0].view(np.uint64)) and np.array_equal(a[1], b[1])
        for x, y in zip(a[2], b[2]):
            assert np.array_equal(x, y)


def test_with_one_stage_the_two_variants_coincide():
    for seed in range(300):
        c = random_case(400000 + seed, max_s=1)
        lat = c["lat"][..., 0]
        a = oracle_c.simulate_requests_mixed(c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["num_stages"], lat)
        b = oracle_c.simulate_requests(c["tstamps"], c["model_ids"], c["slos"], c["m2g"], lat[..., 0], lat[..., 0])
        assert np.array_equal(a[0].view(np.uint64), b[0].view(np.uint64)) and np.array_equal(a[1], b[1])
