"""Test-only stand-in for the GPU library, built on the CPU oracle.

``install(monkeypatch)`` swaps the entry points of ``mms_amd.engine`` that
reach libmmsim for oracle-backed ones, so that the host-side logic (packing,
PlacementEvaluator, approximate_one_case, the search policies) can be tested
on a machine without a GPU.  Nothing outside tests/ may use this; the shipped
package has no such path.
"""
import numpy as np

from mms_amd import _lib, engine as E
from oracle import oracle_c


class _HostWorkload:
    def __init__(self, engine, tstamps, model_ids, slos, num_models):
        self.tstamps = np.ascontiguousarray(tstamps, np.float64)
        self.model_ids = np.ascontiguousarray(model_ids, np.int32)
        self.slos = np.ascontiguousarray(slos, np.float32)
        self.R = len(self.tstamps)
        self.M = int(num_models)

    def close(self):
        pass


class _HostEngine:
    device = -1

    def device_info(self):
        return {"name": "cpu-oracle", "arch": "none", "compute_units": 0, "clock_khz": 0,
                "lds_bytes_per_block": 0, "hbm_bytes": 0}


def _evaluate(engine, workloads, table, sols, flags=0, fixed_overhead=0.011):
    packed = E.pack_placements(sols, table)
    lat, pp = table.arrays()
    num_groups, group_cfg, gm_off, gm_idx = packed
    outs = []
    for w in workloads:
        outs.append(oracle_c.eval_placements(
            w.tstamps, w.model_ids, w.slos, lat, pp, table.batch_sizes, num_groups, group_cfg, gm_off,
            gm_idx, batching=bool(flags & _lib.BATCHING), fixed_overhead=fixed_overhead,
            want_counts=True, want_per_request=bool(flags & _lib.WANT_PER_REQUEST)))
    res = {"n_good": np.stack([o["n_good"] for o in outs]),
           "latency_sum": np.stack([o["latency_sum"] for o in outs]),
           "status": np.zeros((len(outs), len(sols)), np.int32)}
    for k in ("model_num_requests", "model_num_good", "group_num_requests", "group_num_good"):
        res[k] = np.stack([o[k] for o in outs])
    if flags & _lib.WANT_PER_REQUEST:
        res["finish"] = np.stack([o["finish"] for o in outs])
        res["good"] = np.stack([o["good"] for o in outs])
    return res


def _evaluate_successors(engine, workloads, table, bases, parent, group, model, flags=0, normalize=True,
                         fixed_overhead=0.011):
    """The successors as Python objects (what the library builds itself), then the plain oracle."""
    kids = []
    for p, g, m in zip(parent, group, model):
        kid = bases[int(p)].add_model(int(g), int(m))
        kids.append(kid.normalize() if normalize else kid)
    return _evaluate(engine, workloads, table, list(bases) + kids, flags, fixed_overhead)


def _eval_pairs(engine, workloads, table, packed, stream_of, flags=0, fixed_overhead=0.011):
    """Placement b on workloads[stream_of[b]] only; result arrays [B][...]."""
    lat, pp = table.arrays()
    num_groups, group_cfg, gm_off, gm_idx = packed
    B, Gmax = group_cfg.shape
    M = lat.shape[0]
    Rmax = max(w.R for w in workloads)
    res = {"n_good": np.zeros(B, np.int64), "latency_sum": np.zeros(B), "status": np.zeros(B, np.int32),
           "model_num_requests": np.zeros((B, M), np.int32), "model_num_good": np.zeros((B, M), np.int32),
           "group_num_requests": np.zeros((B, Gmax), np.int32), "group_num_good": np.zeros((B, Gmax), np.int32)}
    if flags & _lib.WANT_PER_REQUEST:
        res["finish"] = np.zeros((B, Rmax))
        res["good"] = np.zeros((B, Rmax), bool)
    for b in range(B):
        w = workloads[stream_of[b]]
        off = gm_off[b:b + 1] - gm_off[b, 0]
        idx = gm_idx[gm_off[b, 0]:gm_off[b, -1]]
        o = oracle_c.eval_placements(
            w.tstamps, w.model_ids, w.slos, lat, pp, table.batch_sizes, num_groups[b:b + 1], group_cfg[b:b + 1],
            off, idx, batching=bool(flags & _lib.BATCHING), fixed_overhead=fixed_overhead,
            want_counts=True, want_per_request=bool(flags & _lib.WANT_PER_REQUEST))
        for k in ("n_good", "latency_sum", "model_num_requests", "model_num_good", "group_num_requests",
                  "group_num_good"):
            res[k][b] = o[k][0]
        if flags & _lib.WANT_PER_REQUEST:
            res["finish"][b, :w.R] = o["finish"][0]
            res["good"][b, :w.R] = o["good"][0]
    return res


def model_stats_numpy(tstamps, model_ids, finish, good, skip, M):
    """What mmsim_batch_model_stats returns for one simulation, restated with numpy from the
    conventions of Workload.compute_stats (workload.py:308-354): window [skip, R - skip), order
    statistics sorted[int(q * n)], np.mean / np.std of the accepted requests' latencies."""
    R = len(tstamps)
    lo, hi = min(skip, R), max(min(skip, R), R - skip)
    out = {k: np.zeros(M, np.int32) for k in ("model_num_requests", "model_num_good")}
    out.update({k: np.zeros(M) for k in ("first_start", "last_start", "latency_sum", "latency_mean",
                                         "latency_std", "latency_p90", "latency_p99")})
    ids = model_ids[lo:hi]
    for m in range(M):
        sel = np.nonzero(ids == m)[0] + lo
        ok = sel[np.asarray(good[sel], bool)]
        out["model_num_requests"][m] = len(sel)
        out["model_num_good"][m] = len(ok)
        if len(ok):
            lat = np.sort(finish[ok] - tstamps[ok])
            out["first_start"][m], out["last_start"][m] = tstamps[ok[0]], tstamps[ok[-1]]
            out["latency_sum"][m] = np.sum(lat)
            out["latency_mean"][m], out["latency_std"][m] = np.mean(lat), np.std(lat)
            out["latency_p90"][m] = lat[int(0.90 * len(lat))]
            out["latency_p99"][m] = lat[int(0.99 * len(lat))]
    return out


class _HostBatch:
    """Stand-in for engine.Batch: run / sync / fetch / model_stats on the oracle's outputs."""

    def __init__(self, engine, workloads, table, packed, flags, fixed_overhead=0.011, options=None):
        self.workloads, self.table, self.packed = list(workloads), table, packed
        self.flags, self.fixed_overhead = int(flags), fixed_overhead
        self.n_seeds, self.B, self.M = len(self.workloads), packed[1].shape[0], table.arrays()[0].shape[0]
        self.out = None

    def run(self):
        lat, pp = self.table.arrays()
        num_groups, group_cfg, gm_off, gm_idx = self.packed
        outs = [oracle_c.eval_placements(
            w.tstamps, w.model_ids, w.slos, lat, pp, self.table.batch_sizes, num_groups, group_cfg, gm_off,
            gm_idx, batching=bool(self.flags & _lib.BATCHING), fixed_overhead=self.fixed_overhead,
            want_counts=True, want_per_request=bool(self.flags & _lib.WANT_PER_REQUEST)) for w in self.workloads]
        Rmax = max(w.R for w in self.workloads)
        self.out = {}
        for k in outs[0]:
            if k in ("finish", "good"):
                arr = np.zeros((self.n_seeds, self.B, Rmax), outs[0][k].dtype)
                for s, o in enumerate(outs):
                    arr[s, :, :o[k].shape[1]] = o[k]
                self.out[k] = arr
            else:
                self.out[k] = np.stack([o[k] for o in outs])
        self.out["status"] = np.zeros((self.n_seeds, self.B), np.int32)

    def sync(self):
        return 0.0

    def fetch(self, per_request=True, allow_failed=False):
        return {k: v for k, v in self.out.items() if per_request or k not in ("finish", "good")}

    def model_stats(self, skip):
        per = [[model_stats_numpy(w.tstamps, w.model_ids, self.out["finish"][s, b, :w.R],
                                  self.out["good"][s, b, :w.R], int(skip[s]), self.M)
                for b in range(self.B)] for s, w in enumerate(self.workloads)]
        return {k: np.array([[per[s][b][k] for b in range(self.B)] for s in range(self.n_seeds)])
                for k in per[0][0]}

    def close(self):
        pass


def _simulate_requests_mixed(engine, finish, good, tstamps, model_ids, slos, m2g, num_stages, lat,
                             num_requests=None, fixed_overhead=0.011):
    f, g, cnt, _ = oracle_c.simulate_requests_mixed(tstamps, model_ids, slos, m2g, num_stages, lat, fixed_overhead)
    finish[:] = f
    good[:] = g
    return cnt


def _simulate_requests(engine, finish, good, tstamps, model_ids, slos, m2g, gmax, gsum,
                       num_requests=None, fixed_overhead=0.011):
    f, g, cnt = oracle_c.simulate_requests(tstamps, model_ids, slos, m2g, gmax, gsum, fixed_overhead)
    finish[:] = f
    good[:] = g
    return cnt


def _simulate_requests_mixed_batching(engine, finish, good, tstamps, model_ids, slos, m2g, g2m, num_stages,
                                      lat, batch_sizes, num_requests=None, fixed_overhead=0.011):
    f, g, cnt, _ = oracle_c.simulate_requests_mixed_batching(tstamps, model_ids, slos, m2g, g2m, num_stages,
                                                             lat, batch_sizes, fixed_overhead)
    finish[:] = f
    good[:] = g
    return cnt


def install(monkeypatch):
    host = _HostEngine()
    monkeypatch.setattr(E.Engine, "default", classmethod(lambda cls: host))
    monkeypatch.setattr(E, "DeviceWorkload", _HostWorkload)
    monkeypatch.setattr(E, "evaluate", _evaluate)
    monkeypatch.setattr(E, "evaluate_successors", _evaluate_successors)
    monkeypatch.setattr(E, "Batch", _HostBatch)
    monkeypatch.setattr(E, "eval_pairs", _eval_pairs)
    monkeypatch.setattr(E, "simulate_requests_mixed", _simulate_requests_mixed)
    monkeypatch.setattr(E, "simulate_requests", _simulate_requests)
    monkeypatch.setattr(E, "simulate_requests_mixed_batching", _simulate_requests_mixed_batching)
