"""Request streams fed to the simulators and the statistics they return.

Follows the reference's ``alpa_serve/simulator/workload.py``: ``Request``
(:17-25), the stats tuples (:28-43), the arrival processes that the
benchmark configurations use (``GammaProcess`` :114-162, ``PoissonProcess``
:165-174, ``DeterministicProcess`` :87-111) and ``Workload`` (:266-421).
Arrival generation deliberately goes through numpy's *legacy* global
generator (``np.random.seed`` / ``np.random.gamma``) because seeded
workloads must be the same numbers the reference would draw.
"""
from abc import ABC, abstractmethod
from collections import defaultdict, namedtuple
import dataclasses
from typing import Any, Dict, List, Optional, Sequence

import numpy as np

from mms_amd.util import eps, to_str_round

DEFAULT_WARMUP = 10


@dataclasses.dataclass
class Request:
    """One inference request (workload.py:17-25)."""
    model_name: str
    data: Any
    slo: Optional[float]
    idx: int
    time_stamp: Dict            # debug only
    submit_time: float = None   # filled by a client, unused by the fast path


PerModelStatsResult = namedtuple(
    "PerModelStatsResult",
    ("name", "num_requests", "goodput", "throughput", "latency_mean",
     "latency_std", "latency_p90", "latency_p99", "latency", "request_starts",
     "request_finishes"))

PerDeviceStatsResult = namedtuple("PerDeviceStatsResult", ("num_requests",))


@dataclasses.dataclass
class StatsResult:
    per_model_stats: List[PerModelStatsResult]
    group_num_requests: List[int]
    goodput: float
    latency_mean: float
    num_requests: int
    request_rate: float


class ArrivalProcess(ABC):
    """Interface of an arrival process (workload.py:46-84)."""

    @abstractmethod
    def rate(self):
        """Mean arrival rate (requests per second)."""

    @abstractmethod
    def cv(self):
        """Coefficient of variation of the inter-arrival gaps."""

    @abstractmethod
    def generate_workload(self, model_name: str, start: float, duration: float,
                          slo: Optional[float] = None, seed: int = 0):
        """Workload of requests for ``model_name`` in [start, start+duration)."""

    def params(self):
        return self.rate(), self.cv()

    def __str__(self):
        return f"{type(self).__name__}(rate={self.rate()}, cv={self.cv()})"


def _workload_from_ticks(model_name, ticks, slo):
    return Workload(ticks, [Request(model_name, None, slo, i, {})
                            for i in range(len(ticks))])


class DeterministicProcess(ArrivalProcess):
    """Equally spaced arrivals, gap 1/rate (workload.py:87-111)."""

    def __init__(self, arrival_rate: float):
        self.rate_ = arrival_rate

    def rate(self):
        return self.rate_

    def cv(self):
        return 0

    def generate_workload(self, model_name, start, duration, slo=None, seed=0):
        gap = 1 / self.rate_
        ticks = [start + i * gap for i in range(int(duration * self.rate_))]
        return _workload_from_ticks(model_name, ticks, slo)


class GammaProcess(ArrivalProcess):
    """Gamma-distributed inter-arrival gaps; cv == 1 is Poisson
    (workload.py:114-162)."""

    def __init__(self, arrival_rate: float, cv: float):
        self.rate_ = arrival_rate
        self.cv_ = cv
        self.shape = 1 / (cv * cv)
        self.scale = cv * cv / arrival_rate

    def rate(self):
        return self.rate_

    def cv(self):
        return self.cv_

    def generate_arrivals(self, start: float, duration: float, seed: int = 0):
        """Arrival instants in [start, start+duration).

        Same draw order and the same sequential fp64 accumulation as
        workload.py:135-155: gaps are drawn in blocks of
        ``max(int(rate*duration*1.2), 1)`` from the legacy global generator
        and added one by one (no cumsum, whose pairwise order would round
        differently).
        """
        np.random.seed(seed)
        block = max(int(self.rate_ * duration * 1.2), 1)
        gaps = np.random.gamma(self.shape, self.scale, size=block)
        end = start + duration
        ticks = []
        pos = 0
        now = start + gaps[0]
        while now < end:
            ticks.append(now)
            pos += 1
            if pos >= block:
                gaps = np.random.gamma(self.shape, self.scale, size=block)
                pos = 0
            now += gaps[pos]
        return ticks

    def generate_workload(self, model_name, start, duration, slo=None, seed=0):
        return _workload_from_ticks(
            model_name, self.generate_arrivals(start, duration, seed), slo)


class PoissonProcess(GammaProcess):
    """Poisson arrivals (workload.py:165-174)."""

    def __init__(self, arrival_rate: float):
        super().__init__(arrival_rate, 1)


class Workload:
    """Requests sorted by arrival time (workload.py:266-421)."""

    def __init__(self, arrivals: Sequence[float], requests: List[Request]):
        assert len(arrivals) == len(requests)
        self.arrivals = np.array(arrivals)
        self.requests = requests

        # Filled by the fast simulator on first use (model ids, SLOs, names,
        # profiles) when caching is switched on by a PlacementEvaluator.
        self.enable_simulator_cache = False
        self.cached_data = None

        if len(self.arrivals) > 1:
            gaps = self.arrivals[1:] - self.arrivals[:-1]
            self.rate = 1 / (np.mean(gaps) + eps)
            self.cv = np.std(gaps) * self.rate
        else:
            self.rate = 0
            self.cv = 0

    # -- slicing / combining -------------------------------------------------
    def __len__(self):
        return len(self.arrivals)

    def __getitem__(self, key):
        if not isinstance(key, slice):
            raise NotImplementedError()
        return Workload(self.arrivals[key], self.requests[key])

    def __add__(self, other):
        return Workload.merge(self, other)

    @classmethod
    def empty(cls):
        return cls([], [])

    @classmethod
    def merge(cls, *args):
        """Interleave workloads by arrival time and renumber ``idx``
        (workload.py:381-401).  The order among equal arrival instants is
        whatever ``np.argsort``'s default sort gives, as in the reference."""
        if len(args) == 1:
            return args[0]
        all_arrivals = np.concatenate(tuple(w.arrivals for w in args))
        all_requests = [r for w in args for r in w.requests]
        order = np.argsort(all_arrivals)
        arrivals = [all_arrivals[j] for j in order]
        requests = [all_requests[j] for j in order]
        for i, r in enumerate(requests):
            r.idx = i
        return cls(arrivals, requests)

    def split_round_robin(self, number: int):
        return [self[i::number] for i in range(number)]

    def split_time_interval(self, interval: float):
        """Cut into consecutive windows; a new window opens at the first
        arrival later than ``interval`` after the window's first arrival
        (workload.py:292-306)."""
        if len(self.arrivals) < 1:
            return []
        pieces = []
        lo = 0
        t0 = self.arrivals[0]
        for i, t in enumerate(self.arrivals):
            if t > t0 + interval:
                pieces.append(self[lo:i])
                lo, t0 = i, t
        pieces.append(self[lo:])
        return pieces

    # -- statistics ----------------------------------------------------------
    def compute_stats(self, start: Sequence[float], finish: Sequence[float],
                      good: Sequence[bool], warmup: float):
        """Serving statistics with the first and last ``warmup`` seconds'
        share of requests trimmed (workload.py:308-354).

        Per-model entries are ordered by ascending request count; percentiles
        index the sorted latencies at ``int(q*len)``.  A model without any
        good request reports latency ``[0]`` and throughput 0.  When nothing
        is trimmed all requests are used (the reference leaves its local
        ``requests`` unbound in that case, workload.py:313-322).
        """
        requests = self.requests
        if len(self.arrivals) > 1:
            span = self.arrivals[-1] - self.arrivals[0]
            skip = int(warmup / span * len(self.arrivals))
            if skip > 0:
                start = start[skip:-skip]
                finish = finish[skip:-skip]
                good = good[skip:-skip]
                requests = self.requests[skip:-skip]

        by_model = defaultdict(list)
        for i, r in enumerate(requests):
            by_model[r.model_name].append(i)
        names = sorted(by_model, key=lambda n: len(by_model[n]))  # stable

        per_model = []
        for name in names:
            idx = np.asarray(by_model[name], dtype=np.int32)
            ok = np.asarray(good[idx], dtype=bool)
            ok_start = start[idx][ok]
            ok_finish = finish[idx][ok]
            goodput = np.mean(ok)
            if goodput > 0:
                throughput = len(ok_start) / (ok_start[-1] - ok_start[0])
                latency = ok_finish - ok_start
            else:
                throughput = 0
                latency = [0]
            ordered = np.sort(latency)
            per_model.append(PerModelStatsResult(
                name, len(idx), goodput, throughput, np.mean(latency),
                np.std(latency), ordered[int(0.90 * len(ordered))],
                ordered[int(0.99 * len(ordered))], latency, ok_start,
                ok_finish))

        return StatsResult(per_model, None, np.mean(good),
                           np.mean(finish - start), len(start),
                           len(start) / (start[-1] - start[0]))

    @staticmethod
    def print_stats(stats: StatsResult):
        """Human-readable dump (workload.py:356-375)."""
        if stats.per_model_stats:
            print("--- per model ---")
            for s in stats.per_model_stats:
                print(f"model: {s.name}, #req: {s.num_requests}")
                print(f"goodput: {s.goodput*100:.2f} %, "
                      f"throughput: {s.throughput:.2f} q/s, ")
                print(f"latency mean: {s.latency_mean*1e3:.2f} ms, "
                      f"std: {s.latency_std*1e3:.2f} ms, "
                      f"p90: {s.latency_p90*1e3:.2f} ms")
        if stats.group_num_requests is not None:
            print(f"per group #req: {stats.group_num_requests}")
        print("--- overall ---")
        print(f"total #req: {stats.num_requests}, "
              f"rate: {stats.request_rate:.2f} q/s")
        print(f"average goodput: {stats.goodput*100:.2f} %, "
              f"latency mean: {stats.latency_mean*1e3:.2f} ms")

    def __str__(self):
        return (f"Workload(len={len(self)}, rate={self.rate:.2f}, "
                f"CV={self.cv:.2f}, "
                f"tstamps={to_str_round(self.arrivals[:20])} ...)")
