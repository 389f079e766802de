"""Seeded synthetic inputs: the five benchmark configurations.

Everything here is input generation, shared by the tests, the smoke check and
``bench.py`` so that CPU oracle and GPU always see identical arrays:

* model profiles from a single-device latency ``L_m``
  (``profiling.synthetic_profile``);
* arrivals from ``GammaProcess(rate_m, cv)`` with legacy seed
  ``base_seed*1000 + m``, merged like ``Workload.merge`` (reference
  alpa_serve/simulator/workload.py:135-162, :381-401;
  ``gen_train_workload`` in placement_policy/base_policy.py:267-281 is the
  ``base_seed = 0`` case);
* candidate placements drawn from ``numpy.random.Generator(PCG64(seed))``.
  Draw order inside one placement: for each new group (until the devices are
  used up) first its size, then (config 4 only) its operator-parallel degree,
  then the number of hosted models, then the models (without replacement).
"""
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np

from mms_amd.profiling import ParallelConfig, synthetic_profile
from mms_amd.simulator.workload import GammaProcess, Request, Workload


def gamma_arrivals_fast(rate: float, cv: float, start: float, duration: float, seed: int) -> np.ndarray:
    """Same numbers as ``GammaProcess(rate, cv).generate_arrivals(start,
    duration, seed)`` (workload.py:135-155) without the per-arrival Python
    loop: ``np.cumsum`` accumulates left to right exactly like ``cur += gap``."""
    proc = GammaProcess(rate, cv)
    np.random.seed(seed)
    block = max(int(rate * duration * 1.2), 1)
    end = start + duration
    out = []
    carry = start
    while True:
        gaps = np.random.gamma(proc.shape, proc.scale, size=block)
        gaps[0] = carry + gaps[0]
        ticks = np.cumsum(gaps)
        # The reference draws the next block as soon as the last gap of a block
        # has been consumed, i.e. when every tick of this block lies before `end`.
        stop = int(np.searchsorted(ticks, end, side="left"))  # first index with tick >= end
        if stop < block:
            out.append(ticks[:stop])
            break
        out.append(ticks)
        carry = ticks[-1]
    return np.concatenate(out) if len(out) > 1 else out[0]


def power_law_rates(num_models: int, total: float, alpha: float) -> np.ndarray:
    w = np.arange(1, num_models + 1, dtype=np.float64) ** (-alpha)
    return total * w / w.sum()


@dataclass
class Stream:
    """One arrival seed of a configuration, as the arrays the simulator takes."""
    tstamps: np.ndarray      # float64 [R]
    model_ids: np.ndarray    # int32   [R]
    slos: np.ndarray         # float32 [R]


@dataclass
class SyntheticConfig:
    index: int
    name: str
    num_models: int
    num_devices: int
    latencies: np.ndarray            # L_m
    slo_scales: np.ndarray
    rates: np.ndarray
    cv: float
    duration: float
    base_seeds: Sequence[int]
    batching: bool
    batch_sizes: List[int]
    profiles: list = field(default_factory=list)       # ProfilingResult per model
    placements: list = field(default_factory=list)     # ModelPlacement candidates
    _streams: dict = field(default_factory=dict)

    @property
    def model_names(self):
        return [f"m{m}" for m in range(self.num_models)]

    @property
    def slos(self):
        return (self.slo_scales * self.latencies).astype(np.float64)

    def stream(self, base_seed: int) -> Stream:
        """Merged request stream of all models for one base seed."""
        if base_seed not in self._streams:
            per_model = [gamma_arrivals_fast(self.rates[m], self.cv, 0, self.duration,
                                             base_seed * 1000 + m) for m in range(self.num_models)]
            all_t = np.concatenate(per_model)
            all_m = np.concatenate([np.full(len(a), m, np.int32) for m, a in enumerate(per_model)])
            order = np.argsort(all_t)                 # same call as Workload.merge
            slo32 = self.slos.astype(np.float32)      # slos are stored as float32 (controller.py:336)
            self._streams[base_seed] = Stream(all_t[order], all_m[order], slo32[all_m[order]])
        return self._streams[base_seed]

    def workload(self, base_seed: int) -> Workload:
        """The same stream as a ``Workload`` of ``Request`` objects (small configs)."""
        parts = [GammaProcess(self.rates[m], self.cv).generate_workload(
            self.model_names[m], 0, self.duration, float(self.slos[m]), base_seed * 1000 + m)
            for m in range(self.num_models)]
        return Workload.merge(*parts)

    def model_datas(self):
        from mms_amd.placement_policy.base_policy import ModelData
        return [ModelData(self.model_names[m], float(self.slos[m]), float(self.rates[m]), self.cv,
                          self.profiles[m]) for m in range(self.num_models)]


def _random_partition(rng, num_devices, sizes):
    out = []
    left = num_devices
    while left > 0:
        out.append(int(rng.choice([s for s in sizes if s <= left])))
        left -= out[-1]
    return out


def _random_placement(rng, num_models, num_devices, sizes, k_lo, k_hi, op_choices=None):
    from mms_amd.placement_policy.base_policy import ModelPlacement
    cfgs, models = [], []
    left = num_devices
    while left > 0:
        size = int(rng.choice([s for s in sizes if s <= left]))
        left -= size
        op = 1
        if op_choices:
            op = int(rng.choice([o for o in op_choices if size % o == 0 and size // o >= 1]))
        k = int(rng.integers(k_lo, k_hi + 1))
        ms = rng.choice(num_models, size=min(k, num_models), replace=False)
        cfgs.append(ParallelConfig(1, op, size // op))
        models.append([int(m) for m in ms])
    return ModelPlacement(cfgs, models)


def _all_configs(sizes, op_choices=(1,)):
    return sorted({ParallelConfig(1, o, s // o) for s in sizes for o in op_choices
                   if s % o == 0 and s // o >= 1})


def make_config(index: int, num_placements: Optional[int] = None) -> SyntheticConfig:
    """Configuration ``index`` in 1..5; ``num_placements`` truncates the
    candidate list (candidate c is drawn from its own generator, so a prefix
    of the list is the same placements)."""
    from mms_amd.placement_policy.base_policy import ModelPlacement
    if index == 1:
        M, D = 8, 8
        cfg = SyntheticConfig(1, "cfg1-sanity", M, D, np.full(M, 0.10), np.full(M, 5.0),
                              np.full(M, 2.5), 1.0, 60.0, [0], False, [1])
        pcs = [ParallelConfig(1, 1, 4)]
        cfg.placements = [ModelPlacement([ParallelConfig(1, 1, 4)] * 2, [list(range(M))] * 2)]
    elif index == 2:
        M, D = 32, 16
        lat = np.random.Generator(np.random.PCG64(2)).uniform(0.05, 0.4, M)
        cfg = SyntheticConfig(2, "cfg2-random64", M, D, lat, np.full(M, 5.0), np.full(M, 1.0), 4.0,
                              300.0, [0, 1, 2, 3], False, [1])
        sizes = (1, 2, 4, 8)
        pcs = _all_configs(sizes)
        n = 64 if num_placements is None else num_placements
        cfg.placements = [_random_placement(np.random.Generator(np.random.PCG64(2000 + c)),
                                            M, D, sizes, 2, 6) for c in range(n)]
    elif index == 3:
        M, D = 64, 32
        lat = np.random.Generator(np.random.PCG64(3)).uniform(0.05, 0.4, M)
        cfg = SyntheticConfig(3, "cfg3-greedy-sr-step", M, D, lat, np.full(M, 8.0),
                              power_law_rates(M, 200.0, 0.5), 2.0, 600.0, [0], False, [1])
        pcs = [ParallelConfig(1, 1, 1)]
        sols = []
        for b in (0, 1):
            base = [[g, g + 32, (g + 1 + b) % 64] for g in range(D)]
            for g in range(D):
                for m in range(M):
                    rows = [list(r) for r in base]
                    rows[g].append(m)
                    sols.append(ModelPlacement([ParallelConfig(1, 1, 1)] * D, rows))
        cfg.placements = sols if num_placements is None else sols[:num_placements]
    elif index == 4:
        M, D = 128, 64
        lat = np.random.Generator(np.random.PCG64(4)).uniform(0.05, 0.4, M)
        cfg = SyntheticConfig(4, "cfg4-large-burst", M, D, lat, np.full(M, 5.0),
                              power_law_rates(M, 1000.0, 1.0), 8.0, 1000.0, list(range(8)), False, [1])
        sizes, ops = (2, 4, 8, 16), (1, 2, 4)
        pcs = _all_configs(sizes, ops)
        n = 16384 if num_placements is None else num_placements
        cfg.placements = [_random_placement(np.random.Generator(np.random.PCG64(4000 + c)),
                                            M, D, sizes, 8, 24, ops) for c in range(n)]
    elif index == 5:
        M, D = 96, 48
        tier = np.array([0.06] * 4 + [0.12] * 3 + [0.25] * 2 + [0.5])
        lat = tier[np.arange(M) % 10]
        scales = np.random.Generator(np.random.PCG64(5)).choice([2.0, 5.0, 10.0], size=M)
        cfg = SyntheticConfig(5, "cfg5-batching", M, D, lat, scales, power_law_rates(M, 500.0, 0.8),
                              6.0, 1200.0, [0, 1, 2, 3], True, [1, 2, 4, 8])
        sizes = (1, 2, 4, 8)
        pcs = _all_configs(sizes)
        n = 8192 if num_placements is None else num_placements
        cfg.placements = [_random_placement(np.random.Generator(np.random.PCG64(5000 + c)),
                                            M, D, sizes, 4, 12) for c in range(n)]
    else:
        raise ValueError("config index must be 1..5")

    comm = 0.002 if index == 4 else 0.0
    slope = 0.15 if index == 5 else 0.0
    cfg.profiles = [synthetic_profile(cfg.model_names[m], float(cfg.latencies[m]), pcs,
                                      batch_sizes=cfg.batch_sizes, batch_slope=slope,
                                      stage_comm=comm) for m in range(cfg.num_models)]
    return cfg
