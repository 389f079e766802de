"""Latency/memory profiles of models under a 3-D parallel configuration.

These are the containers the simulator's table build reads
(reference ``alpa_serve/profiling.py``: ``ParallelConfig`` :14,
``LatencyMemData`` :16-41, ``ProfilingResult`` :44-68) plus the canned
test profiles of ``load_test_prof_result`` (:196-357), which the reference's
placement-policy tests use as fixtures.  The pickle/CSV ``ProfilingDatabase``
(:71-193) is an offline artefact store and is not part of the evaluated path.
"""
from collections import namedtuple
import dataclasses
from typing import Any, Dict, List, Sequence

from mms_amd.util import GB

# (data parallel, operator parallel, pipeline parallel); hashable dict key.
ParallelConfig = namedtuple("ParallelConfig", ("dp", "op", "pp"))


@dataclasses.dataclass
class LatencyMemData:
    """Per-stage latency and memory of one model under one ParallelConfig.

    latency:    {batch_size: [seconds per pipeline stage]}
    act_mem:    {batch_size: [activation bytes per stage]}
    weight_mem: [weight bytes per stage]
    """
    latency: Dict
    act_mem: Dict
    weight_mem: List
    metadata: Any = None

    def add_result(self, batch_size: int, latency: List[float],
                   act_mem: List[float], weight_mem: List[float],
                   metadata: Any = None):
        """Record a measurement; for a batch size already present keep the
        one with the smaller bottleneck stage (profiling.py:30-41)."""
        known = self.latency.get(batch_size)
        if known is None:
            self.latency[batch_size] = latency
            self.act_mem[batch_size] = act_mem
        elif max(latency) < max(known):
            self.latency[batch_size] = latency
            self.act_mem[batch_size] = act_mem
            self.weight_mem = weight_mem
            self.metadata = metadata


@dataclasses.dataclass
class ProfilingResult:
    """All profiled configurations of one model (profiling.py:44-68)."""
    model_name: str
    para_dict: Dict            # {ParallelConfig: LatencyMemData}
    preprocess_cpu: float
    postprocess_cpu: float

    def add_result(self, parallel_config: ParallelConfig, batch_size: int,
                   stage_latency: List[float], act_mem: List[float],
                   weight_mem: List[float], metadata: Any = None):
        entry = self.para_dict.get(parallel_config)
        if entry is None:
            self.para_dict[parallel_config] = LatencyMemData(
                latency={batch_size: stage_latency},
                act_mem={batch_size: act_mem},
                weight_mem=weight_mem, metadata=metadata)
        else:
            entry.add_result(batch_size, stage_latency, act_mem, weight_mem,
                             metadata)


def _profile(name: str, rows: Sequence) -> ProfilingResult:
    """rows: (pp, [batch-1 stage latencies], [stage weight GiB])."""
    para = {}
    for pp, lat, mem_gb in rows:
        assert len(lat) == pp and len(mem_gb) == pp
        para[ParallelConfig(1, 1, pp)] = LatencyMemData(
            latency={1: list(lat)},
            act_mem={1: ["TODO"] * pp},
            weight_mem=[g * GB for g in mem_gb])
    return ProfilingResult(name, para_dict=para, preprocess_cpu=0,
                           postprocess_cpu=0)


# Canned profiles, values as in the reference's load_test_prof_result
# (profiling.py:196-357).  Only pipeline-parallel configs (dp=op=1).
_TEST_PROFILES = {
    "alpa/bert-1.3b": [
        (1, [0.099], [2.6]),
        (2, [0.051, 0.052], [1.3] * 2),
        (4, [0.028, 0.027, 0.027, 0.029], [0.65] * 4),
        (8, [0.015] + [0.014] * 6 + [0.016], [0.325] * 8),
    ],
    "alpa/bert-2.6b": [
        (1, [0.148], [5.2]),
        (2, [0.075, 0.076], [2.6] * 2),
    ],
    "test-2GB-100ms": [
        (1, [0.100], [2]),
        (2, [0.051] * 2, [1] * 2),
        (4, [0.026] * 4, [0.5] * 4),
    ],
    "test-4GB-150ms": [
        (1, [0.150], [4]),
        (2, [0.076] * 2, [2] * 2),
        (4, [0.039] * 4, [1] * 4),
    ],
}


def load_test_prof_result(name: str) -> ProfilingResult:
    """Pre-defined profiles for tests (profiling.py:196-357)."""
    rows = _TEST_PROFILES.get(name)
    if rows is None:
        raise ValueError(f"Unsupported model: {name}")
    return _profile(name, rows)


def synthetic_profile(name: str, base_latency: float,
                      configs: Sequence[ParallelConfig],
                      batch_sizes: Sequence[int] = (1,),
                      batch_slope: float = 0.0,
                      pp_overhead: float = 1.05,
                      stage_comm: float = 0.0,
                      weight_bytes: float = 1 * GB) -> ProfilingResult:
    """Profile generated from a single-device batch-1 latency.

    Stage latency of a pp-stage pipeline is ``L(b)`` for pp == 1, else
    ``L(b)/pp * pp_overhead + stage_comm`` with ``L(b) = base*(1+slope*(b-1))``.
    Weights are split evenly over op*pp devices.  This is the benchmark's
    input convention, not something the reference ships.
    """
    para = {}
    for cfg in configs:
        lat = {}
        for b in batch_sizes:
            full = base_latency * (1 + batch_slope * (b - 1))
            stage = full if cfg.pp == 1 else full / cfg.pp * pp_overhead + stage_comm
            lat[b] = [stage] * cfg.pp
        para[cfg] = LatencyMemData(
            latency=lat, act_mem={b: [0.0] * cfg.pp for b in batch_sizes},
            weight_mem=[weight_bytes / (cfg.op * cfg.pp)] * cfg.pp)
    return ProfilingResult(name, para_dict=para, preprocess_cpu=0,
                           postprocess_cpu=0)
