"""The approximate serving simulator, evaluated on the GPU.

Drop-in for the fast-simulator half of the reference's
``alpa_serve/simulator/controller.py``: ``DummyController`` (:282-305),
``approximate_one_case`` (:308-407) and
``approximate_one_case_one_placement`` (:410-503).  The request loops the
reference JIT-compiles with numba (:561-628, :631-798) run as HIP kernels
behind ``libmmsim``; nothing here computes a simulation on the CPU.

The event-driven simulator of the same reference file (``Controller``,
``GroupManager``, ``Client``, ``simulate_one_case``, :30-279) is a different,
slow path and is not provided.
"""
from functools import partial
from typing import Callable

import numpy as np

from mms_amd import _lib, engine as _engine
from mms_amd.profiling import ProfilingResult
from mms_amd.simulator.workload import (DEFAULT_WARMUP, PerModelStatsResult,
                                        StatsResult, Workload)
from mms_amd.util import ServingCase, batchsize_config, eps, inf


def install_remote_methods(obj):
    """Give every public method a ``.remote`` alias of itself, so code written
    against Ray actor handles can drive a plain object
    (reference simulator/util.py:9-16)."""
    for key in dir(obj):
        value = getattr(obj, key)
        if callable(value) and not key.startswith("_"):
            wrapped = partial(value)
            wrapped.remote = wrapped
            setattr(obj, key, wrapped)


class DummyController:
    """Collects name -> ProfilingResult from ``register_model`` calls and
    ignores everything else (controller.py:282-305)."""

    def __init__(self):
        self.name2profiling = {}
        install_remote_methods(self)

    def register_model(self, name: str, model_def: Callable):
        assert isinstance(model_def, partial)
        for a in model_def.args:
            if isinstance(a, ProfilingResult):
                self.name2profiling[name] = a
                break

    def create_mesh_group_manager(self, *args, **kwargs):
        pass

    def create_replica(self, *args, **kwargs):
        pass

    def sync(self):
        pass


def _placement_to_replica_table(placement, num_models):
    """m_id2g_id of controller.py:418-422: groups hosting each model, ascending."""
    group_models = placement.group_models
    num_groups = len(placement.group_configs)
    m_id2g_id = np.full((num_models, max(num_groups, 1)), -1, dtype=np.int32)
    fill = [0] * num_models
    for g_id, m_ids in enumerate(group_models):
        for m_id in m_ids:
            m_id2g_id[m_id][fill[m_id]] = g_id
            fill[m_id] += 1
    return m_id2g_id


def approximate_one_case_one_placement(placement, model_names, prof_ress, model_ids, slos,
                                       arrivals, mixed=True, enable_batching=False):
    """Simulate one placement on one request stream; returns
    ``(start, finish, good, model_num_requests, model_num_good_requests,
    group_num_requests, group_num_good_requests)`` as controller.py:410-503.

    The stage-latency table follows :467-476 (and :451-461 with batching); the
    request loop runs on the GPU through the C ABI's single-placement calls.
    """
    eng = _engine.Engine.default()
    group_configs = placement.group_configs
    num_groups = len(group_configs)
    num_models = len(model_names)
    if num_groups == 0:
        raise ValueError("placement has no groups")   # np.max([]) in the reference (:465)
    arrivals = np.asarray(arrivals, dtype=np.float64)
    num_requests = len(arrivals)
    m_id2g_id = _placement_to_replica_table(placement, num_models)
    if not mixed:
        # one clock per group: largest and summed stage latency of every (model, group), with the
        # pipeline penalty, rounded to float32 on assignment (:433-443, :496-499)
        group_max_latency = np.empty((num_models, num_groups), dtype=np.float32)
        group_sum_latency = np.empty((num_models, num_groups), dtype=np.float32)
        for m_id in range(num_models):
            for g_id in range(num_groups):
                value = prof_ress[m_id].para_dict.get(group_configs[g_id], None)
                if value:
                    penalty = 0.009 * len(value.latency[1])
                    group_max_latency[m_id][g_id] = max(value.latency[1]) * (1 + penalty)
                    group_sum_latency[m_id][g_id] = sum(value.latency[1]) * (1 + penalty)
                else:
                    group_max_latency[m_id][g_id] = group_sum_latency[m_id][g_id] = np.inf
        finish = np.empty(num_requests, dtype=np.float64)
        good = np.empty(num_requests, dtype=bool)
        counts = _engine.simulate_requests(eng, finish, good, arrivals, model_ids, slos, m_id2g_id,
                                           group_max_latency, group_sum_latency, num_requests)
        return (arrivals, finish, good) + tuple(counts)
    num_stages = np.array([c.pp for c in group_configs], dtype=np.int32)
    max_num_stages = int(np.max(num_stages))
    batch_sizes = list(batchsize_config) if enable_batching else [1]

    table = _engine.LatencyTable(prof_ress, batch_sizes)
    cols = [table.config_id(c) for c in group_configs]
    lat, _ = table.arrays()                       # [M][C][Smax][NB]
    stage_latency = np.ascontiguousarray(lat[:, cols, :max_num_stages, :])

    start = arrivals
    finish = np.empty(num_requests, dtype=np.float64)
    good = np.empty(num_requests, dtype=bool)
    if enable_batching:
        g_id2m_id = np.full((num_groups, num_models), -1, dtype=np.int32)
        fill = [0] * num_groups
        for m_id, g_ids in enumerate(m_id2g_id):          # :424-430
            for g_id in g_ids:
                if g_id >= 0:
                    g_id2m_id[g_id][fill[g_id]] = m_id
                    fill[g_id] += 1
        counts = _engine.simulate_requests_mixed_batching(
            eng, finish, good, arrivals, model_ids, slos, m_id2g_id, g_id2m_id, num_stages,
            stage_latency, batch_sizes, num_requests)
    else:
        counts = _engine.simulate_requests_mixed(
            eng, finish, good, arrivals, model_ids, slos, m_id2g_id, num_stages,
            stage_latency[..., 0], num_requests)
    return (start, finish, good) + tuple(counts)


def approximate_one_case(case: ServingCase, seed: int = 0, warmup: int = DEFAULT_WARMUP,
                         debug: bool = False, fast_stats: bool = False,
                         enable_batching: bool = False):
    """Score one serving case with the approximate simulator
    (controller.py:308-407).  ``seed`` and ``debug`` are accepted and unused,
    as in the reference; ``warmup`` only matters when ``fast_stats`` is off."""
    from mms_amd.placement_policy.base_policy import (ModelPlacement,
                                                      ModelPlacementWithReplacement)

    register_models, generate_workload, place_models = case
    workload = generate_workload()

    if workload.enable_simulator_cache and workload.cached_data:
        model_ids, slos, model_names, prof_ress = workload.cached_data
        placement = place_models(None)
    else:
        controller = DummyController()
        register_models(controller)
        placement = place_models(controller)
        # model id == registration order (:331-334)
        model_names, prof_ress = zip(*controller.name2profiling.items())
        name2id = {name: i for i, name in enumerate(model_names)}
        model_ids = np.array([name2id.get(r.model_name, -1) for r in workload.requests],
                             dtype=np.int32)
        slos = np.array([r.slo for r in workload.requests], dtype=np.float32)
        if workload.enable_simulator_cache:
            workload.cached_data = (model_ids, slos, model_names, prof_ress)

    arrivals = workload.arrivals
    if isinstance(placement, ModelPlacement):
        (start, finish, good, model_num_requests, model_num_good_requests,
         group_num_requests, group_num_good_requests) = approximate_one_case_one_placement(
             placement, model_names, prof_ress, model_ids, slos, arrivals,
             enable_batching=enable_batching)
    elif isinstance(placement, ModelPlacementWithReplacement):
        # A new segment starts at the first arrival strictly later than the next
        # change time; every segment starts from idle clocks (:345-391).
        change_times = list(placement.start_times[1:]) + [inf]
        cuts = [0]
        pt = 0
        for i in range(len(arrivals)):
            if arrivals[i] > change_times[pt]:
                cuts.append(i)
                pt += 1
        cuts.append(len(arrivals))
        pieces = []
        for seg, (lo, hi) in enumerate(zip(cuts[:-1], cuts[1:])):
            pieces.append(approximate_one_case_one_placement(
                placement.placements[seg], model_names, prof_ress, model_ids[lo:hi],
                slos[lo:hi], arrivals[lo:hi], enable_batching=enable_batching))
        start = np.concatenate([p[0] for p in pieces])
        finish = np.concatenate([p[1] for p in pieces])
        good = np.concatenate([p[2] for p in pieces])
        model_num_requests = np.sum([p[3] for p in pieces], axis=0)
        model_num_good_requests = np.sum([p[4] for p in pieces], axis=0)
        group_num_requests = np.sum([p[5] for p in pieces], axis=0)
        group_num_good_requests = np.sum([p[6] for p in pieces], axis=0)
    else:
        raise TypeError(f"unsupported placement type: {type(placement)}")

    if fast_stats:
        stats = fast_stats_result(model_names, start, finish, good, model_num_requests,
                                  model_num_good_requests, group_num_requests)
    else:
        stats = workload.compute_stats(start, finish, good, warmup)
        stats.group_num_requests = tuple(group_num_requests)
    return stats, placement


def fast_stats_result(model_names, start, finish, good, model_num_requests,
                      model_num_good_requests, group_num_requests):
    """The no-warmup statistics of controller.py:393-403."""
    interval = start[-1] - start[0]
    per_model = [PerModelStatsResult(
        model_names[i], model_num_requests[i],
        model_num_good_requests[i] / (model_num_requests[i] + eps),
        model_num_requests[i] / interval, 0, 0, 0, 0, [], [], [])
        for i in range(len(model_names))]
    return StatsResult(per_model, tuple(group_num_requests), np.mean(good),
                       np.mean(finish - start), len(start), len(start) / interval)
