"""Placement data types, the batched placement evaluator and the search
primitives built on it.

Mirrors the reference's ``alpa_serve/placement_policy/base_policy.py``:
``ModelPlacement`` (:18-55), ``ModelPlacementWithReplacement`` (:58-68),
``ModelData`` (:71-77), ``ClusterEnv`` (:80-84), ``BasePlacementPolicy``
(:87-140), ``PlacementEvaluator`` (:143-264) and ``gen_train_workload``
(:267-281).  The evaluator is where this package differs in construction:
the reference scores a list of placements one at a time on the CPU, this one
hands the whole list to the GPU as one batch (one placement per lane).
"""
import dataclasses
import time
from functools import partial
from typing import List

import numpy as np

from mms_amd import _lib, engine as _engine
from mms_amd.profiling import ParallelConfig, ProfilingResult
from mms_amd.simulator.controller import approximate_one_case
from mms_amd.simulator.executable import Executable
from mms_amd.simulator.workload import (GammaProcess, PerModelStatsResult,
                                        StatsResult, Workload)
from mms_amd.util import ServingCase, eps, inf


@dataclasses.dataclass
class ModelPlacement:
    """Groups of devices and the models each group hosts."""
    group_configs: List[ParallelConfig]
    group_models: List[List[int]]

    def add_model(self, group_id: int, model_id: int):
        """New placement with ``model_id`` appended to group ``group_id``;
        the configs object is shared, the touched row is copied."""
        rows = list(self.group_models)
        rows[group_id] = list(rows[group_id]) + [model_id]
        return ModelPlacement(self.group_configs, rows)

    def normalize(self):
        """Canonical form: models sorted inside each group, groups ordered by
        their model tuple, everything as tuples (hashable).  The order of
        groups decides which replica wins a clock tie in the simulator, so
        the sort must be the stable sort on the model tuples (:29-35)."""
        rows = [tuple(sorted(ms)) for ms in self.group_models]
        order = sorted(range(len(self.group_configs)), key=rows.__getitem__)
        return ModelPlacement(tuple(self.group_configs[i] for i in order),
                              tuple(rows[i] for i in order))

    def copy(self):
        return ModelPlacement(list(self.group_configs), [list(ms) for ms in self.group_models])

    def verify(self, model_datas, cluster_env):
        """Asserts the memory budget of every group and that no group lists a
        model twice (:41-55)."""
        for cfg, ms in zip(self.group_configs, self.group_models):
            need = sum(weight_mem_of(model_datas[m], cfg) for m in ms)
            assert need <= cluster_env.mem_budget
        assert all(len(set(ms)) == len(ms) for ms in self.group_models)


def weight_mem_of(model_data, parallel_config):
    """Per-device weight memory of a model under a config: the largest stage;
    ``inf`` (1e100) when the model has no profile for it (:44-48)."""
    entry = model_data.profiling_result.para_dict.get(parallel_config)
    return max(entry.weight_mem) if entry is not None else inf


def weight_mem_table(group_configs, model_datas):
    """{config: [per-model weight memory]} for the configs in use (:299-305)."""
    return {c: [weight_mem_of(x, c) for x in model_datas] for c in group_configs}


@dataclasses.dataclass
class ModelPlacementWithReplacement:
    """Placements that replace one another at the given start times."""
    start_times: List[float]
    placements: List[ModelPlacement]

    def verify(self, model_datas, cluster_env):
        for p in self.placements:
            p.verify(model_datas, cluster_env)

    def __str__(self):
        return f"ModelPlacementWithReplacement(num_segments={len(self.placements)})"


@dataclasses.dataclass
class ModelData:
    name: str
    slo: float
    rate: float
    cv: float
    profiling_result: ProfilingResult


@dataclasses.dataclass
class ClusterEnv:
    num_devices: int
    mem_budget: float
    num_devices_per_node: int = 8


class BasePlacementPolicy:
    """Base class: subclasses implement ``solve_placement``."""

    def __init__(self, verbose: int = 0):
        self.verbose = verbose

    def place_models(self, controller, cluster_env: ClusterEnv, model_datas: List[ModelData],
                     train_workload: Workload = None):
        """Solve, apply to ``controller`` (if any), verify, return (:93-107)."""
        tic = time.time()
        placement, debug_info = self.solve_placement(model_datas, cluster_env, train_workload)
        solver_time = time.time() - tic

        self.place_models_impl(controller, cluster_env, model_datas, placement)

        if self.verbose >= 1:
            print(f"placement solution: {placement}")
            print(f"debug info: {debug_info}")
            print(f"solver time: {solver_time:.2f} s")

        placement.verify(model_datas, cluster_env)
        return placement

    def place_models_impl(self, controller, cluster_env: ClusterEnv, model_datas: List[ModelData],
                          placement: ModelPlacement):
        """Create one mesh group manager per group and one replica per hosted
        model through the controller's ``.remote`` methods (:109-140)."""
        if isinstance(placement, ModelPlacementWithReplacement):
            return
        group_configs, group_models = placement.group_configs, placement.group_models
        assert len(group_configs) == len(group_models)
        per_node = cluster_env.num_devices_per_node
        for g_id, cfg in enumerate(group_configs):
            n = np.prod(cfg)
            if n <= per_node:
                shape = (1, n)
            else:
                assert n % per_node == 0
                shape = (n // per_node, per_node)
            controller.create_mesh_group_manager.remote(g_id, shape)
        controller.sync()
        for g_id, cfg in enumerate(group_configs):
            for m_id in group_models[g_id]:
                controller.create_replica.remote(model_datas[m_id].name, g_id, [cfg])
        controller.sync()


class PlacementEvaluator:
    """Scores lists of placements with the approximate simulator.

    Same constructor and methods as the reference (:143-264).  ``get_scores``
    and ``get_stats`` send the whole list to the GPU in one batch; the
    request stream and the per-config latency table are uploaded once and
    reused across calls, which is what ``workload.cached_data`` does for the
    reference's per-placement loop (:155, :170, controller.py:323-339).

    ``method`` must be "fast_simulator": the event-driven simulator is not
    part of this package.  ``parallel`` selected one Ray task per placement
    in the reference; the GPU batch already evaluates placements in parallel,
    so the flag is accepted and has no effect.
    """

    def __init__(self, model_datas: List[ModelData], cluster_env: ClusterEnv, workload: Workload,
                 method: str, parallel: bool, enable_batching: bool = False):
        if method != "fast_simulator":
            raise NotImplementedError(
                f"evaluator method {method!r}: only 'fast_simulator' is available")
        self.parallel = parallel
        self.model_datas = model_datas
        self.cluster_env = cluster_env
        self.workload = workload
        self.method = method
        self.enable_batching = enable_batching

        workload.cached_data = None
        workload.enable_simulator_cache = True

        self._engine = None
        self._device_workload = None
        self._table = None

    # -- device-side state, created on first use --------------------------------
    def _prepare(self):
        if self._device_workload is not None:
            return
        from mms_amd.util import batchsize_config
        self._engine = _engine.Engine.default()
        wl = self.workload
        # model id = registration order = index in model_datas; a name registered
        # twice keeps its first position and its last profile (dict semantics of
        # DummyController.name2profiling, controller.py:290-296, :332-334)
        name2prof = {}
        for d in self.model_datas:
            name2prof[d.name] = d.profiling_result
        names = tuple(name2prof.keys())
        profs = tuple(name2prof.values())
        name2id = {n: i for i, n in enumerate(names)}
        model_ids = np.array([name2id.get(r.model_name, -1) for r in wl.requests], dtype=np.int32)
        slos = np.array([r.slo for r in wl.requests], dtype=np.float32)
        wl.cached_data = (model_ids, slos, names, profs)
        self._names = names
        self._num_requests_per_model = np.bincount(model_ids[model_ids >= 0], minlength=len(names))
        self._device_workload = _engine.DeviceWorkload(self._engine, wl.arrivals, model_ids, slos,
                                                       len(names))
        self._table = _engine.LatencyTable(
            profs, list(batchsize_config) if self.enable_batching else [1])

    def _run(self, sols, flags):
        self._prepare()
        if self.enable_batching:
            flags |= _lib.BATCHING
        return _engine.evaluate(self._engine, [self._device_workload], self._table, sols, flags)

    @staticmethod
    def _is_plain(sols):
        return all(isinstance(s, ModelPlacement) for s in sols)

    # -- public API ---------------------------------------------------------------
    def get_scores(self, sols: List[ModelPlacement]):
        """goodput - latency_mean/10000 + num_replicas/1e6 per placement (:225-226)."""
        if len(sols) == 0:
            return []
        if not self._is_plain(sols):
            return [self.get_goodput_simulation(s, self.model_datas, self.cluster_env,
                                                self.workload, self.method) for s in sols]
        out = self._run(sols, 0)
        R = len(self.workload)
        goodput = out["n_good"][0] / R
        latency_mean = out["latency_sum"][0] / R
        replicas = np.fromiter((sum(len(x) for x in s.group_models) for s in sols), np.int64, len(sols))
        scores = goodput - latency_mean / 10000 + replicas / 1000000
        return [float(x) for x in scores]

    def get_stats(self, sols: List[ModelPlacement]):
        """(goodput, per-model goodput, group_num_requests, StatsResult) per
        placement (:263-264) with the fast statistics of controller.py:393-403."""
        if len(sols) == 0:
            return []
        if not self._is_plain(sols):
            return [self.get_stats_simulation(s, self.model_datas, self.cluster_env,
                                              self.workload, self.method) for s in sols]
        out = self._run(sols, _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS)
        arrivals = self.workload.arrivals
        R = len(arrivals)
        interval = arrivals[-1] - arrivals[0]
        ret = []
        for b, sol in enumerate(sols):
            mreq = out["model_num_requests"][0, b]
            mgood = out["model_num_good"][0, b]
            greq = out["group_num_requests"][0, b, :len(sol.group_configs)]
            per_model = [PerModelStatsResult(
                self._names[i], mreq[i], mgood[i] / (mreq[i] + eps), mreq[i] / interval,
                0, 0, 0, 0, [], [], []) for i in range(len(self._names))]
            goodput = np.float64(out["n_good"][0, b]) / R
            latency_mean = out["latency_sum"][0, b] / R
            stats = StatsResult(per_model, tuple(greq), goodput, latency_mean, R, R / interval)
            ret.append((stats.goodput, [x.goodput for x in per_model], stats.group_num_requests, stats))
        return ret

    # -- one placement at a time, same signatures as the reference's static methods -----
    @staticmethod
    def _serving_case(sol, model_datas, workload, method):
        if method != "fast_simulator":
            raise NotImplementedError("only 'fast_simulator' is available")

        def register_models(controller):
            for data in model_datas:
                controller.register_model.remote(
                    data.name, partial(Executable, data.profiling_result))

        def generate_workload(start=0):
            return workload

        def place_models(controller):
            return sol

        return ServingCase(register_models, generate_workload, place_models)

    @staticmethod
    def get_goodput_simulation(sol, model_datas, cluster_env, workload, method):
        case = PlacementEvaluator._serving_case(sol, model_datas, workload, method)
        stats, _ = approximate_one_case(case, fast_stats=True)
        if isinstance(sol, ModelPlacement):
            num_replicas = sum(len(x) for x in sol.group_models)
        else:
            num_replicas = sum(len(x) for p in sol.placements for x in p.group_models)
        return stats.goodput - stats.latency_mean / 10000 + num_replicas / 1000000

    @staticmethod
    def get_stats_simulation(sol, model_datas, cluster_env, workload, method):
        case = PlacementEvaluator._serving_case(sol, model_datas, workload, method)
        stats, _ = approximate_one_case(case, fast_stats=True)
        return (stats.goodput, [x.goodput for x in stats.per_model_stats],
                stats.group_num_requests, stats)


def gen_train_workload(model_datas: List[ModelData], seed: int = 0,
                       simulation_min_duration: float = 100,
                       simulation_min_samples: int = 30000):
    """Gamma arrivals per model (seed + model index), merged; long enough for
    ``simulation_min_samples`` requests in total (:267-281)."""
    total_rate = sum(d.rate for d in model_datas)
    duration = max(simulation_min_duration, simulation_min_samples / total_rate)
    parts = [GammaProcess(d.rate, d.cv).generate_workload(d.name, 0, duration=duration, slo=d.slo,
                                                          seed=seed + i)
             for i, d in enumerate(model_datas)]
    return Workload.merge(*parts)
