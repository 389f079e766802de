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
from typing import List, Optional

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
        out = ModelPlacement(tuple(self.group_configs[i] for i in order),
                             tuple(rows[i] for i in order))
        out._canonical = True  # not a field: lets add_model_normalized skip the sorts that change nothing
        return out

    def add_model_normalized(self, group_id: int, model_id: int):
        """``add_model(group_id, model_id).normalize()``; cheaper when this placement is already in
        canonical form (only the touched row is re-sorted)."""
        if not getattr(self, "_canonical", False):
            return self.add_model(group_id, model_id).normalize()
        rows = list(self.group_models)
        rows[group_id] = tuple(sorted(rows[group_id] + (model_id,)))
        order = sorted(range(len(rows)), key=rows.__getitem__)
        cfgs = self.group_configs
        out = ModelPlacement(tuple([cfgs[i] for i in order]), tuple([rows[i] for i in order]))
        out._canonical = True
        return out

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


class _PerModelFastStats:
    """The ``per_model_stats`` list of the fast statistics (controller.py:397-400), its
    ``PerModelStatsResult`` entries made when they are read: a search that scores a thousand
    placements per call reads the entries of the few it goes on with."""

    def __init__(self, names, num_requests, goodputs, interval):
        self._names, self._req, self._goodputs, self._interval = names, num_requests, goodputs, interval

    def __len__(self):
        return len(self._names)

    def _entry(self, i):
        req = self._req[i]
        return PerModelStatsResult(self._names[i], req, self._goodputs[i], req / self._interval,
                                   0, 0, 0, 0, [], [], [])

    def __getitem__(self, key):
        if isinstance(key, slice):
            return [self._entry(i) for i in range(*key.indices(len(self)))]
        if key < 0:
            key += len(self)
        if not 0 <= key < len(self):
            raise IndexError(key)
        return self._entry(key)

    def __iter__(self):
        return (self._entry(i) for i in range(len(self)))

    def __eq__(self, other):
        return list(self) == list(other)

    def __repr__(self):
        return repr(list(self))


class PlacementEvaluator:
    """Scores lists of placements with the approximate simulator.

    Same constructor and methods as the reference (:143-264).  ``get_scores``
    and ``get_stats`` send the whole list to the GPU in one batch; the
    request stream and the per-config latency table are uploaded once and
    reused across calls, which is what ``workload.cached_data`` does for the
    reference's per-placement loop (:155, :170, controller.py:323-339).

    ``method`` "fast_simulator" is the GPU path.  Any other method is, as in the
    reference (:172-174, :199-224), the event-driven simulator
    (``mms_amd.simulator.event_sim``): host code, one placement after another,
    meant as a slower cross-check of a few placements, not for searches.
    ``parallel`` selected one Ray task per placement in the reference; the GPU
    batch already evaluates placements in parallel, so the flag is accepted and
    has no effect.
    """

    def __init__(self, model_datas: List[ModelData], cluster_env: ClusterEnv, workload: Workload,
                 method: str, parallel: bool, enable_batching: bool = False):
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

    @staticmethod
    def _num_replicas(sol):
        if isinstance(sol, ModelPlacement):
            return sum(len(x) for x in sol.group_models)
        return sum(len(x) for p in sol.placements for x in p.group_models)

    def _mixed_stats(self, sols):
        """Fast statistics (controller.py:393-403) of a list that holds ModelPlacementWithReplacement
        entries: every segment of every entry (a plain placement being one segment over the whole
        workload) is a lane of one GPU launch (controller.py:345-391 evaluated as a batch)."""
        from mms_amd.simulator.controller import replacement_fast_stats, simulate_replacements
        self._prepare()
        wl = self.workload
        model_ids, slos, names, profs = wl.cached_data
        as_replacements = [s if isinstance(s, ModelPlacementWithReplacement)
                           else ModelPlacementWithReplacement([0], [s]) for s in sols]
        if not hasattr(self, "_segment_workloads"):
            self._segment_workloads = {}
        res = simulate_replacements(as_replacements, names, profs, model_ids, slos, wl.arrivals,
                                    _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS,
                                    enable_batching=self.enable_batching, table=self._table,
                                    workload_cache=self._segment_workloads)
        return [replacement_fast_stats(names, wl.arrivals, r) for r in res]

    # -- public API ---------------------------------------------------------------
    def get_scores(self, sols: List[ModelPlacement]):
        """goodput - latency_mean/10000 + num_replicas/1e6 per placement (:225-226)."""
        if len(sols) == 0:
            return []
        if self.method != "fast_simulator":
            return [self.get_goodput_simulation(sol, self.model_datas, self.cluster_env, self.workload, self.method)
                    for sol in sols]
        if not self._is_plain(sols):
            return [st.goodput - st.latency_mean / 10000 + self._num_replicas(sol) / 1000000
                    for sol, st in zip(sols, self._mixed_stats(sols))]
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
        if self.method != "fast_simulator":
            return [self.get_stats_simulation(sol, self.model_datas, self.cluster_env, self.workload, self.method)
                    for sol in sols]
        if not self._is_plain(sols):
            return [(st.goodput, [x.goodput for x in st.per_model_stats], st.group_num_requests, st)
                    for st in self._mixed_stats(sols)]
        stats_of = self.get_stats_lazy(sols)
        return [stats_of(b) for b in range(len(sols))]

    def get_stats_lazy(self, sols: List[ModelPlacement], successors=None):
        """One batch for all of ``sols`` like ``get_stats``; returns a function
        that builds the ``get_stats`` entry of placement ``b`` when asked.  For
        callers that evaluate more placements than they will read (the look-ahead
        of the greedy search).  Plain placements and the fast simulator only.

        ``successors`` = (parent, group, model) index lists: the batch then also holds,
        behind ``sols``, the placements ``sols[parent[k]].add_model(group[k],
        model[k]).normalize()``, built inside the library (``mmsim_eval_successors``)
        instead of as Python objects; entry ``len(sols) + k`` is successor k."""
        assert self.method == "fast_simulator" and self._is_plain(sols)
        flags = _lib.WANT_MODEL_COUNTS | _lib.WANT_GROUP_COUNTS
        num_groups = [len(s.group_configs) for s in sols]
        if successors is None or len(successors[0]) == 0:
            out = self._run(sols, flags)
        else:
            self._prepare()
            parent, group, model = successors
            out = _engine.evaluate_successors(self._engine, [self._device_workload], self._table, sols, parent, group,
                                              model, flags | (_lib.BATCHING if self.enable_batching else 0))
            num_groups = num_groups + [num_groups[p] for p in parent]
        arrivals = self.workload.arrivals
        R = len(arrivals)
        interval = arrivals[-1] - arrivals[0]
        # per-model goodput of every placement at once: good / (requests + eps), the division of controller.py:399
        model_goodput = out["model_num_good"][0] / (out["model_num_requests"][0] + eps)
        goodputs = out["n_good"][0].astype(np.float64) / R
        latency_means = out["latency_sum"][0] / R

        def stats_of(b):
            greq = out["group_num_requests"][0, b, :num_groups[b]]
            per_model_goodput = list(model_goodput[b])
            per_model = _PerModelFastStats(self._names, out["model_num_requests"][0, b], per_model_goodput, interval)
            stats = StatsResult(per_model, tuple(greq), goodputs[b], latency_means[b], R, R / interval)
            return (stats.goodput, per_model_goodput, stats.group_num_requests, stats)
        return stats_of

    # -- one placement at a time, same signatures as the reference's static methods -----
    @staticmethod
    def _serving_case(sol, model_datas, cluster_env, workload, method):
        def register_models(controller):
            for data in model_datas:
                controller.register_model.remote(
                    data.name, partial(Executable, data.profiling_result))

        def generate_workload(start=0):
            return workload

        def place_models(controller):
            if method == "fast_simulator":
                return sol
            # the event-driven simulator builds the groups and replicas on its controller (:216-218)
            BasePlacementPolicy().place_models_impl(controller, cluster_env, model_datas, sol)

        return ServingCase(register_models, generate_workload, place_models)

    @staticmethod
    def _one_case(sol, model_datas, cluster_env, workload, method):
        case = PlacementEvaluator._serving_case(sol, model_datas, cluster_env, workload, method)
        if method == "fast_simulator":
            return approximate_one_case(case, fast_stats=True)[0]
        from mms_amd.simulator.event_sim import simulate_one_case
        return simulate_one_case(case)[0]

    @staticmethod
    def get_goodput_simulation(sol, model_datas, cluster_env, workload, method):
        stats = PlacementEvaluator._one_case(sol, model_datas, cluster_env, workload, method)
        if isinstance(sol, ModelPlacement):
            num_replicas = sum(len(x) for x in sol.group_models)
        else:
            num_replicas = sum(len(x) for p in sol.placements for x in p.group_models)
        return stats.goodput - stats.latency_mean / 10000 + num_replicas / 1000000

    @staticmethod
    def get_stats_simulation(sol, model_datas, cluster_env, workload, method):
        stats = PlacementEvaluator._one_case(sol, model_datas, cluster_env, workload, method)
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


# ----------------------------------------------------------------------------------------
# Search primitives.  They only differ from the reference in what sits behind
# evaluator.get_scores / get_stats; the order of candidates, the tie-breaking
# (np.argsort / np.argmax on the returned lists) and the use of numpy's global
# random generator follow base_policy.py:284-796 so that a search explores the
# same candidates in the same order.
# ----------------------------------------------------------------------------------------

def _group_memory(sol, weight_mem):
    return [sum(weight_mem[c][m] for m in ms) for c, ms in zip(sol.group_configs, sol.group_models)]


def replica_placement_round_robin(init_sol: ModelPlacement, model_datas: List[ModelData],
                                  cluster_env: ClusterEnv, workload: Workload, verbose: int):
    """Deal models to groups in turn while memory allows (:284-326)."""
    assert len(init_sol.group_configs) == len(init_sol.group_models)
    num_groups = len(init_sol.group_configs)
    weight_mem = weight_mem_table(init_sol.group_configs, model_datas)
    sol = init_sol
    group_mem = _group_memory(sol, weight_mem)
    g = 0
    progress = True
    while progress:
        progress = False
        for m in range(len(model_datas)):
            need = weight_mem[sol.group_configs[g]][m]
            if m not in sol.group_models[g] and need + group_mem[g] <= cluster_env.mem_budget:
                progress = True
                group_mem[g] += need
                sol = sol.add_model(g, m)
                sol.verify(model_datas, cluster_env)
                g = (g + 1) % num_groups
    return sol


def _fast_greedy_step(sol, stats, weight_mem, cluster_env):
    """One iteration of the greedy search (:339-372): the model with most unserved
    requests gets a replica on the least loaded group that still has memory for it.
    Returns the (group, model) to add or None when nothing fits."""
    overall_goodput, goodputs, group_num_requests, fullstats = stats
    unserved = [s.num_requests * (1 - gp) for s, gp in zip(fullstats.per_model_stats, goodputs)]
    model_order = np.argsort(unserved)[::-1]
    group_order = np.argsort(group_num_requests)
    group_mem = _group_memory(sol, weight_mem)
    for g_id in group_order:
        cfg = sol.group_configs[g_id]
        for m_id in model_order:
            if m_id not in sol.group_models[g_id] and \
                    weight_mem[cfg][m_id] + group_mem[g_id] <= cluster_env.mem_budget:
                return g_id, m_id
    return None


def replica_placement_fast_greedy(init_sol: ModelPlacement, model_datas: List[ModelData],
                                  cluster_env: ClusterEnv, workload: Workload,
                                  evaluator: PlacementEvaluator, verbose: int):
    """Repeatedly give the model with most unserved requests a replica on the
    least loaded group that still has memory for it (:329-400)."""
    return replica_placement_fast_greedy_lockstep([init_sol], model_datas, cluster_env, workload,
                                                  evaluator, verbose)[0]


def _fast_greedy_successors(sol, weight_mem, cluster_env):
    """Every (group, model) that ``_fast_greedy_step`` could return for ``sol``, whatever the statistics:
    the model is not on the group yet and fits beside what the group holds (the same sum as there)."""
    group_mem = _group_memory(sol, weight_mem)
    out = []
    for g_id, (cfg, hosted) in enumerate(zip(sol.group_configs, sol.group_models)):
        need = weight_mem[cfg]
        for m_id in range(len(need)):
            if m_id not in hosted and need[m_id] + group_mem[g_id] <= cluster_env.mem_budget:
                out.append((g_id, m_id))
    return out


# Most placements one evaluator call of the greedy search may hold when it looks ahead: up to this many,
# every placement is a lane of a wavefront that has a CU to itself, so the call takes as long as for one.
FAST_GREEDY_LOOKAHEAD_LANES = 16384
FAST_GREEDY_LOOKAHEAD = True  # what ``lookahead=None`` means (module switch for measurements)


def replica_placement_fast_greedy_lockstep(init_sols: List[ModelPlacement], model_datas: List[ModelData],
                                           cluster_env: ClusterEnv, workload: Workload,
                                           evaluator: PlacementEvaluator, verbose: int, lookahead: Optional[bool] = None):
    """``replica_placement_fast_greedy`` for several initial placements at once.

    The reference runs one greedy search per enumerated group layout, each
    scoring one placement per iteration (model_parallelism.py:341-344,
    :533-541).  The searches do not depend on each other, so they are advanced
    together: every iteration evaluates the current placement of every search
    that is still running in one evaluator call (one lane each on the GPU), and
    each search takes exactly the step it would take alone.

    A step needs the statistics of one placement, and a call for one placement
    takes the GPU as long as a call for thousands.  So with ``lookahead`` a
    call also evaluates every placement the step could lead to (current
    placement + one replica that fits); when the step is known, the statistics
    of the placement it leads to are already there and the next step is taken
    at once: two steps per call, each the step the search would take alone.
    Used while the call stays within ``FAST_GREEDY_LOOKAHEAD_LANES`` placements
    and the evaluator is the batched one.  Returns the final placements in the
    order of ``init_sols``."""
    tic = time.time()
    if evaluator is None:
        evaluator = PlacementEvaluator(model_datas, cluster_env, workload, "fast_simulator", False)
    sols = list(init_sols)
    weight_mems = [weight_mem_table(sol.group_configs, model_datas) for sol in sols]
    running = list(range(len(sols)))
    if lookahead is None:
        lookahead = FAST_GREEDY_LOOKAHEAD
    can_look = (lookahead and getattr(evaluator, "method", None) == "fast_simulator"
                and hasattr(evaluator, "get_stats_lazy"))
    it = 0
    while running:
        kids_of, kids_at = {}, {}
        look = can_look and all(isinstance(sols[i], ModelPlacement) for i in running)
        if look:
            for i in running:
                kids_of[i] = _fast_greedy_successors(sols[i], weight_mems[i], cluster_env)
            # (the batching simulator runs eight placements per wavefront instead of sixty-four)
            cap = FAST_GREEDY_LOOKAHEAD_LANES // (8 if getattr(evaluator, "enable_batching", False) else 1)
            look = len(running) + sum(len(k) for k in kids_of.values()) <= cap
        batch = [sols[i] for i in running]
        first = {i: at for at, i in enumerate(running)}
        if look:
            # the successors are named, not built: (parent, group, model) each; the library makes the placements
            parent, group, model = [], [], []
            for i in running:
                kids_at[i] = len(batch) + len(parent)
                parent += [first[i]] * len(kids_of[i])
                group += [g for g, _ in kids_of[i]]
                model += [m for _, m in kids_of[i]]
            stats_of = evaluator.get_stats_lazy(batch, (parent, group, model))
        else:
            all_stats = evaluator.get_stats(batch)
            stats_of = all_stats.__getitem__
        still = []
        for i in running:
            stats = stats_of(first[i])
            choice = _fast_greedy_step(sols[i], stats, weight_mems[i], cluster_env)
            if choice is None:
                continue
            sols[i] = sols[i].add_model(*choice).normalize()
            if verbose >= 2:
                print(f"iter: {it}, search: {i}, score: {stats[0]:.4f}, elapsed: {time.time() - tic:.2f}, "
                      f"best placement: {sols[i]}, ")
            if look and choice in kids_of[i]:
                stats = stats_of(kids_at[i] + kids_of[i].index(choice))
                choice = _fast_greedy_step(sols[i], stats, weight_mems[i], cluster_env)
                if choice is None:
                    continue
                sols[i] = sols[i].add_model(*choice).normalize()
                if verbose >= 2:
                    print(f"iter: {it}+, search: {i}, score: {stats[0]:.4f}, elapsed: {time.time() - tic:.2f}, "
                          f"best placement: {sols[i]}, ")
            still.append(i)
        running = still
        it += 1
    return sols


def _beam_loop(init_sol, evaluator, beam_size, verbose, expand, tic):
    """Common driver of the two beam searches: expand every beam member, score
    the new candidates in one batch, keep the top ``beam_size`` (:439-479)."""
    beam = [init_sol]
    best_score, best_sol = -1, init_sol
    visited = set()
    it = 0
    while True:
        next_sols = []
        for sol in beam:
            expand(sol, visited, next_sols)
        if not next_sols:
            break
        scores = evaluator.get_scores(next_sols)
        top = np.argsort(scores)[::-1][:beam_size]
        beam = []
        for idx in top:
            beam.append(next_sols[idx])
            if scores[idx] > best_score:
                best_score, best_sol = scores[idx], next_sols[idx]
        if verbose >= 1:
            print(f"iter: {it}, best score: {best_score:.4f}, iter score: {scores[top[0]]:.4f}, "
                  f"iter #sol: {len(next_sols)}, elapsed: {time.time() - tic:.2f}, "
                  f"best placement: {best_sol}, ")
        it += 1
    return best_sol


def replica_placement_beam_search(init_sol: ModelPlacement, model_datas: List[ModelData],
                                  cluster_env: ClusterEnv, workload: Workload,
                                  evaluator: PlacementEvaluator, beam_size: int, verbose: int):
    """Beam search over "add one replica" moves (:403-479).  Note the strict
    ``<`` against the memory budget here, unlike the greedy search."""
    tic = time.time()
    if evaluator is None:
        evaluator = PlacementEvaluator(model_datas, cluster_env, workload, "fast_simulator", False)
    num_models, num_groups = len(model_datas), len(init_sol.group_configs)
    weight_mem = weight_mem_table(init_sol.group_configs, model_datas)

    def expand(sol, visited, out):
        group_mem = _group_memory(sol, weight_mem)
        for g_id in range(num_groups):
            cfg = sol.group_configs[g_id]
            for m_id in range(num_models):
                if weight_mem[cfg][m_id] + group_mem[g_id] < cluster_env.mem_budget and \
                        m_id not in sol.group_models[g_id]:
                    cand = sol.add_model(g_id, m_id).normalize()
                    if cand.group_models not in visited:
                        visited.add(cand.group_models)
                        out.append(cand)

    return _beam_loop(init_sol, evaluator, beam_size, verbose, expand, tic)


def replica_placement_on_last_group(init_sol: ModelPlacement, model_datas: List[ModelData],
                                    cluster_env: ClusterEnv, workload: Workload,
                                    evaluator: PlacementEvaluator, beam_size: int, verbose: int):
    """Beam search that only fills the last group, also trying to swap the
    new model with one of an earlier group (:482-580)."""
    tic = time.time()
    if evaluator is None:
        evaluator = PlacementEvaluator(model_datas, cluster_env, workload, "fast_simulator", False)
    num_models, num_groups = len(model_datas), len(init_sol.group_configs)
    weight_mem = weight_mem_table(init_sol.group_configs, model_datas)
    last = num_groups - 1

    def expand(sol, visited, out):
        group_mem = _group_memory(sol, weight_mem)
        cfg = sol.group_configs[last]
        for m_id in range(num_models):
            if not (weight_mem[cfg][m_id] + group_mem[last] < cluster_env.mem_budget and
                    m_id not in sol.group_models[last]):
                continue
            cand = sol.add_model(last, m_id)
            key = cand.normalize().group_models
            if key in visited:
                continue
            visited.add(key)
            out.append(cand)
            at = list(cand.group_models[last]).index(m_id)
            for g2 in range(num_groups - 1):
                for at2 in range(len(cand.group_models[g2])):
                    if cand.group_models[last][at] in cand.group_models[g2] or \
                            cand.group_models[g2][at2] in cand.group_models[last]:
                        continue
                    rows = [list(x) for x in cand.group_models]
                    rows[last][at], rows[g2][at2] = rows[g2][at2], rows[last][at]
                    swapped = ModelPlacement(cand.group_configs, rows)
                    skey = swapped.normalize().group_models
                    if skey not in visited:
                        visited.add(skey)
                        out.append(swapped)

    return _beam_loop(init_sol, evaluator, beam_size, verbose, expand, tic)


def swap_two_models(sol: ModelPlacement):
    """Swap two random replicas of two random groups if that creates no duplicate (:583-595)."""
    rows = sol.group_models
    g1 = np.random.choice(len(rows))
    g2 = np.random.choice(len(rows))
    i1 = np.random.choice(len(rows[g1]))
    i2 = np.random.choice(len(rows[g2]))
    if rows[g1][i1] in rows[g2] or rows[g2][i2] in rows[g1]:
        return sol
    new_rows = [list(x) for x in rows]
    new_rows[g1][i1], new_rows[g2][i2] = new_rows[g2][i2], new_rows[g1][i1]
    return ModelPlacement(sol.group_configs, new_rows)


def swap_two_models_from_two_groups(sol: ModelPlacement, g_id_1, g_id_2):
    """As :598-608, including its two return shapes."""
    rows = sol.group_models
    i1 = np.random.choice(len(rows[g_id_1]))
    i2 = np.random.choice(len(rows[g_id_2]))
    if rows[g_id_1][i1] in rows[g_id_2] or rows[g_id_2][i2] in rows[g_id_1]:
        return False, sol
    new_rows = [list(x) for x in rows]
    new_rows[g_id_1][i1], new_rows[g_id_2][i2] = new_rows[g_id_2][i2], new_rows[g_id_1][i1]
    return ModelPlacement(sol.group_configs, new_rows)


def mutate_one_model(sol: ModelPlacement, num_models: int):
    """Replace one random replica by a random model (:611-620)."""
    rows = sol.group_models
    g = np.random.choice(len(rows))
    new_m = np.random.choice(num_models)
    if new_m in rows[g]:
        return sol
    i = np.random.choice(len(rows[g]))
    new_rows = [list(x) for x in rows]
    new_rows[g][i] = new_m
    return ModelPlacement(sol.group_configs, new_rows)


def fit_mem_budget(group_config, group_models, model_num_unserved, weight_mem, mem_budget):
    """In place: drop the least needed models until the group fits, then add
    the most needed ones while it still fits (:775-796)."""
    group_models.sort(key=lambda m: model_num_unserved[m])
    used = sum(weight_mem[group_config][m] for m in group_models)
    while used > mem_budget:
        used -= weight_mem[group_config][group_models[0]]
        del group_models[0]
    for m in reversed(np.argsort(model_num_unserved)):
        if m in group_models:
            continue
        if used + weight_mem[group_config][m] <= mem_budget:
            group_models.append(m)
            used += weight_mem[group_config][m]
            continue
        break


def merge_two_groups(group_configs, group_models, model_num_unserved, weight_mem, mem_budget):
    """In place: fuse two random groups of equal config into one of twice the
    pipeline depth (:720-743)."""
    for _ in range(10):
        g1 = np.random.choice(len(group_models))
        g2 = np.random.choice(len(group_models))
        if g1 != g2 and group_configs[g1] == group_configs[g2]:
            break
    else:
        return
    old = group_configs[g1]
    new_cfg = ParallelConfig(old.dp, old.op, old.pp * 2)
    if new_cfg not in weight_mem:
        return          # no model is profiled for the deeper pipeline (the reference raises KeyError here)
    merged = list(set(group_models[g1] + group_models[g2]))
    fit_mem_budget(new_cfg, merged, model_num_unserved, weight_mem, mem_budget)
    group_configs[g1] = new_cfg
    group_models[g1] = merged
    del group_configs[g2]
    del group_models[g2]


def split_one_group(group_configs, group_models, model_num_unserved, weight_mem, mem_budget):
    """In place: halve the pipeline depth of a random group with even depth
    and deal its models to the two halves (:746-772)."""
    for _ in range(10):
        g = np.random.choice(len(group_models))
        if group_configs[g].pp % 2 == 0:
            break
    else:
        return
    old = group_configs[g]
    new_cfg = ParallelConfig(old.dp, old.op, old.pp // 2)
    group_models[g].sort(key=lambda m: model_num_unserved[m])
    half_a, half_b = group_models[g][::2], group_models[g][1::2]
    fit_mem_budget(new_cfg, half_a, model_num_unserved, weight_mem, mem_budget)
    fit_mem_budget(new_cfg, half_b, model_num_unserved, weight_mem, mem_budget)
    group_configs[g] = new_cfg
    group_models[g] = half_a
    group_configs.append(new_cfg)
    group_models.append(half_b)


def _choice_cdf(p):
    """What ``np.random.choice(len(p), p=p)`` makes of ``p`` before it draws."""
    cdf = np.asarray(p, dtype=np.float64).cumsum()
    cdf /= cdf[-1]
    return cdf


def _weighted_choice(cdf):
    """``np.random.choice(len(p), p=p)`` with ``cdf = _choice_cdf(p)``: the same single draw from
    numpy's global generator and the same index, without re-validating ``p`` on every call."""
    return int(cdf.searchsorted(np.random.random_sample(), side="right"))


def evolutionary_search(init_sols: List[ModelPlacement], model_datas: List[ModelData],
                        cluster_env: ClusterEnv, evaluator: PlacementEvaluator, num_iter: int,
                        verbose: int):
    """Population search: sample parents by score, merge/split groups and
    mutate models toward the unserved ones, score the whole population in one
    batch per iteration (:623-717)."""
    tic = time.time()
    pop_size = 1024
    mutate_one_model_prob = 0.05
    merge_group_prob = 0.08
    split_group_prob = 0.08
    num_models = len(model_datas)
    mem_budget = cluster_env.mem_budget

    weight_mem = {}
    for m_id, x in enumerate(model_datas):
        for c, entry in x.profiling_result.para_dict.items():
            weight_mem.setdefault(c, [inf] * num_models)[m_id] = max(entry.weight_mem)

    best_score, best_sol = -1, None
    visited = set()
    cur_sols = init_sols
    # np.random.uniform() of the reference (:672-678) is 0.0 + 1.0 * random_sample(): the same draw and the same
    # value from numpy's global generator, at a tenth of the call cost (a child takes some fifty of them)
    uniform = np.random.random_sample
    for it in range(num_iter):
        stats = evaluator.get_stats(cur_sols)
        scores = np.array([x[0] for x in stats])
        weights = scores / np.sum(scores)
        parent_cdf = _choice_cdf(weights)
        unserved_cache = [None] * len(stats)

        top = np.argmax(scores)
        if scores[top] > best_score:
            best_score, best_sol = scores[top], cur_sols[top]

        next_sols = []
        while len(next_sols) < pop_size:
            idx = _weighted_choice(parent_cdf)      # np.random.choice(len(scores), p=weights)
            sol = cur_sols[idx]
            if unserved_cache[idx] is None:
                goodputs, fullstats = stats[idx][1], stats[idx][3]
                per_model = fullstats.per_model_stats
                if isinstance(per_model, _PerModelFastStats):   # the same products, without making the entries
                    raw = per_model._req * (1 - np.asarray(goodputs, dtype=np.float64))
                else:
                    raw = [s.num_requests * (1 - gp) for s, gp in zip(per_model, goodputs)]
                share = raw / np.sum(raw)
                unserved_cache[idx] = (share, _choice_cdf(share))
            unserved, unserved_cdf = unserved_cache[idx]

            group_configs = list(sol.group_configs)
            group_models = [list(x) for x in sol.group_models]
            if uniform() < merge_group_prob:
                merge_two_groups(group_configs, group_models, unserved, weight_mem, mem_budget)
            if uniform() < split_group_prob:
                split_one_group(group_configs, group_models, unserved, weight_mem, mem_budget)
            for g in range(len(group_models)):
                for i in range(len(group_models[g])):
                    if uniform() < mutate_one_model_prob:
                        new_m = _weighted_choice(unserved_cdf)      # np.random.choice(num_models, p=unserved)
                        if new_m not in group_models[g]:
                            group_models[g][i] = new_m
            child = ModelPlacement(group_configs, group_models).normalize()
            next_sols.append(child)
            visited.add(child.group_models)

        if verbose >= 1:
            print(f"iter: {it}, best score: {best_score:.4f}, iter avg-score: {np.mean(scores):.4f}, "
                  f"iter #sol: {len(scores)}, visited #sol: {len(visited)}, "
                  f"elapsed: {time.time() - tic:.2f}, best sol: {best_sol}, ")
        cur_sols = next_sols + [best_sol]
    return best_sol
