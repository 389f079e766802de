"""Placement policies that use model (pipeline / operator) parallelism.

Mirrors the simulator-driven policies of the reference's
``alpa_serve/placement_policy/model_parallelism.py``:
``ModelParallelismGreedy`` (:208-241), ``ModelParallelismRR`` (:258-291),
``ModelParallelismSearch`` (:294-547) and ``ModelParallelismEqual``
(:549-564).  ``ModelParallelismILP`` (:25-205) formulates an integer program
for the external ``pulp``/CBC solver and never calls the simulator; it is not
provided.
"""
import math
from typing import List, Tuple

import numpy as np

from mms_amd.placement_policy.base_policy import (
    BasePlacementPolicy, ClusterEnv, ModelData, ModelPlacement, PlacementEvaluator,
    evolutionary_search, gen_train_workload, replica_placement_fast_greedy,
    replica_placement_fast_greedy_lockstep, replica_placement_round_robin)
from mms_amd.profiling import ParallelConfig
from mms_amd.simulator.workload import Workload
from mms_amd.util import decompose2tok, get2tok, get_factors, get_partitions


class ModelParallelismILP(BasePlacementPolicy):
    def __init__(self, *args, **kwargs):
        raise NotImplementedError(
            "ModelParallelismILP needs the pulp/CBC integer-programming solver and does not "
            "use the placement simulator; it is outside this package")


class ModelParallelismGreedy(BasePlacementPolicy):
    """Equal groups of ``group_size`` devices (pp = group_size), filled greedily."""

    def __init__(self, group_size: int = 2, use_evo_search: bool = False, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.group_size = group_size
        self.use_evo_search = use_evo_search

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        if train_workload is None:
            train_workload = gen_train_workload(model_datas)
        evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload, "fast_simulator", False)
        assert cluster_env.num_devices % self.group_size == 0
        num_groups = cluster_env.num_devices // self.group_size
        sol = ModelPlacement([ParallelConfig(1, 1, self.group_size)] * num_groups,
                             [[] for _ in range(num_groups)])
        sol = replica_placement_fast_greedy(sol, model_datas, cluster_env, train_workload, evaluator,
                                            self.verbose)
        if self.use_evo_search:
            sol = evolutionary_search([sol], model_datas, cluster_env, evaluator, 200, self.verbose)
        return sol, None


class ModelParallelismRR(BasePlacementPolicy):
    """Groups of 4 pipeline stages (plus power-of-two leftovers), round robin."""

    def __init__(self, max_bs: int = 1, max_pp: int = 8, max_op: int = 4, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.max_bs, self.max_pp, self.max_op = max_bs, max_pp, max_op
        self.evaluator_method = "fast_simulator"

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        if train_workload is None:
            train_workload = gen_train_workload(model_datas)
        regular = cluster_env.num_devices // 4
        rest = decompose2tok(cluster_env.num_devices % 4)
        init_sol = ModelPlacement([ParallelConfig(1, 1, 4)] * regular + [ParallelConfig(1, 1, s) for s in rest],
                                  [[] for _ in range(regular + len(rest))])
        sol = replica_placement_round_robin(init_sol, model_datas, cluster_env, train_workload, self.verbose)
        return sol, {}


def solve_separation_placement(self, eco_separation: List[Tuple[List[ModelData], ClusterEnv]],
                               model_id_map, train_workload: Workload):
    """Solve every (model cluster, device share) on its own and stitch the
    groups together under the global model ids (:244-255)."""
    sol = ModelPlacement([], [])
    for i, (sub_model_datas, sub_cluster_env) in enumerate(eco_separation):
        eco_sol, _ = self.solve_placement_one_eco(sub_model_datas, sub_cluster_env, train_workload)
        sol.group_configs += eco_sol.group_configs
        sol.group_models += [[model_id_map[(i, m)] for m in group] for group in eco_sol.group_models]
    return sol


def solve_separations_lockstep(self, separations, model_id_map, model_datas: List[ModelData],
                               cluster_env: ClusterEnv, train_workload: Workload):
    """``solve_separation_placement`` for every separation, with all greedy searches advanced together.

    The reference solves each (model cluster, device share) of each separation with its own evaluator
    over the full training workload, in which the other clusters' requests name unknown models and are
    skipped (:244-255, :323-353).  A placement that hosts only the cluster's models, scored on the same
    workload under the global model ids, gives the same counts for those models and the same score, so
    one evaluator serves all sub-problems: every iteration scores the current placement of every search
    (all layouts of all distinct sub-problems) in one call.  A sub-problem is a (cluster, device count)
    pair; separations share them, so each is solved once.  Returns one stitched placement per separation,
    equal to what solving them one by one returns."""
    from types import SimpleNamespace
    from mms_amd.placement_policy.base_policy import _fast_greedy_step, weight_mem_table
    evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload,
                                   self.evaluator_method, self.parallel_evaluator)
    subs = {}
    for sep in separations:
        for ci, (sub_model_datas, sub_env) in enumerate(sep):
            key = (ci, sub_env.num_devices)
            if key not in subs:
                subs[key] = SimpleNamespace(
                    model_datas=sub_model_datas, env=sub_env,
                    gmap=[model_id_map[(ci, j)] for j in range(len(sub_model_datas))],
                    sols=self.enumerate_group_configs_uneven(sub_env))

    def to_global(sub, sol):
        return ModelPlacement(list(sol.group_configs), [[sub.gmap[m] for m in ms] for ms in sol.group_models])

    searches = [(sub, i) for sub in subs.values() for i in range(len(sub.sols))]
    weight_mems = [weight_mem_table(sub.sols[i].group_configs, sub.model_datas) for sub, i in searches]
    running = list(range(len(searches)))
    while running:
        all_stats = evaluator.get_stats([to_global(searches[r][0], searches[r][0].sols[searches[r][1]])
                                         for r in running])
        still = []
        for r, (overall, goodputs, group_num_requests, full) in zip(running, all_stats):
            sub, i = searches[r]
            sol = sub.sols[i]
            local = (overall, [goodputs[g] for g in sub.gmap], group_num_requests,
                     SimpleNamespace(per_model_stats=[full.per_model_stats[g] for g in sub.gmap]))
            choice = _fast_greedy_step(sol, local, weight_mems[r], sub.env)
            if choice is not None:
                sub.sols[i] = sol.add_model(*choice).normalize()
                still.append(r)
        running = still
    # the best layout of every sub-problem (first of equal scores, as np.argmax in :353)
    finals = [to_global(sub, sol) for sub in subs.values() for sol in sub.sols]
    scores = evaluator.get_scores(finals)
    at = 0
    for sub in subs.values():
        n = len(sub.sols)
        sub.best = sub.sols[int(np.argmax(scores[at:at + n]))]
        at += n
    stitched = []
    for sep in separations:
        sol = ModelPlacement([], [])
        for ci, (_, sub_env) in enumerate(sep):
            sub = subs[(ci, sub_env.num_devices)]
            sol.group_configs += list(sub.best.group_configs)
            sol.group_models += [[sub.gmap[m] for m in group] for group in sub.best.group_models]
        stitched.append(sol)
    return stitched


class ModelParallelismSearch(BasePlacementPolicy):
    """Enumerate group partitions, fill each greedily, keep the best score."""

    def __init__(self, max_bs: int = 1, max_pp: int = 8, max_op: int = 4,
                 use_evo_search: bool = False, use_separation: bool = False, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.max_bs, self.max_pp, self.max_op = max_bs, max_pp, max_op
        self.n_iter = 1
        self.seed = 0
        self.beam_size = 3
        self.use_evo_search = use_evo_search
        self.use_separation = use_separation
        self.evaluator_method = "fast_simulator"
        self.parallel_evaluator = False
        self.parallel_initial_placement = False

    def solve_placement_one_eco(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                                train_workload: Workload = None):
        """:323-353"""
        evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload,
                                       self.evaluator_method, self.parallel_evaluator)
        sols = self.enumerate_group_configs_uneven(cluster_env)
        # one greedy search per layout, advanced together (one evaluator call per iteration for all of them)
        sols = replica_placement_fast_greedy_lockstep(sols, model_datas, cluster_env, train_workload,
                                                      evaluator, self.verbose)
        scores = evaluator.get_scores(sols)
        return sols[int(np.argmax(scores))], {}

    def enumerate_separations(self, model_datas: List[ModelData], cluster_env: ClusterEnv):
        """Cluster models of similar single-device latency and enumerate how
        to split the devices among the clusters (:356-408)."""
        same_model_threshold = 0.38
        one = ParallelConfig(1, 1, 1)
        model_id_map = {}
        clusters = []
        cluster_latencies = []
        for model_id, data in enumerate(model_datas):
            latency = max(data.profiling_result.para_dict[one].latency[1])
            for i, cluster in enumerate(clusters):
                ref = max(cluster[0].profiling_result.para_dict[one].latency[1])
                if math.fabs(latency - ref) / ref < same_model_threshold:
                    model_id_map[(i, len(cluster))] = model_id
                    cluster.append(data)
                    break
            else:
                model_id_map[(len(clusters), 0)] = model_id
                clusters.append([data])
                cluster_latencies.append(latency)

        partitions = get_partitions(cluster_env.num_devices, len(clusters))
        ratio = np.empty(len(clusters), dtype=np.float32)
        for i, cluster in enumerate(clusters):
            ratio[i] = sum(x.rate for x in cluster)
        ratio = ratio / np.sum(ratio)

        for threshold in [1.0, 0.5, 0.3, 0.2, 0.1]:
            reduced = []
            for partition in partitions:
                throughputs = [x / l for x, l in zip(partition, cluster_latencies)]
                norm = np.array(throughputs) / sum(throughputs)
                if np.max(np.abs(ratio - norm)) < threshold:
                    reduced.append(partition)
            if len(reduced) < 100:
                break
        print(f"original: {len(partitions)}  reduced: {len(reduced)}")
        separations = [[(clusters[i], ClusterEnv(n, cluster_env.mem_budget)) for i, n in enumerate(partition)]
                       for partition in reduced]
        return separations, model_id_map

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        """:411-456"""
        if train_workload is None:
            train_workload = gen_train_workload(model_datas)
        best_sol, _ = self.solve_placement_one_eco(model_datas, cluster_env, train_workload)
        evaluator = None

        if self.use_separation:
            separations, model_id_map = self.enumerate_separations(model_datas, cluster_env)
            print("number of combinations: ", len(separations))
            sols = solve_separations_lockstep(self, separations, model_id_map, model_datas, cluster_env,
                                              train_workload)
            evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload,
                                           self.evaluator_method, self.parallel_evaluator)
            scores = evaluator.get_scores(sols)
            best_idx = int(np.argmax(scores))
            evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload,
                                           self.evaluator_method, self.parallel_evaluator)
            score_mixed = evaluator.get_scores([best_sol])[0]
            print(f"score_mixed: {score_mixed:.3f}, score_separate: {scores[best_idx]:.3f}")
            if scores[best_idx] > score_mixed:
                best_sol = sols[best_idx]

        if self.use_evo_search:
            if evaluator is None:   # the reference reaches this with `evaluator` unbound unless use_separation is set
                evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload,
                                               self.evaluator_method, self.parallel_evaluator)
            best_sol = evolutionary_search([best_sol], model_datas, cluster_env, evaluator, 200, self.verbose)
        return best_sol, {}

    def _configs_for(self, group_size):
        for pp in get_factors(group_size):
            op = group_size // pp
            if pp <= self.max_pp and op <= self.max_op:
                yield ParallelConfig(1, op, pp)

    def enumerate_group_configs_uneven(self, cluster_env: ClusterEnv):
        """Power-of-two group sizes; devices that do not fill a group form
        smaller power-of-two pipeline groups (:459-479)."""
        sols = []
        n, per_node = cluster_env.num_devices, cluster_env.num_devices_per_node
        for group_size in get2tok(n):
            if group_size > per_node and group_size % per_node != 0:
                continue
            regular = n // group_size
            rest = decompose2tok(n % group_size)
            for cfg in self._configs_for(group_size):
                sols.append(ModelPlacement([cfg] * regular + [ParallelConfig(1, 1, s) for s in rest],
                                           [[] for _ in range(regular + len(rest))]))
        return sols

    def enumerate_group_configs(self, cluster_env):
        """Group sizes that divide the device count (:482-500)."""
        sols = []
        n, per_node = cluster_env.num_devices, cluster_env.num_devices_per_node
        for group_size in get_factors(n):
            if group_size > per_node and group_size % per_node != 0:
                continue
            for cfg in self._configs_for(group_size):
                sols.append(ModelPlacement([cfg] * (n // group_size), [[] for _ in range(n // group_size)]))
        return sols

    def greedy_group_configs(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                             train_workload: Workload, evaluator: PlacementEvaluator, beam_size=3):
        """Grow the device count one by one, keeping the ``beam_size`` best
        group layouts for every prefix (:502-547)."""
        assert beam_size >= 1, "beam size should >= 1."
        n, per_node = cluster_env.num_devices, cluster_env.num_devices_per_node
        beams = [[ModelPlacement([], [])]]
        for cur in range(1, n + 1):
            starts = []
            for last_size in range(1, (cur - 1) % per_node + 1 + 1):
                for cfg in self._configs_for(last_size):
                    for sol in beams[cur - last_size]:
                        pre = sol.copy()
                        pre.group_configs.append(cfg)
                        pre.group_models = [[] for _ in range(len(pre.group_configs))]
                        starts.append(pre)
            candidates = replica_placement_fast_greedy_lockstep(
                starts, model_datas, cluster_env, train_workload, evaluator, self.verbose)
            scores = evaluator.get_scores(candidates)
            keep = np.argsort(scores)[::-1][:beam_size]
            beams.append([candidates[i] for i in keep])
        return beams[n]


class ModelParallelismEqual(BasePlacementPolicy):
    """One model per group, all groups (op, pp) (:549-564)."""

    def __init__(self, pp, op, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.pp = pp
        self.op = op

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        num_groups = cluster_env.num_devices // (self.op * self.pp)
        sol = ModelPlacement([ParallelConfig(1, self.op, self.pp)] * num_groups,
                             [[i] for i in range(num_groups)])
        return sol, None
