"""Placement policies without model parallelism: every device is its own
group and models are replicated selectively.

Mirrors ``SelectiveReplicationGreedy`` (:126-153), ``SelectiveReplicationUniform``
(:156-176), ``SelectiveReplicationSearch`` (:179-203) and
``SelectiveReplicationReplacement`` (:206-244) of the reference's
``alpa_serve/placement_policy/selective_replication.py``.  The ILP variant
(:23-123) needs the external pulp/CBC solver and is not provided.
"""
from typing import List

import numpy as np

from mms_amd.placement_policy.base_policy import (
    BasePlacementPolicy, ClusterEnv, ModelData, ModelPlacement, ModelPlacementWithReplacement,
    PlacementEvaluator, evolutionary_search, gen_train_workload, replica_placement_beam_search,
    replica_placement_fast_greedy)
from mms_amd.profiling import ParallelConfig
from mms_amd.simulator.workload import Workload

_ONE = ParallelConfig(1, 1, 1)


def _one_device_groups(cluster_env):
    n = cluster_env.num_devices
    return ModelPlacement([_ONE] * n, [[] for _ in range(n)])


class SelectiveReplicationILP(BasePlacementPolicy):
    def __init__(self, *args, **kwargs):
        raise NotImplementedError(
            "SelectiveReplicationILP needs the pulp/CBC integer-programming solver and does not "
            "use the placement simulator; it is outside this package")


class SelectiveReplicationGreedy(BasePlacementPolicy):
    """Greedy replica placement on single-device groups.

    With ``use_evo_search`` the reference calls ``evolutionary_search`` with
    the wrong argument list from a module that does not import it
    (selective_replication.py:152); here the call is made with the argument
    list ``evolutionary_search`` actually has, 200 iterations as in
    ModelParallelismGreedy.
    """

    def __init__(self, use_evo_search: bool = False, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.use_evo_search = use_evo_search

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        if train_workload is None:
            train_workload = gen_train_workload(model_datas)
        evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload, "fast_simulator", False)
        sol = replica_placement_fast_greedy(_one_device_groups(cluster_env), model_datas, cluster_env,
                                            train_workload, evaluator, self.verbose)
        if self.use_evo_search:
            sol = evolutionary_search([sol], model_datas, cluster_env, evaluator, 200, self.verbose)
        return sol, None


class SelectiveReplicationUniform(BasePlacementPolicy):
    """Group i hosts models i, i+1, ... (mod M), as many as fit (:156-176).
    Rows of ``group_models`` are numpy arrays, as in the reference."""

    def __init__(self, verbose: int = 0):
        super().__init__(verbose=verbose)

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        num_models = len(model_datas)
        model_memory = model_datas[0].profiling_result.para_dict[_ONE].weight_mem[0]
        per_group = min(int(cluster_env.mem_budget / model_memory), num_models)
        rows = [np.arange(i, i + per_group) % num_models for i in range(cluster_env.num_devices)]
        return ModelPlacement([_ONE] * cluster_env.num_devices, rows), None


class SelectiveReplicationSearch(BasePlacementPolicy):
    """Beam search (width 3) over "add one replica" moves (:179-203)."""

    def __init__(self, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.beam_size = 3

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        if train_workload is None:
            train_workload = gen_train_workload(model_datas)
        evaluator = PlacementEvaluator(model_datas, cluster_env, train_workload, "fast_simulator", False)
        sol = replica_placement_beam_search(_one_device_groups(cluster_env), model_datas, cluster_env,
                                            train_workload, evaluator, self.beam_size, self.verbose)
        return sol, None


class SelectiveReplicationReplacement(BasePlacementPolicy):
    """A fresh greedy placement for every ``replacement_interval`` seconds of
    the workload (:206-244)."""

    def __init__(self, replacement_interval: int, use_evo_search: bool = False, verbose: int = 0):
        super().__init__(verbose=verbose)
        self.replacement_interval = replacement_interval
        self.use_evo_search = use_evo_search

    def solve_placement(self, model_datas: List[ModelData], cluster_env: ClusterEnv,
                        train_workload: Workload = None):
        if train_workload is None:
            train_workload = gen_train_workload(model_datas)
        start_times, placements = [], []
        for piece in train_workload.split_time_interval(self.replacement_interval):
            evaluator = PlacementEvaluator(model_datas, cluster_env, piece, "fast_simulator", False)
            sol = replica_placement_fast_greedy(_one_device_groups(cluster_env), model_datas, cluster_env,
                                                piece, evaluator, self.verbose)
            if self.use_evo_search:   # see SelectiveReplicationGreedy about the reference's call here
                sol = evolutionary_search([sol], model_datas, cluster_env, evaluator, 200, self.verbose)
            start_times.append(piece.arrivals[0])
            placements.append(sol)
        return ModelPlacementWithReplacement(start_times, placements), None
