"""Model placement policies (search drivers over the GPU placement evaluator).

Same names as the reference's ``alpa_serve.placement_policy`` package.
"""
from mms_amd.placement_policy.base_policy import (
    ModelData, ClusterEnv, ModelPlacement, ModelPlacementWithReplacement,
    PlacementEvaluator, BasePlacementPolicy, gen_train_workload)
from mms_amd.placement_policy.model_parallelism import (
    ModelParallelismILP, ModelParallelismRR, ModelParallelismGreedy,
    ModelParallelismSearch, ModelParallelismEqual)
from mms_amd.placement_policy.selective_replication import (
    SelectiveReplicationILP, SelectiveReplicationGreedy, SelectiveReplicationUniform,
    SelectiveReplicationSearch, SelectiveReplicationReplacement)
