"""Model placement policies (search drivers over the GPU placement evaluator)."""
from mms_amd.placement_policy.base_policy import (
    ModelData, ClusterEnv, ModelPlacement, ModelPlacementWithReplacement,
    PlacementEvaluator, BasePlacementPolicy, gen_train_workload)
