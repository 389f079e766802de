"""Make ``import alpa_serve...`` resolve to this package for the placement-
evaluation path, so scripts written against the reference run unchanged.

    import mms_amd.compat; mms_amd.compat.install()
    from alpa_serve.placement_policy import ModelData, ClusterEnv, SelectiveReplicationGreedy
    from alpa_serve.simulator.controller import approximate_one_case

Only the modules of that path are aliased (the reference's package layout:
alpa_serve/{profiling,util}.py, alpa_serve/simulator/{workload,controller,
executable}.py, alpa_serve/placement_policy/*).  ``install`` refuses to shadow
a real ``alpa_serve`` installation unless ``force=True``.
"""
import importlib
import importlib.util
import sys
import types

_ALIASES = {
    "alpa_serve.profiling": "mms_amd.profiling",
    "alpa_serve.util": "mms_amd.util",
    "alpa_serve.simulator.workload": "mms_amd.simulator.workload",
    "alpa_serve.simulator.controller": "mms_amd.simulator.controller",
    "alpa_serve.simulator.executable": "mms_amd.simulator.executable",
    "alpa_serve.trace": "mms_amd.trace",
    "alpa_serve.placement_policy": "mms_amd.placement_policy",
    "alpa_serve.placement_policy.base_policy": "mms_amd.placement_policy.base_policy",
    "alpa_serve.placement_policy.model_parallelism": "mms_amd.placement_policy.model_parallelism",
    "alpa_serve.placement_policy.selective_replication": "mms_amd.placement_policy.selective_replication",
}


def install(force: bool = False) -> None:
    if "alpa_serve" in sys.modules and getattr(sys.modules["alpa_serve"], "__mms_amd_alias__", False):
        return
    if not force and importlib.util.find_spec("alpa_serve") is not None:
        raise RuntimeError("a real alpa_serve package is importable; pass force=True to shadow it")
    root = types.ModuleType("alpa_serve")
    root.__mms_amd_alias__ = True
    root.__path__ = []
    sim = types.ModuleType("alpa_serve.simulator")
    sim.__path__ = []
    sys.modules["alpa_serve"] = root
    sys.modules["alpa_serve.simulator"] = sim
    root.simulator = sim
    for alias, target in _ALIASES.items():
        mod = importlib.import_module(target)
        sys.modules[alias] = mod
        parent, _, leaf = alias.rpartition(".")
        setattr(sys.modules[parent], leaf, mod)
