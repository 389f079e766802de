"""Record what the reference's placement searches return on seeded inputs.

The searches (alpa_serve/placement_policy/base_policy.py:329-479,
model_parallelism.py:208-241, 294-353, selective_replication.py:126-203) break
ties with np.argsort / np.argmax on numbers that, once every request is served,
differ only by rounding noise, so their outcome cannot be derived by reading.
The reference's own test (tests/serve/test_placement_policy.py:24-77) asserts
coarse properties of three outcomes; this script records the outcomes
themselves -- final placement and its score -- for those inputs and a few more,
into ``search_vectors.json`` next to this file.  tests/test_policies.py
requires the drop-in policies to return the same placements.

Runs only in the build container (needs /root/reference).  ``numba``, ``ray``
and the trace package's plotting imports are not installed and are not
executed by the code recorded here; inert placeholder modules are registered
so that the imports succeed.  numba's jit is replaced by the identity, so the
reference's request loop runs as the plain Python it is written in.

Run:  python tests/golden/make_search_vectors.py
"""
import json
import os
import sys
import types
from unittest import mock

import numpy as np

sys.dont_write_bytecode = True
HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = "/root/reference"


def _import_reference():
    numba = types.ModuleType("numba")
    numba.jit = lambda *a, **k: (lambda f: f)
    sys.modules.setdefault("numba", numba)
    for name in ("ray", "ray.actor", "ray.util", "ray.util.scheduling_strategies", "pulp",
                 "alpa_serve.trace", "matplotlib", "matplotlib.pyplot"):
        sys.modules.setdefault(name, mock.MagicMock(name=name))
    sys.path.insert(0, REFERENCE)
    import alpa_serve.placement_policy as pp
    import alpa_serve.profiling as prof
    return pp, prof


def main():
    pp, prof = _import_reference()
    GB = 1 << 30
    PC = prof.ParallelConfig

    def models(n, slo, rate, cv, name="test-2GB-100ms"):
        return [pp.ModelData(f"m{i}", slo, rate, cv, prof.load_test_prof_result(name)) for i in range(n)]

    def dump(placement):
        return {"group_configs": [list(c) for c in placement.group_configs],
                "group_models": [[int(m) for m in ms] for ms in placement.group_models]}

    cases = []

    def record(name, policy_name, kwargs, model_spec, cluster_spec):
        # model_spec: (n, slo, rate, cv[, profile]) or a list of such tuples (models m0, m1, ... in that order)
        if isinstance(model_spec, list):
            model_datas = []
            for n, slo, rate, cv, prof_name in model_spec:
                model_datas += [pp.ModelData(f"m{len(model_datas) + i}", slo, rate, cv,
                                             prof.load_test_prof_result(prof_name)) for i in range(n)]
        else:
            model_datas = models(*model_spec)
        cluster_env = pp.ClusterEnv(*cluster_spec)
        policy = getattr(pp, policy_name)(**kwargs)
        placement, _ = policy.solve_placement(model_datas, cluster_env)
        wl = pp.base_policy.gen_train_workload(model_datas)
        ev = pp.base_policy.PlacementEvaluator(model_datas, cluster_env, wl, "fast_simulator", False)
        score = float(ev.get_scores([placement])[0])
        stats = ev.get_stats([placement])[0]
        cases.append({"name": name, "policy": policy_name, "kwargs": kwargs,
                      "models": [list(x) for x in model_spec] if isinstance(model_spec, list) else list(model_spec),
                      "cluster": list(cluster_spec),
                      "placement": dump(placement), "score": score,
                      "goodput": float(stats[0]),
                      "group_num_requests": [int(x) for x in stats[2]]})
        if kwargs.get("use_separation"):
            # the best of the separated solutions too (the search may prefer the unseparated one)
            import alpa_serve.placement_policy.model_parallelism as mp
            separations, model_id_map = policy.enumerate_separations(model_datas, cluster_env)
            sols = [mp.solve_separation_placement(policy, sep, model_id_map, wl) for sep in separations]
            # (a fresh evaluator: the sub-problems' evaluators replaced the workload's cached model ids)
            ev2 = pp.base_policy.PlacementEvaluator(model_datas, cluster_env, wl, "fast_simulator", False)
            scores = [float(x) for x in ev2.get_scores(sols)]
            best = int(np.argmax(scores))
            cases[-1]["separations"] = {"count": len(separations), "scores": scores,
                                        "best": dump(sols[best]), "best_score": scores[best]}
        print(name, dump(placement)["group_models"], score, flush=True)

    def record_replacement(name, interval, model_spec, cluster_spec):
        """SelectiveReplicationReplacement (selective_replication.py:206-244): one greedy placement per interval
        of the workload; the composite is then scored by the reference's own approximate_one_case, segment by
        segment (simulator/controller.py:345-391)."""
        model_datas = models(*model_spec)
        cluster_env = pp.ClusterEnv(*cluster_spec)
        rep, _ = pp.SelectiveReplicationReplacement(interval).solve_placement(model_datas, cluster_env)
        wl = pp.base_policy.gen_train_workload(model_datas)
        ev = pp.base_policy.PlacementEvaluator(model_datas, cluster_env, wl, "fast_simulator", False)
        # (get_scores of the reference cannot take the composite: base_policy.py:225 reads sol.group_models)
        stats = ev.get_stats([rep])[0]
        cases.append({"name": name, "policy": "SelectiveReplicationReplacement", "kwargs": {"replacement_interval": interval},
                      "models": list(model_spec), "cluster": list(cluster_spec),
                      "start_times": [float(t) for t in rep.start_times],
                      "placements": [dump(p) for p in rep.placements],
                      "goodput": float(stats[0]), "model_goodput": [float(x) for x in stats[1]],
                      "latency_mean": float(stats[3].latency_mean),
                      "group_num_requests": [int(x) for x in stats[2]]})
        print(name, len(rep.placements), "segments", float(stats[0]), flush=True)

    # the three situations of the reference's own test
    record("ref_test_sr_greedy", "SelectiveReplicationGreedy", {}, (4, 1, 5, 1), (4, 4.5 * GB))
    record("ref_test_sr_search", "SelectiveReplicationSearch", {}, (4, 1, 5, 1), (4, 4.5 * GB))
    record("ref_test_mp_greedy", "ModelParallelismGreedy", {"group_size": 2}, (4, 1, 5, 1), (4, 4.5 * GB))
    record("ref_test_mp_search", "ModelParallelismSearch", {}, (4, 0.4, 4, 8), (4, 2.5 * GB))
    # loaded systems, where requests are really dropped
    record("loaded_sr_greedy", "SelectiveReplicationGreedy", {}, (4, 0.5, 9, 4), (4, 4.5 * GB))
    record("loaded_mp_greedy", "ModelParallelismGreedy", {"group_size": 2}, (6, 0.4, 6, 4), (4, 6.5 * GB))
    record("loaded_mp_search", "ModelParallelismSearch", {}, (5, 0.5, 7, 6, "test-4GB-150ms"), (8, 8.5 * GB))

    # two kinds of models: the search also splits the devices between them (model_parallelism.py:356-456)
    record("separation_mp_search", "ModelParallelismSearch", {"use_separation": True},
           [(3, 0.5, 5, 3, "test-2GB-100ms"), (2, 0.9, 3, 2, "test-4GB-150ms")], (6, 8.5 * GB))

    # a placement per 150 s of a loaded workload (5 models do not all fit 4 devices at once)
    record_replacement("replacement_sr", 150, (5, 0.5, 7, 4), (4, 4.5 * GB))

    path = os.path.join(HERE, "search_vectors.json")
    with open(path, "w") as f:
        json.dump({"cases": cases}, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
