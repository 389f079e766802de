"""Record what the reference's event-driven simulator returns on seeded inputs.

``simulate_one_case`` (alpa_serve/simulator/controller.py:257-279) runs a
discrete-event model of the serving system: HTTP, dispatch and executor
overheads drawn from numpy's global generator, shortest-queue dispatch, a
stage-clock admission test in every group manager, and per-device streams.
Its outcome depends on the order in which those draws are consumed, so it
cannot be derived by reading; no test of the reference covers it.  This script
runs the reference's own classes on three small seeded cases and records, per
request, the finish time (bit pattern) and the good flag, plus the per-group
request counts, into ``event_sim_vectors.json`` next to this file.
tests/test_event_sim.py requires the drop-in ``simulate_one_case`` to
reproduce them bit for bit.

Runs only in the build container (needs /root/reference).  ``numba``, ``ray``
and the trace package's plotting imports are not installed and are not
executed by the code recorded here; inert placeholder modules are registered
so that the imports succeed.

Run:  python tests/golden/make_event_sim_vectors.py
"""
import json
import os
import sys
import types
from functools import partial
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
    import alpa_serve.simulator.controller as ctl
    import alpa_serve.simulator.workload as wl
    from alpa_serve.simulator.executable import Executable
    from alpa_serve.simulator.event_loop import run_event_loop
    return pp, prof, ctl, wl, Executable, run_event_loop


# name, numpy seed, models as (rate, cv, slo), profile, duration, groups as (pp, models), registered but unplaced models
CASES = [
    ("light_two_stage", 11, [(4, 1, 1.0), (3, 2, 1.0), (2, 1, 1.0)], "test-2GB-100ms", 40.0,
     [(2, [0, 1, 2]), (1, [0, 1]), (1, [2])], []),
    ("overload_drops", 12, [(14, 3, 0.4), (9, 2, 0.4), (11, 4, 0.5), (5, 1, 0.3)], "test-2GB-100ms", 30.0,
     [(2, [0, 1, 2, 3]), (2, [0, 2])], []),
    ("unplaced_model_and_deep_pipeline", 13, [(6, 2, 0.6), (6, 2, 0.6), (3, 1, 0.6)], "test-2GB-100ms", 30.0,
     [(4, [0, 1])], [2]),
]


def main():
    pp, prof, ctl, wl, Executable, run_event_loop = _import_reference()
    PC = prof.ParallelConfig
    out = []
    for name, seed, models, prof_name, duration, groups, unplaced in CASES:
        profile = prof.load_test_prof_result(prof_name)
        model_datas = [pp.ModelData(f"m{i}", slo, rate, cv, profile) for i, (rate, cv, slo) in enumerate(models)]
        placement = pp.base_policy.ModelPlacement([PC(1, 1, p) for p, _ in groups], [list(ms) for _, ms in groups])
        cluster_env = pp.ClusterEnv(sum(p for p, _ in groups), 64 * (1 << 30))

        def register_models(controller):
            for md in model_datas:
                controller.register_model.remote(md.name, partial(Executable, md.profiling_result))

        def generate_workload(start=0):
            ws = [wl.GammaProcess(md.rate, md.cv).generate_workload(md.name, start, duration, slo=md.slo, seed=seed * 100 + i)
                  for i, md in enumerate(model_datas)]
            return wl.Workload.merge(*ws)

        def place_models(controller):
            pp.base_policy.BasePlacementPolicy().place_models_impl(controller, cluster_env, model_datas, placement)

        # the steps of simulate_one_case (controller.py:257-279), keeping the client to read its per-request arrays
        np.random.seed(seed)
        controller = ctl.Controller()
        register_models(controller)
        place_models(controller)
        client = ctl.Client(controller)
        workload = generate_workload()
        stats = run_event_loop(ctl.run_workload(client, workload, 5))
        start, finish, good = client.res_dict[workload]
        assert np.array_equal(start, workload.arrivals)
        groups_seen = [int(x.num_total_requests) for x in controller.group_info.values()]
        out.append({
            "name": name, "seed": seed, "models": [list(m) for m in models], "profile": prof_name,
            "duration": duration, "groups": [[p, list(ms)] for p, ms in groups], "unplaced": unplaced, "warmup": 5,
            "num_requests": len(workload),
            "arrivals_hex": [float(x).hex() for x in workload.arrivals],
            "finish_hex": [float(x).hex() for x in finish],
            "good": [int(bool(x)) for x in good],
            "group_num_requests": groups_seen,
            "goodput": float(stats.goodput), "latency_mean": float(stats.latency_mean),
            "per_model": [[s.name, int(s.num_requests), float(s.goodput), float(s.latency_p99)] for s in stats.per_model_stats],
        })
        print(name, len(workload), "requests, goodput", float(stats.goodput), "groups", groups_seen, flush=True)
    path = os.path.join(HERE, "event_sim_vectors.json")
    with open(path, "w") as f:
        json.dump({"cases": out}, f, indent=0)
    print("wrote", path)


if __name__ == "__main__":
    main()
