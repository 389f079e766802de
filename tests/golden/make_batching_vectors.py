"""Write golden vectors for the batching simulator from the reference itself.

No test of the reference exercises ``simulate_requests_mixed_batching``
(alpa_serve/simulator/controller.py:631-798), and no closed form covers its
heap / FIFO / batch-growth rules, so this script imports that one function
from the reference checkout at /root/reference (only present in the build
container) and records its outputs on seeded random inputs.  The inputs come
from ``tests/randcase.py``; the outputs are stored next to this script in
``batching_vectors.npz`` and are what ``tests/test_oracle_batching.py``
checks both oracle restatements against.

The reference module imports ``numba`` (only as a decorator on *other*
functions) and, through the serving runtime, ``ray``; neither is installed
and neither is executed by the function recorded here, so inert placeholder
modules are registered for the import to succeed.  Nothing is written into
the reference tree.

Run:  python tests/golden/make_batching_vectors.py
"""
import os
import sys
import types
from unittest import mock

import numpy as np

sys.dont_write_bytecode = True
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))          # tests/ for randcase
REFERENCE = "/root/reference"


def _import_reference_function():
    numba = types.ModuleType("numba")
    numba.jit = lambda *a, **k: (lambda f: f)
    sys.modules.setdefault("numba", numba)
    for name in ("ray", "ray.actor", "ray.util", "ray.util.scheduling_strategies"):
        sys.modules.setdefault(name, mock.MagicMock(name=name))
    sys.path.insert(0, REFERENCE)
    import alpa_serve.simulator.controller as ctl
    return ctl


def cases():
    from randcase import random_case
    out = []
    for seed in range(240):
        nb = 1 + seed % 4
        out.append((random_case(50_000 + seed, nb=nb, max_r=80, load=1.0 + seed % 5,
                                inf_slo=False), nb))
    for seed in range(24):                     # longer, heavier: deep queues and big batches
        nb = 2 + seed % 3
        out.append((random_case(60_000 + seed, max_m=6, max_g=4, max_s=4, max_r=600, nb=nb,
                                load=4.0 + 4 * (seed % 4), tie_prob=0.05, p_unknown=0.01,
                                p_inf_row=0.02, p_odd_slo=0.01, inf_slo=False), nb))
    return out


def main():
    ctl = _import_reference_function()
    blob = {}
    all_cases = cases()
    for n, (c, nb) in enumerate(all_cases):
        ctl.batchsize_config[:] = [1, 2, 4, 8, 16][:nb]
        R = c["R"]
        finish = np.full(R, np.nan)
        good = np.zeros(R, dtype=bool)
        counts = ctl.simulate_requests_mixed_batching(
            finish, good, c["tstamps"], c["model_ids"], c["slos"], c["m2g"], c["g2m"],
            c["num_stages"], c["lat"], R)
        for key in ("tstamps", "model_ids", "slos", "m2g", "g2m", "num_stages", "lat"):
            blob[f"c{n}_{key}"] = c[key]
        blob[f"c{n}_nb"] = np.int32(nb)
        blob[f"c{n}_finish"] = finish
        blob[f"c{n}_good"] = good
        for name, arr in zip(("mreq", "mgood", "greq", "ggood"), counts):
            blob[f"c{n}_{name}"] = np.asarray(arr, np.int32)
    blob["num_cases"] = np.int32(len(all_cases))
    path = os.path.join(HERE, "batching_vectors.npz")
    np.savez_compressed(path, **blob)
    print(f"wrote {len(all_cases)} cases to {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
