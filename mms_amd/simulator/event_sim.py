"""The event-driven serving simulator: the slower, more detailed model that the
approximate simulator is checked against.

Drop-in for ``Controller``, ``GroupManager``, ``Client`` and
``simulate_one_case`` of the reference's ``alpa_serve/simulator/controller.py``
(:30-279) together with what they stand on (``simulator/event_loop.py``,
``simulator/executable.py:7-46``, ``simulator/cluster.py``).  This is host
code: one request at a time through a model of the serving system, nothing a
GPU lane could share with its neighbours.

What is modelled, per request (reference lines in brackets):

1. the client submits it at its arrival time and the controller sees it one
   HTTP overhead later (:221-227, :239-243);
2. the controller sends it to the group with the shortest queue among those
   that host the model, first listed wins ties, and the group manager sees it
   one dispatch overhead later (:183-211); a model without replicas is
   answered at once with "rejected" (:193-194);
3. the group manager walks its stage clocks, ``t = max(clock[k], t) +
   latency[k]``, and rejects the request if ``t + 0.004`` exceeds arrival +
   SLO; otherwise it commits the clocks and starts the executable one executor
   overhead later (:76-98);
4. the executable occupies the group's devices stage by stage: a stage waits for
   its device's stream and holds it for the stage latency
   (executable.py:31-46, event_loop.py:158-166);
5. the request is good if it was not rejected and finish - arrival <= SLO
   (:226-227).

The three overheads are drawn from numpy's global generator exactly where the
reference draws them: 2048 dispatch overheads when the controller is made
(:113-114), 2048 executor overheads per group manager when it is made
(:52-53), one HTTP overhead per request when the workload is submitted
(:239-240); the first two lists are cycled.  With the generator seeded the
same, the results are the reference's bit for bit
(``tests/test_event_sim.py``).

The reference runs this on asyncio coroutines over a priority queue of wake-up
times; here every request is a small state machine over one heap.  Events at
exactly the same time run in the order they were scheduled (the reference's
order among exact ties follows the internals of ``heapq`` with a comparison on
the time alone; with continuous random overheads such ties do not occur).
"""
import heapq
from functools import partial
from itertools import count, cycle
from typing import Callable, Dict, List, Optional

import numpy as np

from mms_amd.profiling import ProfilingResult
from mms_amd.simulator.workload import DEFAULT_WARMUP, Workload


def _install_remote_methods(obj):
    for key in dir(obj):
        value = getattr(obj, key)
        if callable(value) and not key.startswith("_"):
            wrapped = partial(value)
            wrapped.remote = wrapped
            setattr(obj, key, wrapped)


class GroupManager:
    """One group of devices: admission by stage clocks, execution on per-stage streams
    (controller.py:30-98, cluster.py, executable.py)."""

    fixed_overhead = 0.004

    def __init__(self, virtual_mesh_shape):
        self.virtual_mesh_shape = tuple(virtual_mesh_shape)
        self.num_devices = int(np.prod(virtual_mesh_shape))
        self.stage_clock = [0] * self.num_devices
        self.latency_dict: Dict[str, Dict[int, List[float]]] = {}
        self.parallel_config = None          # of the group's replicas (they share one mesh group)
        self.stream_clock: List[float] = []  # one stream per pipeline stage: the first device of the stage's mesh
        self.alpa_overhead = cycle(np.abs(np.random.normal(loc=0.005, scale=0.0005, size=(2048,))))

    def create_replica(self, name: str, model_def: Callable, parallel_config):
        assert name not in self.latency_dict
        profile = next(a for a in model_def.args if isinstance(a, ProfilingResult))
        if self.parallel_config is None:
            # the first replica launches the group's meshes (executable.py:17-24, cluster.py:43-51)
            assert self.num_devices == parallel_config.dp * parallel_config.op * parallel_config.pp
            self.parallel_config = parallel_config
            self.stream_clock = [0] * parallel_config.pp
        else:
            assert parallel_config == self.parallel_config
        self.latency_dict[name] = profile.para_dict[parallel_config].latency


class Controller:
    """The serving controller (controller.py:101-215): model and group registry, shortest-queue dispatch."""

    def __init__(self):
        self.model_groups: Dict[str, List[int]] = {}
        self.model_defs: Dict[str, Callable] = {}
        self.managers: Dict[int, GroupManager] = {}
        self.queue_size: Dict[int, int] = {}
        self.num_total_requests: Dict[int, int] = {}
        self.dispatch_overhead = cycle(np.abs(np.random.normal(loc=0.0025, scale=0.0005, size=(2048,))))
        _install_remote_methods(self)

    def create_mesh_group_manager(self, group_id: int, virtual_mesh_shape=None, num_gpus: int = 0):
        assert group_id not in self.managers, f"Mesh group {group_id} is already launched"
        self.managers[group_id] = GroupManager(virtual_mesh_shape)
        self.queue_size[group_id] = 0
        self.num_total_requests[group_id] = 0

    def register_model(self, name: str, model_def: Callable, init_args: Optional[List] = None,
                       init_kwargs: Optional[Dict] = None, override: bool = False):
        if name in self.model_groups and not override:
            raise ValueError(f"Model {name} is already registered")
        assert isinstance(model_def, partial)
        if name in self.model_groups:
            for g in self.model_groups[name]:
                del self.managers[g].latency_dict[name]
        self.model_groups[name] = []
        self.model_defs[name] = model_def

    def create_replica(self, name: str, group_id: int, append_init_args: Optional[List] = None,
                       append_init_kwargs: Optional[Dict] = None):
        assert group_id in self.managers, f"Group {group_id} does not exist"
        assert group_id not in self.model_groups[name], f"Model {name} is already created on group {group_id}"
        self.model_groups[name].append(group_id)
        self.managers[group_id].create_replica(name, self.model_defs[name], append_init_args[0])

    def select_group_id(self, group_ids):
        best, best_size = -1, float("inf")
        for g in group_ids:
            if self.queue_size[g] < best_size:
                best, best_size = g, self.queue_size[g]
        assert best != -1
        return best

    def sync(self):
        pass


class Client:
    """Submits a workload and keeps per-request start / finish / good (controller.py:214-253)."""

    def __init__(self, controller: Controller, debug: bool = False):
        self.controller = controller
        self.debug = debug
        self.res_dict = {}

    def submit_workload(self, workload: Workload):
        ctl = self.controller
        n = len(workload)
        start, finish, good = np.zeros(n), np.zeros(n), np.zeros(n, dtype=bool)
        self.res_dict[workload] = (start, finish, good)
        http_overheads = np.abs(np.random.normal(loc=0.0025, scale=0.0005, size=(n,)))

        heap, order = [], count()
        SUBMIT, DISPATCH, MANAGE, STAGE = range(4)
        for i in range(n):
            heapq.heappush(heap, (workload.arrivals[i], next(order), SUBMIT, i, -1, 0))

        def answer(i, now, group, served):
            if group >= 0:  # back in the controller (:207-211)
                ctl.queue_size[group] -= 1
                ctl.num_total_requests[group] += 1
            finish[i] = now
            good[i] = bool((now - start[i]) <= workload.requests[i].slo and served)

        while heap:
            now, _, kind, i, g, k = heapq.heappop(heap)
            req = workload.requests[i]
            if kind == SUBMIT:
                start[i] = now
                heapq.heappush(heap, (http_overheads[i] + now, next(order), DISPATCH, i, -1, 0))
            elif kind == DISPATCH:
                assert req.model_name in ctl.model_groups, f"Model '{req.model_name}' is not registered."
                groups = ctl.model_groups[req.model_name]
                if not groups:
                    answer(i, now, -1, False)
                    continue
                g = ctl.select_group_id(groups)
                ctl.queue_size[g] += 1
                heapq.heappush(heap, (next(ctl.dispatch_overhead) + now, next(order), MANAGE, i, g, 0))
            elif kind == MANAGE:
                mgr = ctl.managers[g]
                if req.slo is not None:
                    lat = mgr.latency_dict[req.model_name][1]
                    t, clocks = now, []
                    for s in range(len(lat)):
                        t = max(mgr.stage_clock[s], t) + lat[s]
                        clocks.append(t)
                    if clocks[-1] + mgr.fixed_overhead > start[i] + req.slo:
                        answer(i, now, g, False)
                        continue
                    mgr.stage_clock[:len(lat)] = clocks
                heapq.heappush(heap, (next(mgr.alpa_overhead) + now, next(order), STAGE, i, g, 0))
            else:
                mgr = ctl.managers[g]
                lat = mgr.latency_dict[req.model_name][1]
                if k == len(lat):
                    answer(i, now, g, True)
                    continue
                mgr.stream_clock[k] = max(mgr.stream_clock[k], now) + lat[k]
                heapq.heappush(heap, (now + (mgr.stream_clock[k] - now), next(order), STAGE, i, g, k + 1))

    def compute_stats(self, workload: Workload, warmup: float):
        start, finish, good = self.res_dict[workload]
        return workload.compute_stats(start, finish, good, warmup)


def simulate_one_case(case, warmup=DEFAULT_WARMUP, debug=False):
    """One serving case through the event-driven simulator (controller.py:257-279).
    Returns (StatsResult, placement)."""
    register_models, generate_workload, place_models = case
    controller = Controller()
    register_models(controller)
    placement = place_models(controller)
    client = Client(controller, debug=debug)
    workload = generate_workload()
    client.submit_workload(workload)
    stats = client.compute_stats(workload, warmup)
    stats.group_num_requests = tuple(controller.num_total_requests[g] for g in controller.managers)
    return stats, placement
