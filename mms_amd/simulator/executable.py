"""Carrier of a model's profile for registration calls.

The placement evaluator registers models as ``partial(Executable, profile)``
(reference base_policy.py:202-205) and the approximate simulator only reads
the ``ProfilingResult`` back out of that partial (controller.py:290-296).  The
reference's class additionally replays stage latencies on its event loop
(simulator/executable.py:31-46); here that replay is part of
``mms_amd.simulator.event_sim.Client.submit_workload``, which needs the
profile only.
"""
from mms_amd.profiling import ProfilingResult


class Executable:
    def __init__(self, profiling_result: ProfilingResult, parallel_config=None, virtual_mesh=None):
        self.profile = profiling_result
        self.parallel_config = parallel_config
        self.virtual_mesh = virtual_mesh
        if parallel_config is not None:
            self.stage_latency = profiling_result.para_dict[parallel_config].latency

