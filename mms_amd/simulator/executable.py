"""Carrier of a model's profile for registration calls.

The placement evaluator registers models as ``partial(Executable, profile)``
(reference base_policy.py:202-205) and the approximate simulator only reads
the ``ProfilingResult`` back out of that partial (controller.py:290-296).  The
reference's class additionally replays stage latencies on an event loop
(simulator/executable.py:7-46); that behaviour belongs to the event-driven
simulator and is not provided here.
"""
from mms_amd.profiling import ProfilingResult


class Executable:
    def __init__(self, profiling_result: ProfilingResult, parallel_config=None, virtual_mesh=None):
        self.profile = profiling_result
        self.parallel_config = parallel_config
        self.virtual_mesh = virtual_mesh
        if parallel_config is not None:
            self.stage_latency = profiling_result.para_dict[parallel_config].latency

    async def handle_request(self, request):
        raise NotImplementedError(
            "mms_amd provides the approximate simulator only; the event-driven "
            "simulator that would call this is outside its scope")
