"""mms_amd: MI355X-native placement evaluation behind AlpaServe's Python API.

The package mirrors the module layout of the reference (``alpa_serve``) for
the placement-evaluation path only: ``profiling``, ``util``,
``simulator.workload``, ``simulator.controller`` and ``placement_policy``.
The request-loop simulators run as hand-written HIP kernels (gfx950) behind
the C-ABI library ``libmmsim`` (``mms_amd/csrc``, ``include/mmsim.h``).
"""
__version__ = "0.1.0"
