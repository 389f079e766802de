"""CPU oracle for the placement-evaluation path -- TEST INFRASTRUCTURE ONLY.

Nothing under this folder is part of the shipped library.  It may be imported
only by the tests, by the smoke check and by the benchmark's CPU-baseline leg,
and only as the checker, never as the thing measured or shipped.
"""
