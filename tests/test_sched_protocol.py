"""The turn taking of the plain simulator's scheduled launch, checked on the CPU under ThreadSanitizer.

``sched_model.cpp`` restates the protocol of ``mms_amd/csrc/sim_mixed.hip`` (claim an item's word with an
acquiring compare-and-swap, simulate a segment from the parked state, park, release-store the next segment
number) with wavefronts as threads and the parked state as plain memory.  The sanitizer must find no data race
and the model's own checks must pass over many random workgroups (items of different sizes and segment counts,
1 to 8 regions, wavefronts that leave after 0, 1, 3 or very many fruitless looks); the same model with the memory
orders taken out must be reported as racy, which shows that the check can fail.  No GPU involved."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _build(tmp_path, name, extra):
    exe = str(tmp_path / name)
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-pthread", *extra,
           os.path.join(HERE, "sched_model.cpp"), "-o", exe]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        pytest.skip("this g++ cannot build with -fsanitize=thread: " + proc.stderr[-300:])
    return exe


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_turn_taking_has_no_data_race_and_completes_every_item(tmp_path):
    exe = _build(tmp_path, "sched_model", [])
    for seed in (1, 2, 3, 4):
        proc = subprocess.run([exe, str(seed), "250"], capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stdout + proc.stderr
        assert "data race" not in proc.stderr and proc.stdout.startswith("ok:"), proc.stdout + proc.stderr


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_the_same_protocol_without_its_memory_orders_is_reported(tmp_path):
    exe = _build(tmp_path, "sched_model_broken", ["-DSCHED_MODEL_BROKEN"])
    reported = False
    for seed in (3, 4, 5):
        proc = subprocess.run([exe, str(seed), "100"], capture_output=True, text=True, timeout=300)
        if "data race" in proc.stderr:
            reported = True
            break
    assert reported, "ThreadSanitizer saw no race in the protocol without acquire / release"
