"""Builds libmmsim.so (HIP, gfx950 only) into the package folder.

    python -m mms_amd.csrc.build        # or: from mms_amd.csrc.build import build; build()

Every translation unit is compiled by hipcc for gfx950 with fp contraction
off, then linked into one shared library next to the Python package, where
``mms_amd._lib`` looks for it.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, "libmmsim.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["mmsim_api.hip", "sim_mixed.hip", "sim_batching.hip", "sim_scalar.hip", "stats.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


# The simulators run one or two wavefronts per SIMD (LDS decides how many), so instruction-level parallelism
# inside a wavefront is what hides latency: schedule for it.  Measured on the plain simulator (configuration 4 / its
# counts mode / configuration 3 / configuration 2 / its counts mode): iterative-ilp 534.3 / 606.5 / 24.1 / 4.56 /
# 4.84 ms, max-ilp 531.4 / 606.1 / 23.9 / 4.72 / 5.13 ms (half a per cent on the large batch, three to six per cent
# the other way on the small multi-stage batches that the searches send: iterative-ilp stays), iterative-minreg
# 527.9 / 612.4 / 30.1 ms, the default strategy 7 % behind; on the batching simulator max-ilp with the block
# alignment -1.6 % (iterative-ilp fails on it).
# Blocks that are only reached by a branch start on a 64-byte boundary: a taken branch costs a lone wavefront
# tens of cycles, less when its target starts an instruction cache line (measured: -1 % in the counts mode; 32- and
# 128-byte boundaries, aligning every block, and switching block placement or tail duplication off are all slower).
SOURCE_FLAGS = {"sim_mixed.hip": ["-mllvm", "-amdgpu-sched-strategy=iterative-ilp", "-mllvm", "-align-all-nofallthru-blocks=6"],
                "sim_batching.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp", "-mllvm", "-align-all-nofallthru-blocks=6"]}


def _compile(src, extra, src_dir=HERE, obj_dir=OBJ_DIR):
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *SOURCE_FLAGS.get(src, []), *extra, "-c", os.path.join(src_dir, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    noise = "packed-fp32-ops' is not a recognized feature"
    warn = [l for l in proc.stderr.splitlines() if l.strip() and noise not in l]
    return obj, "\n".join(warn)


def build(verbose=False, extra_flags=(), src_dir=HERE, out=OUT):
    """Compiles SOURCES from `src_dir` and links them into `out`."""
    obj_dir = os.path.join(src_dir, "build")
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(5, len(SOURCES))) as pool:
        results = list(pool.map(lambda s: _compile(s, list(extra_flags), src_dir, obj_dir), SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, w in results:
            if w:
                print(w, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return out


if __name__ == "__main__":
    print(build(verbose=True))
