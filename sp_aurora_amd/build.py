"""Builds libsp_aurora_hip.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

Usage:  python -m sp_aurora_amd.build        (cross-compiles; no GPU needed)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libsp_aurora_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
# (source, object, extra flags).  flash_fwd.hip makes three objects: the zigzag variants of the 16-bit forward kernel
# and the variants for tensors of 2 GiB and more per (batch, head) are translation units of their own, so that the
# parts of the longest compile run side by side; flash_bwd.hip likewise makes two.
# The forward kernels' softmax phase gains 1-3 % from the scheduler that maximises instruction-level
# parallelism; the backward kernels lose 2 % with it.
_FWD = ["-mllvm", "-amdgpu-sched-strategy=max-ilp"]
UNITS = [
    ("flash_fwd.hip", "flash_fwd.o", _FWD),
    ("flash_fwd.hip", "flash_fwd_zigzag.o", _FWD + ["-DSPA_FWD_ZIGZAG_UNIT"]),
    ("flash_fwd.hip", "flash_fwd_big.o", _FWD + ["-DSPA_FWD_BIG_UNIT"]),
    ("flash_fwd.hip", "flash_fwd_splitkv.o", _FWD + ["-DSPA_FWD_SPLITKV_UNIT"]),
    ("flash_bwd.hip", "flash_bwd.o", []),
    ("flash_bwd.hip", "flash_bwd_big.o", ["-DSPA_BWD_BIG_UNIT"]),
    ("spa_abi.hip", "spa_abi.o", []),
    ("merge.hip", "merge.o", []),
    ("decode_fwd.hip", "decode_fwd.o", []),
    ("relayout.hip", "relayout.o", []),
]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # packed fp32 VALU ops are kept off on purpose (scalar fp32 code only)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out:
        print(out)


def build(verbose: bool = True) -> str:
    """Compile every HIP source into sp_aurora_amd/libsp_aurora_hip.so and return its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    objdir = os.path.join(HERE, "_obj")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, obj) for _, obj, _ in UNITS]
    # the translation units are independent: compile them side by side (the attention files take most of the time)
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(len(UNITS), os.cpu_count() or 1)) as pool:
        jobs = [pool.submit(_run, [hipcc] + FLAGS + extra + ["-c", "-o", os.path.join(objdir, obj), os.path.join(CSRC, src)], verbose)
                for src, obj, extra in UNITS]
        for j in jobs:
            j.result()
    _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", LIB_PATH] + objs, verbose)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
