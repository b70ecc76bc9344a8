"""Builds libmorello_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

`python -m morello_amd.build` compiles every translation unit under morello_amd/csrc and
links them into morello_amd/libmorello_amd.so.  hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmorello_amd.so")
OBJ_DIR = os.path.join(HERE, "build")
GEN_DIR = os.path.join(OBJ_DIR, "gen")   # generated assembly (the k loops of the two 256 x 256 tiles)
# generator -> the file the kernel header of the same tile includes
GENERATED = {"gen_gemm_wide.py": "gemm_wide_gfx950.inc", "gen_gemm_loop.py": "gemm_loop_gfx950.inc"}

SOURCES = ["api.hip", "generic.hip", "gemm_mfma.hip", "gemm_sched.hip", "gemm_nt.hip", "gemv.hip", "conv_gemm.hip", "conv_i8.hip", "conv_windows.hip", "conv_small.hip", "unfold.hip", "softmax.hip", "parts.hip", "mfma_rate.hip", "attention.hip", "plan.hip"]

# -packed-fp32-ops off: the compiler must not form v_pk_{add,mul,fma}_f32.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
    # The first kernel arguments (up to 14 dwords) arrive preloaded in SGPRs with the wave instead of
    # through a load the first instructions wait for: it takes a load's latency off the start of
    # kernels that only run for a few microseconds (k_conv_i8 and k_attn keep all of theirs within
    # the fourteen; a 3 us Softmax or conversion gains 0.2 us, the long kernels nothing).
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


# Per-file additions.
EXTRA_FLAGS = {}


def _hipcc() -> str:
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    # MRL_HIPCC_EXTRA: extra compiler arguments for one-off measurement builds (-D switches the kernels document)
    cmd = [_hipcc(), *FLAGS, *EXTRA_FLAGS.get(src, []), *os.environ.get("MRL_HIPCC_EXTRA", "").split(), "-I", GEN_DIR, "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def generate() -> None:
    """Runs the assembly generators.  Their output (2 MB of text) goes beside the object files, not
    into the source directory, and is never kept in the tree; a copy left in the source directory
    by an older build would shadow it (a quoted #include looks there first), so it is removed."""
    os.makedirs(GEN_DIR, exist_ok=True)
    for script, inc in GENERATED.items():
        stale = os.path.join(CSRC, inc)
        if os.path.exists(stale):
            os.remove(stale)
        res = subprocess.run([sys.executable, os.path.join(CSRC, script), os.path.join(GEN_DIR, inc)],
                             capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"{script} failed:\n{res.stdout}\n{res.stderr}")


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    generate()
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    # The process-level harness (stand-in for an emitted program) links against the library.
    harness = os.path.join(HERE, "mrl_harness")
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", os.path.join(CSRC, "harness_main.cpp"), "-o", harness,
           "-L" + HERE, "-lmorello_amd", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("harness build failed:\n" + res.stderr)
    if verbose:
        print(f"built {OUT} and {harness}")
    return OUT


if __name__ == "__main__":
    build()
