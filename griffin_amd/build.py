"""Build librglru_hip.so (hand-written gfx950 kernels + the C ABI) in-tree with hipcc.

    python -m griffin_amd.build            # compile griffin_amd/librglru_hip.so

hipcc cross-compiles without a GPU present, so this runs on a CPU-only machine.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "librglru_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["rglru_scan.hip", "rglru_fused.hip", "rglru_fused_bwd.hip", "rglru_decode.hip", "rglru_gate_gemm.hip",
           "rglru_block_ops.hip"]
ARCH = "gfx950"


def hipcc_path() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    candidate = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")
    if os.path.exists(candidate):
        return candidate
    raise RuntimeError("hipcc not found: the RG-LRU HIP library cannot be built")


def build(verbose: bool = False) -> str:
    """Compile every kernel for gfx950 and link the shared library; returns its path."""
    flags = [
        "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wno-unused-command-line-argument", "-ffp-contract=off", "-fno-strict-aliasing",
        "-I", os.path.join(os.path.dirname(HERE), "include"),
    ]
    noise = "is not a recognized feature for this target"
    logs: list[str] = []

    def run(cmd: list[str]) -> None:
        if verbose:
            print(" ".join(cmd))
        proc = subprocess.run(cmd, capture_output=True, text=True)
        log = "\n".join(line for line in (proc.stdout + proc.stderr).splitlines() if noise not in line)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + log)
        if log.strip():
            logs.append(log)

    # one object per source, compiled side by side, then one link
    tmp = LIB_PATH + ".tmp"
    with tempfile.TemporaryDirectory(prefix="rglru_build_") as objdir:
        objects = [os.path.join(objdir, os.path.splitext(s)[0] + ".o") for s in SOURCES]
        jobs = [[hipcc_path(), *flags, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objects)]
        with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
            list(pool.map(run, jobs))
        run([hipcc_path(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *objects, "-o", tmp])
    if verbose and logs:
        print("\n".join(logs))
    # A kernel template whose body the host pass cannot instantiate (seen with a target builtin called directly in a
    # __global__ template) loses its launch stub without any diagnostic; the library then links but does not load.
    missing = [line.split()[-1] for line in
               subprocess.run(["nm", "-D", "--undefined-only", tmp], capture_output=True, text=True).stdout.splitlines()
               if "__device_stub__" in line]
    if missing:
        os.remove(tmp)
        raise RuntimeError("hipcc produced a library with undefined kernel stubs (would not load): " + ", ".join(missing[:4]))
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
