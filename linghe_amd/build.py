"""Build libfq_gfx950.so (the C-ABI library with the gfx950 kernels) in-tree.

    python -m linghe_amd.build

hipcc cross-compiles for gfx950 without a GPU.  The translation units are
compiled in parallel and linked into ``linghe_amd/libfq_gfx950.so``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libfq_gfx950.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["fq_api.hip", "fq_tile_kernels.hip", "fq_row_kernels.hip", "fq_router.hip", "fq_stream.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # parity with the fp32 CPU oracle needs separate mul/add roundings
    "-ffp-contract=off",
    # NaNs are not part of the contract of these kernels: lets fmaxf be a single
    # v_max_f32 (no canonicalisation) and DPP moves fold into their consumer
    "-fno-honor-nans",
    "-mno-amdgpu-ieee",
    # packed fp32 VALU ops are not to be generated for this machine pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the -packed-fp32-ops feature and says so: harmless
    err = "\n".join(l for l in proc.stderr.splitlines() if "not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, err))
    if err.strip():
        sys.stderr.write(err + "\n")


def build_library(extra_flags=(), verbose: bool = False, csrc: str = CSRC, out: str = LIB_PATH) -> str:
    """Compile the translation units under `csrc` and link them into `out`."""
    hipcc = _hipcc()
    objdir = os.path.join(os.path.dirname(os.path.abspath(out)), "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, "-c", os.path.join(csrc, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        _run(cmd)

    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        list(pool.map(compile_one, zip(SOURCES, objs)))
    tmp = out + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp])
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    print(build_library(verbose=True))
