"""Builds libspotlight_hip.so for gfx950 with hipcc, in-tree.

Run as ``python -m spotlight_amd.build``.  The library links against the HIP
runtime only; there is no torch in it.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libspotlight_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = ["pack.hip", "hamming.hip", "topk.hip", "attn.hip", "select_attend.hip", "fused_step.hip", "fused_step_f32_g1.hip", "fused_step_f32_g2.hip", "fused_step_f32_g4.hip", "fused_step_f32_g5.hip", "fused_step_bf16_g1.hip", "fused_step_bf16_g2.hip", "fused_step_bf16_g4.hip", "fused_step_bf16_g5.hip", "fused_step_f16_g1.hip", "fused_step_f16_g2.hip", "fused_step_f16_g4.hip", "fused_step_f16_g5.hip", "hash.hip", "hash_rows.hip", "cache.hip", "decode.hip"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libspotlight_hip.so cannot be built")
    return exe


STAMPS_LIB_PATH = os.path.join(HERE, "libspotlight_hip_stamps.so")


def build_library(verbose: bool = True, jobs: int = 4, stamps: bool = False) -> str:
    """Compile every kernel source and link the shared library.  Always
    recompiles; returns the path of the built library.  ``stamps``: the
    measurement build (-DSL_PHASE_STAMPS, csrc/phase_stamps.h) as a second
    library, libspotlight_hip_stamps.so, which SPOTLIGHT_HIP_LIB selects."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = _hipcc()
    objdir = os.path.join(CSRC, "build_stamps" if stamps else "build")
    os.makedirs(objdir, exist_ok=True)
    flags = HIPCC_FLAGS + (["-DSL_PHASE_STAMPS"] if stamps else [])
    lib_path = STAMPS_LIB_PATH if stamps else LIB_PATH

    def run(cmd) -> None:
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        # the host pass does not know the gfx feature named in HIPCC_FLAGS and says so; harmless
        noise = "'-packed-fp32-ops' is not a recognized feature"
        out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
        if out.strip():
            print(out, flush=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}")

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        run([hipcc, *flags, "-c", os.path.join(CSRC, src), "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", lib_path])
    return lib_path


if __name__ == "__main__":
    print(build_library(stamps="--stamps" in sys.argv[1:], jobs=8 if "-j8" in sys.argv[1:] else 4))
    sys.exit(0)
