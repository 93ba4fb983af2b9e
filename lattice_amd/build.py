"""Builds ``liblattice_hip_q4.so`` for gfx950 with hipcc, in-tree, next to this file.

``python -m lattice_amd.build`` compiles every translation unit under ``csrc/``
(in parallel) and links them.  hipcc cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import os
import shlex
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblattice_hip_q4.so")
SOURCES = ["lq4_api.hip", "lq4_gemv.hip", "lq4_gemv_b1.hip", "lq4_gemv_dma.hip", "lq4_gemv_multi.hip", "lq4_gemv_i8.hip", "lq4_gemv_mfma.hip", "lq4_gemm.hip", "lq4_gemm_wreg.hip", "lq4_gemm_skinny.hip", "lq4_moe.hip", "lq4_moe_i8.hip", "lq4_moe_b1.hip", "lq4_topk.hip", "lq4_elementwise.hip", "lq4_q8.hip", "lq4_q3.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
_NOISE = "'-packed-fp32-ops' is not a recognized feature for this target"  # host pass only


def _run(cmd):
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if _NOISE not in l)
    if p.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{p.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    extra = shlex.split(os.environ.get("LQ4_CXXFLAGS", ""))  # e.g. -DNAME for experiments
    objs = [os.path.join(CSRC, s.replace(".hip", ".o")) for s in SOURCES]

    def compile_one(pair):
        src, obj = pair
        cmd = [hipcc, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        list(ex.map(compile_one, zip(SOURCES, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
