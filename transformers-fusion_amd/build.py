"""Compiles the HIP sources under csrc/ into libtfq.so (gfx950 only), in-tree.

hipcc cross-compiles without a GPU, so this runs on a CPU-only machine; the
built library is what the tests, the smoke check and the benchmark load.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtfq.so")

SOURCES = ["tfq_api.hip", "tfq_codec.hip", "tfq_codec_short.hip", "tfq_gemv.hip", "tfq_chain.hip", "tfq_dense.hip", "tfq_gemv_generic.hip", "tfq_moe.hip", "tfq_gemm.hip",
           "tfq_lut.hip", "tfq_container.hip", "tfq_engines.hip"]

# -ffp-contract=off: the decode arithmetic is ordered to match the reference
#   bit for bit, fusion happens only where the source says fmaf.
# -packed-fp32-ops off: v_pk_*_f32 forms are not used on this target.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
] + os.environ.get("TFQ_EXTRA_HIPCC_FLAGS", "").split()


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_library(verbose: bool = False) -> str:
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc(), *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(f"[build] {src} FAILED\n{out}", file=sys.stderr)
        elif out.strip() and verbose:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    subprocess.check_call(cmd)
    return LIB


SHIMS = os.path.join(HERE, "libtfq_shims.so")


def build_shims(verbose: bool = False) -> str:
    """Host C++ (g++, no HIP): the reference-named C++ entry points over the C ABI."""
    cmd = ["g++", "-std=c++20", "-O2", "-fPIC", "-Wall", "-shared", os.path.join(CSRC, "tfq_shims.cpp"),
           "-o", SHIMS, "-L" + HERE, "-ltfq", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return SHIMS


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_shims(verbose=True))
