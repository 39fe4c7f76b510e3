"""Builds librecsdk_hip.so (the HIP kernels and their C ABI) for gfx950 with hipcc.

Run as `python -m recsdk_amd.build`; the shared library is written next to this file's
package as recsdk_amd/lib/librecsdk_hip.so.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "librecsdk_hip.so")

SOURCES = ["api.hip", "by_addr.hip", "dedup.hip", "tables.hip", "sparse.hip", "tbe.hip", "faae.hip", "swap.hip", "regroup.hip", "offset_mapper.hip", "host_rows.hip", "hot.hip", "ingest.hip", "ckpt.hip", "sort.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    # update formulas must round like their scalar definition (no fused multiply-add contraction)
    "-ffp-contract=off",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stderr=subprocess.PIPE, text=True)))
        objs.append(obj)
    failed = []
    for src, p in procs:   # wait for every compiler before reporting, so that none is left running
        _, err = p.communicate()
        # the host pass does not know the packed-fp32 feature name and says so once per function: harmless
        err = "\n".join(ln for ln in err.splitlines() if "packed-fp32-ops" not in ln)
        if err.strip():
            print(err, file=sys.stderr, flush=True)
        if p.returncode != 0:
            failed.append(src)
    if failed:
        raise RuntimeError("hipcc failed on " + ", ".join(failed))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
