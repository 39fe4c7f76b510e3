"""Builds libembcache_hip.so: Embcache::SwapManager and Embcache::FeatureFilter over librecsdk_hip.so, compiled against
the reference's own headers where they lie in the reference checkout (nothing is copied).

    python -m recsdk_amd.embcache.build

A maintainer of the reference swaps swap_manager.cpp and feature_filter.cpp for the two sources next to this file in
torchrec_embcache's build and links librecsdk_hip.so; this script does the same out of tree, together with the
reference's evict_feature_record.cpp (unchanged) that FeatureFilter's member needs.  Without a reference checkout the
build is skipped and build() returns None.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = os.environ.get("RECSDK_REFERENCE", "/root/reference")
CSRC = os.path.join(REF, "training", "torch_rec_v1", "torchrec_embcache", "src", "torchrec_embcache", "csrc")
LIBDIR = os.path.join(os.path.dirname(HERE), "lib")
OUTDIR = os.path.join(HERE, "_build")
OUT = os.path.join(OUTDIR, "libembcache_hip.so")
SHIM = os.path.join(OUTDIR, "libembcache_dropin_test.so")   # tests/embcache_dropin_shim.cpp over OUT


def flags():
    """compile flags shared with the test shim: the reference's headers, PyTorch's (the headers include c10), HIP's"""
    from torch.utils.cpp_extension import include_paths
    import torch
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    inc = ["-I" + CSRC, "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include"] + ["-I" + p for p in include_paths()]
    return ["-std=c++17", "-O2", "-fPIC", f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-D__HIP_PLATFORM_AMD__=1", "-w"] + inc


def build(verbose=True):
    if not os.path.isdir(CSRC):
        if verbose:
            print("recsdk_amd.embcache: no reference checkout, skipping", file=sys.stderr)
        return None
    os.makedirs(OUTDIR, exist_ok=True)
    srcs = [os.path.join(HERE, "swap_manager_hip.cpp"), os.path.join(HERE, "feature_filter_hip.cpp"),
            os.path.join(CSRC, "feature_filter", "evict_feature_record.cpp")]
    cmd = (["g++", "-shared", "-o", OUT] + flags() + srcs +
           ["-L" + LIBDIR, "-lrecsdk_hip", "-L/opt/rocm/lib", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN/../../lib", "-Wl,-rpath,/opt/rocm/lib"])
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # the entry points the GPU test drives the two classes through
    shim = (["g++", "-shared", "-o", SHIM] + flags() + [os.path.join(ROOT, "tests", "embcache_dropin_shim.cpp")] +
            ["-L" + OUTDIR, "-lembcache_hip", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print(" ".join(shim), flush=True)
    subprocess.check_call(shim)
    return OUT


if __name__ == "__main__":
    build()
