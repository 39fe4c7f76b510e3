"""Builds librecsdk_torch_ops.so: the reference's torch operator names (fbgemm::split_embedding_*) and its torch class
hybrid::IdsMapper for ROCm tensors over librecsdk_hip.so.  Host C++ only (no kernels); needs the installed PyTorch headers.

Run as `python -m recsdk_amd.torch_ops.build`; load with `recsdk_amd.torch_ops.load()` or
`torch.ops.load_library(recsdk_amd/lib/librecsdk_torch_ops.so)`.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIBDIR = os.path.join(ROOT, "recsdk_amd", "lib")
LIB = os.path.join(LIBDIR, "librecsdk_torch_ops.so")


def build(verbose=True):
    import torch
    from torch.utils.cpp_extension import include_paths

    if not os.path.isfile(os.path.join(LIBDIR, "librecsdk_hip.so")):
        raise RuntimeError("build librecsdk_hip.so first (python -m recsdk_amd.build)")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-D__HIP_PLATFORM_AMD__=1",
           "-DUSE_ROCM=1", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(rocm, "include")]
    cmd += ["-isystem" + p for p in include_paths()]
    cmd += [os.path.join(HERE, "fbgemm_ops.cpp"), os.path.join(HERE, "hybrid_ops.cpp"), "-L" + LIBDIR, "-lrecsdk_hip", "-L" + torch_lib, "-lc10", "-lc10_hip",
            "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
