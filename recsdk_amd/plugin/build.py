"""Builds the AccCTR plugin replacement, lib_ock_ctr_common.so, and its test driver.

The plugin implements the reference's plugin interface (ock::ctr::Factory / Unique / EmbCache::EmbCacheManager) on
librecsdk_hip.so, so it is compiled against the reference's own interface headers, read where they lie in a reference
checkout: <reference>/training/tf_rec_v1/src/AccCTR/src/include and .../common/util/error_code.h.  Nothing of the
reference is copied; without a checkout (RECSDK_REFERENCE_ROOT, default /root/reference) there is nothing to build
against and build() returns None.

Outputs, next to this file under _build/ (kept out of version control):
  lib_ock_ctr_common.so   what HybridMgmt dlopens; put its directory on LD_LIBRARY_PATH
  plugin_driver           tests/plugin_driver.cpp, the check the GPU test runs

Run as `python -m recsdk_amd.plugin.build`.  Pass --old-abi to compile with _GLIBCXX_USE_CXX11_ABI=0 (into
_build/old_abi/), which is how the reference builds AccCTR and what a TensorFlow 1.15 build of its host runtime needs.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_build")
PLUGIN = os.path.join(OUT, "lib_ock_ctr_common.so")
DRIVER = os.path.join(OUT, "plugin_driver")
# the same two files compiled with _GLIBCXX_USE_CXX11_ABI=0, as the reference builds AccCTR (AccCTR/src/CMakeLists.txt:30)
OUT_OLD_ABI = os.path.join(HERE, "_build", "old_abi")
PLUGIN_OLD_ABI = os.path.join(OUT_OLD_ABI, "lib_ock_ctr_common.so")
DRIVER_OLD_ABI = os.path.join(OUT_OLD_ABI, "plugin_driver")


def reference_includes():
    ref = os.environ.get("RECSDK_REFERENCE_ROOT", "/root/reference")
    src = os.path.join(ref, "training", "tf_rec_v1", "src", "AccCTR", "src")
    inc = [os.path.join(src, "include"), os.path.join(src, "common", "util")]
    if not all(os.path.isdir(d) for d in inc) or not os.path.isfile(os.path.join(inc[0], "factory.h")):
        return None
    return inc


def build(old_abi=False, verbose=True):
    inc = reference_includes()
    if inc is None:
        return None
    libdir = os.path.join(ROOT, "recsdk_amd", "lib")
    if not os.path.isfile(os.path.join(libdir, "librecsdk_hip.so")):
        raise RuntimeError("build librecsdk_hip.so first (python -m recsdk_amd.build)")
    out = OUT_OLD_ABI if old_abi else OUT
    plugin = PLUGIN_OLD_ABI if old_abi else PLUGIN
    driver = DRIVER_OLD_ABI if old_abi else DRIVER
    rpath = "$ORIGIN/../../../lib" if old_abi else "$ORIGIN/../../lib"
    os.makedirs(out, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    common = ["-std=c++17", "-O2", "-Wall", "-Wno-unused-function"]
    if old_abi:
        common.append("-D_GLIBCXX_USE_CXX11_ABI=0")
    common += ["-I" + d for d in inc]
    cmds = [
        # default visibility: callers of the reference's library link the interface's out-of-line members
        # (the InitializerInfo constructors, the initializer classes) from it, as the reference's core does
        [hipcc, *common, "-fPIC", "-shared", "-I" + os.path.join(ROOT, "include"),
         os.path.join(HERE, "ock_ctr_plugin.cpp"), "-L" + libdir, "-lrecsdk_hip", "-Wl,-rpath," + rpath,
         "-Wl,-soname,lib_ock_ctr_common.so", "-o", plugin],
        ["g++", *common, os.path.join(ROOT, "tests", "plugin_driver.cpp"), "-L" + out, "-l_ock_ctr_common",
         "-Wl,-rpath,$ORIGIN", "-ldl", "-lpthread", "-o", driver],
    ]
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return plugin, driver


if __name__ == "__main__":
    if build(old_abi="--old-abi" in sys.argv[1:]) is None:
        print("no reference checkout found: nothing built", file=sys.stderr)
        sys.exit(1)
