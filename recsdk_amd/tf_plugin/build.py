"""Builds librecsdk_tf_ops.so, the TensorFlow kernels of the reference's four custom ops over librecsdk_hip.so.

    python -m recsdk_amd.tf_plugin.build

Needs an importable TensorFlow (its headers and link flags come from tf.sysconfig).  Where TensorFlow is not installed
the build is skipped and build() returns None: nothing else in this repository needs the library.
"""
import importlib.util
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SRC = os.path.join(HERE, "recsdk_tf_ops.cc")
LIBDIR = os.path.join(os.path.dirname(HERE), "lib")
OUT = os.path.join(LIBDIR, "librecsdk_tf_ops.so")


def build(verbose=True):
    if importlib.util.find_spec("tensorflow") is None:
        if verbose:
            print("recsdk_amd.tf_plugin: TensorFlow is not installed here, skipping", file=sys.stderr)
        return None
    import tensorflow as tf

    os.makedirs(LIBDIR, exist_ok=True)
    cmd = (["g++", "-std=c++17", "-O2", "-shared", "-fPIC", SRC, "-o", OUT, "-I", os.path.join(ROOT, "include")]
           + tf.sysconfig.get_compile_flags() + tf.sysconfig.get_link_flags()
           + ["-L", LIBDIR, "-lrecsdk_hip", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build()
