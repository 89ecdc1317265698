"""Compiles the native parts in-tree: libcuhnsw_amd.so (HIP engine + C ABI, gfx950)
and the pybind11 module cuhnsw_bind that wraps it.

  python -m cuhnsw_amd.build
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libcuhnsw_amd.so")
BIND = os.path.join(HERE, "cuhnsw_bind" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -ffp-contract=off: the distance arithmetic is written with explicit fused
# multiply-adds in a fixed order and must not be re-associated or re-fused.
# packed fp32 instructions are switched off for the device code.
HIP_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
  print("+", " ".join(cmd), flush=True)
  subprocess.check_call(cmd)


def build_lib():
  srcs = [os.path.join(CSRC, "engine.hip"), os.path.join(CSRC, "index_file.cpp")]
  _run([HIPCC] + HIP_FLAGS + ["-x", "hip"] + srcs + ["-o", LIB])
  return LIB


def build_bind():
  import pybind11
  inc = [
      "-I" + pybind11.get_include(),
      "-I" + sysconfig.get_paths()["include"],
      "-I" + os.path.join(HERE, "..", "include"),
  ]
  _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden"] +
       inc + [os.path.join(CSRC, "bindings.cc"), "-o", BIND,
              "-L" + HERE, "-lcuhnsw_amd", "-Wl,-rpath,$ORIGIN"])
  return BIND


def build_all():
  build_lib()
  build_bind()


if __name__ == "__main__":
  build_all()
  sys.exit(0)
