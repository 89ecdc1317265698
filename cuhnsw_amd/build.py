"""Compiles the native parts in-tree: libcuhnsw_amd.so (HIP engine + C ABI, gfx950)
and the pybind11 module cuhnsw_bind that wraps it.

  python -m cuhnsw_amd.build
"""
import json
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


RESOURCES = os.path.join(HERE, "..", "profiles", "kernel_resources.json")


def _run(cmd):
  print("+", " ".join(cmd), flush=True)
  subprocess.check_call(cmd)


def _demangle(names):
  try:
    out = subprocess.run(["c++filt"] + names, capture_output=True, text=True, check=True).stdout.split("\n")
    return [o.strip() for o in out[:len(names)]]
  except (OSError, subprocess.CalledProcessError):
    return names


def build_lib():
  """Compiles the library and records, from the compiler's resource-usage remarks of this very build, what
  every kernel in it takes: registers, spills, scratch bytes, wavefronts per SIMD (profiles/kernel_resources.json;
  `python -m cuhnsw_amd.kernel_report` adds where in the first-pass kernels the scratch accesses sit)."""
  from cuhnsw_amd import kernel_report
  srcs = [os.path.join(CSRC, "engine.hip"), os.path.join(CSRC, "index_file.cpp")]
  cmd = [HIPCC] + HIP_FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-x", "hip"] + srcs + ["-o", LIB]
  print("+", " ".join(cmd), flush=True)
  r = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
  other = [l for l in r.stderr.split("\n") if "kernel-resource-usage" not in l and "not a recognized feature" not in l
           and not l.lstrip().startswith(("|", "^", "In file included from")) and "__launch_bounds__" not in l
           and "__global__" not in l]
  if "".join(other).strip():
    print("\n".join(l for l in other if l.strip()), file=sys.stderr)
  if r.returncode != 0:
    raise subprocess.CalledProcessError(r.returncode, cmd)
  usage = kernel_report.parse_remarks(r.stderr)
  names = sorted(usage)
  table = {plain: usage[mangled] for mangled, plain in zip(names, _demangle(names))}
  try:
    with open(RESOURCES, "w") as f:
      json.dump({"flags": HIP_FLAGS, "kernels": table}, f, indent=1, sort_keys=True)
      f.write("\n")
  except OSError as e:   # a read-only tree: the library is what matters
    print("kernel resources not recorded:", e, file=sys.stderr)
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
