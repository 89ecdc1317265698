"""Builds the GPU test harnesses (tests only; compiled here, loaded on the GPU box)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libheap_replay.so")
SELECT_LIB = os.path.join(HERE, "libselect_replay.so")


def build():
  from cuhnsw_amd import build as native
  for src, lib in (("heap_replay.hip", LIB), ("select_replay.hip", SELECT_LIB)):
    cmd = [native.HIPCC] + native.HIP_FLAGS + ["-I" + os.path.join(ROOT, "cuhnsw_amd", "csrc"), "-x", "hip",
                                               os.path.join(HERE, src), "-o", lib]
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)
  return LIB
