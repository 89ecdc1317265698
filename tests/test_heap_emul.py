"""The product's LDS heap code (cuhnsw_amd/csrc/heap_emul.h) must move elements
exactly as libstdc++'s std::priority_queue does — checked on the host with a
harness that replays tie-rich random push/pop sequences on both."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
  exe = str(tmp_path_factory.mktemp("heap") / "heap_check")
  subprocess.check_call(["g++", "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "cuhnsw_amd", "csrc"),
                         "-o", exe, os.path.join(ROOT, "tests", "cpu_harness", "heap_check.cpp")])
  return exe


@pytest.mark.parametrize("seed,ops,key_range", [(1, 20000, 16), (2, 20000, 2), (3, 20000, 1),
                                                (4, 8000, 1000), (5, 4000, 10 ** 7)])
def test_heap_matches_libstdcxx(harness, seed, ops, key_range):
  r = subprocess.run([harness, str(seed), str(ops), str(key_range)], capture_output=True, text=True)
  assert r.returncode == 0, r.stdout + r.stderr
