"""Device heap code (cuhnsw_amd/csrc/heap_coop.h) replayed on the GPU against the
literal libstdc++ model: the heap array must match slot by slot after every dump
point, including when it spills from LDS into global memory."""
import ctypes
import os
import random

import numpy as np
import pytest

import heap_model as hm

pytestmark = pytest.mark.gpu
LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpu_harness", "libheap_replay.so")


@pytest.mark.parametrize("minq,key_range,lds_cap,max_size", [
    (False, 16, 4096, 301), (True, 16, 4096, 3000), (False, 3, 64, 2000), (True, 1, 128, 700),
    (False, 10 ** 6, 4096, 5000), (True, 10 ** 6, 512, 5000),
])
def test_device_heap_matches_literal(minq, key_range, lds_cap, max_size):
  if not os.path.exists(LIB):
    pytest.fail("tests/gpu_harness/libheap_replay.so is not built (run __graft_entry__.build())")
  lib = ctypes.CDLL(LIB)
  rnd = random.Random(key_range + lds_cap)
  n_ops, dump_every, cap = 6000, 10, 8192
  keys = np.empty(n_ops, np.float32)
  lit, snaps, popped = [], [], []
  for op in range(n_ops):
    if not lit or (rnd.random() < 0.6 and len(lit) < max_size):
      keys[op] = float(rnd.randrange(key_range))
      hm.push_literal(lit, (float(keys[op]), op), minq)
      popped.append(-1)
    else:
      keys[op] = -1.0
      popped.append(lit[0][1])
      hm.pop_literal(lit, minq)
    if (op + 1) % dump_every == 0:
      snaps.append(list(lit))
  n_dumps = n_ops // dump_every
  dk = np.zeros((n_dumps, cap), np.float32)
  di = np.zeros((n_dumps, cap), np.uint32)
  sizes = np.zeros(n_dumps, np.int32)
  got_popped = np.zeros(n_ops, np.int32)
  vp = ctypes.c_void_p
  lib.heap_replay.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp]
  rc = lib.heap_replay(keys.ctypes.data, n_ops, int(minq), lds_cap, cap, dump_every, dk.ctypes.data, di.ctypes.data,
                       sizes.ctypes.data, got_popped.ctypes.data)
  assert rc == 0
  assert list(got_popped) == popped
  for i, snap in enumerate(snaps):
    assert sizes[i] == len(snap), "dump %d" % i
    assert [float(k) for k in dk[i, :len(snap)]] == [e[0] for e in snap], "dump %d" % i
    assert [int(v) for v in di[i, :len(snap)]] == [e[1] for e in snap], "dump %d" % i
