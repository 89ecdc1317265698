"""The cooperative (lane-parallel) heap algorithm the GPU kernels use must be
move-for-move identical to libstdc++'s heaps.  Here its lane-level model is checked
against the literal model on the CPU; tests/test_gpu_heap.py replays the same kind
of sequences through the real device code."""
import random

import pytest

import heap_model as hm


@pytest.mark.parametrize("minq", [False, True])
@pytest.mark.parametrize("key_range", [1, 3, 16, 10 ** 6])
def test_cooperative_model_equals_literal(minq, key_range):
  rnd = random.Random(key_range * 2 + minq)
  lit, coop, size = [], [], 0
  for step in range(12000):
    if not lit or (rnd.random() < 0.56 and len(lit) < 5000):
      v = (float(rnd.randrange(key_range)), step)
      hm.push_literal(lit, v, minq)
      size = hm.push_coop(coop, size, v, minq)
    else:
      hm.pop_literal(lit, minq)
      size = hm.pop_coop(coop, size, minq)
    assert size == len(lit) and coop[:size] == lit


def test_literal_model_is_a_heap_and_pops_in_order():
  rnd = random.Random(7)
  a = []
  for i in range(500):
    hm.push_literal(a, (float(rnd.randrange(50)), i))
  last = float("inf")
  while a:
    assert all(a[(i - 1) // 2][0] >= a[i][0] for i in range(1, len(a)))
    assert a[0][0] <= last
    last = a[0][0]
    hm.pop_literal(a)
