"""Pins the oracle's distance arithmetic (oracle/hnsw_oracle.cpp canon_dist), the
restatement of cpp/include/cuda_dist_kernels.cuh:112-124 of the reference:
closed forms in float64, exactness on integer-valued data, special cases."""
import numpy as np
import pytest

from helpers import integer_vectors


@pytest.mark.parametrize("d", [1, 3, 4, 50, 63, 64, 65, 96, 128, 200, 960, 1000])
def test_dot_and_l2_match_float64(oracle, d):
  rng = np.random.default_rng(d)
  a = rng.standard_normal(d).astype(np.float32)
  b = rng.standard_normal(d).astype(np.float32)
  dot64 = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
  l264 = float(np.sum((a.astype(np.float64) - b.astype(np.float64)) ** 2))
  scale = float(np.sum(np.abs(a.astype(np.float64) * b.astype(np.float64)))) + 1.0
  assert abs(oracle.distance(a, b, "dot") - (1.0 - dot64)) <= 1e-6 * scale
  assert abs(oracle.api_distance(a, b, "dot") - (-dot64)) <= 1e-6 * scale
  assert abs(oracle.distance(a, b, "l2") - l264) <= 1e-5 * l264 + 1e-12
  assert oracle.api_distance(a, b, "l2") == oracle.distance(a, b, "l2")


@pytest.mark.parametrize("d", [5, 50, 128, 333])
def test_exact_on_integer_data(oracle, d):
  x = integer_vectors(40, d, seed=d, hi=200)
  for i in range(0, 40, 2):
    a, b = x[i], x[i + 1]
    l2 = int(np.sum((a.astype(np.int64) - b.astype(np.int64)) ** 2))
    dot = int(np.dot(a.astype(np.int64), b.astype(np.int64)))
    assert l2 < 2 ** 24 and dot < 2 ** 24
    assert oracle.distance(a, b, "l2") == float(l2)
    assert oracle.api_distance(a, b, "dot") == float(-dot)
    assert oracle.distance(a, b, "dot") == float(np.float32(1.0) - np.float32(dot))


def test_symmetry_and_identity(oracle):
  rng = np.random.default_rng(3)
  a = rng.standard_normal(77).astype(np.float32)
  b = rng.standard_normal(77).astype(np.float32)
  for t in ("dot", "l2"):
    assert oracle.distance(a, b, t) == oracle.distance(b, a, t)
  assert oracle.distance(a, a, "l2") == 0.0
  # dropped term / wrong sign would show here: one-hot vectors
  e0 = np.zeros(9, np.float32); e0[0] = 2.0
  e8 = np.zeros(9, np.float32); e8[8] = 3.0
  assert oracle.distance(e0, e8, "l2") == 13.0
  assert oracle.api_distance(e0, e0, "dot") == -4.0
  assert oracle.distance(e0, e8, "dot") == 1.0


def test_canonical_order_is_64_partials_pairwise(oracle):
  """The summation order is part of the contract with the GPU kernels: element i
  goes to partial i mod 64 (fused multiply-add), partials combine pairwise."""
  rng = np.random.default_rng(11)
  for d in (50, 130, 960):
    a = (rng.standard_normal(d) * 1e3).astype(np.float32)
    b = (rng.standard_normal(d) * 1e-3).astype(np.float32)
    p = np.zeros(64, np.float64)  # float64 emulation of fp32 fma: product exact, one rounding
    p32 = np.zeros(64, np.float32)
    for i in range(d):
      p32[i % 64] = np.float32(np.float64(a[i]) * np.float64(b[i]) + np.float64(p32[i % 64]))
    s = 1
    while s < 64:
      for j in range(0, 64, 2 * s):
        p32[j] = np.float32(p32[j] + p32[j + s])
      s *= 2
    assert oracle.api_distance(a, b, "dot") == -p32[0]
