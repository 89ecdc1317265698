"""Shared helpers of the test-suite (small synthetic data, tiny hand-built graphs)."""
import numpy as np


def gauss_mixture(n, d, centres=32, seed=0, sigma=0.5, normalise=True):
  rng = np.random.default_rng(seed)
  c = rng.standard_normal((centres, d)).astype(np.float32)
  x = c[rng.integers(0, centres, n)] + np.float32(sigma) * rng.standard_normal((n, d)).astype(np.float32)
  if normalise:
    x /= np.linalg.norm(x, axis=1, keepdims=True)
  return x.astype(np.float32)


def integer_vectors(n, d, seed=0, hi=8):
  """Small-integer coordinates: squared L2 distances are exact in fp32 in any
  summation order and collide often (ties)."""
  rng = np.random.default_rng(seed)
  return rng.integers(0, hi, (n, d)).astype(np.float32)


def ring_graph(n, max_m0, hops=(1, 2)):
  """Level-0 links of a connected ring: node i links to i±h for h in hops."""
  links0 = np.zeros((n, 1 + max_m0), dtype=np.uint32)
  for i in range(n):
    nb = []
    for h in hops:
      for s in (+1, -1):
        j = (i + s * h) % n
        if j != i and j not in nb:
          nb.append(j)
    nb = nb[:max_m0]
    links0[i, 0] = len(nb)
    links0[i, 1:1 + len(nb)] = nb
  return links0


def recall(found_ids, truth_ids):
  k = truth_ids.shape[1]
  return float(np.mean([len(set(a) & set(b)) / k for a, b in zip(found_ids, truth_ids)]))
