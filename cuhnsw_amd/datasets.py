"""Seeded synthetic data sets of the benchmark configurations.

The shapes and laws are the ones the benchmark configs name (Gaussian mixtures,
optionally L2-normalised, or clipped/rounded for the SIFT/GIST-like cases).  The
seeds are frozen here: data uses default_rng(1000 + cfg), queries
default_rng(2000 + cfg).
"""
import numpy as np

CONFIGS = {
    # name: n, d, centres, law, options, queries, topk, ef list
    "C1": dict(cfg=1, n=100_000, d=50, centres=1000, law="gauss_nrz", nq=1000,
               topk=10, ef=[300],
               opt=dict(dist_type="dot", max_m=12, max_m0=24,
                        ef_construction=110, level_mult=1.0 / np.log(24.0))),
    "C2": dict(cfg=2, n=1_183_514, d=50, centres=1000, law="gauss_nrz",
               nq=10_000, topk=10, ef=[300],
               opt=dict(dist_type="dot", max_m=12, max_m0=24,
                        ef_construction=110)),
    "C3": dict(cfg=3, n=1_000_000, d=128, centres=2000, law="sift", nq=10_000,
               topk=10, ef=[64, 128, 300],
               opt=dict(dist_type="l2", max_m=16, max_m0=32,
                        ef_construction=200)),
    "C4": dict(cfg=4, n=1_000_000, d=960, centres=500, law="gist", nq=1000,
               topk=10, ef=[300],
               opt=dict(dist_type="l2", max_m=16, max_m0=32,
                        ef_construction=200)),
    "C5": dict(cfg=5, n=10_000_000, d=96, centres=10_000, law="gauss_nrz",
               nq=100_000, topk=100, ef=[64, 128, 256, 512],
               opt=dict(dist_type="dot", max_m=16, max_m0=32,
                        ef_construction=150)),
    # the run the reference's README times (examples/example1.py:206-226 there): the 1 183 514 x 50 angular
    # index, ONE batch of 1 000 000 random unit vectors as queries, topk 100, ef_search 300
    "R1": dict(cfg=2, n=1_183_514, d=50, centres=1000, law="gauss_nrz", query_law="unit_normal",
               nq=1_000_000, topk=100, ef=[300],
               opt=dict(dist_type="dot", max_m=12, max_m0=24,
                        ef_construction=110)),
}


def _centres(rng, law, k, d):
  if law == "gauss_nrz":
    return rng.standard_normal((k, d)).astype(np.float32)
  if law == "sift":
    return rng.uniform(0.0, 128.0, (k, d)).astype(np.float32)
  if law == "gist":
    return rng.uniform(0.0, 1.0, (k, d)).astype(np.float32)
  raise ValueError(law)


def _draw(rng, centres, law, n, chunk=262_144):
  k, d = centres.shape
  out = np.empty((n, d), dtype=np.float32)
  for s in range(0, n, chunk):
    e = min(n, s + chunk)
    pick = rng.integers(0, k, e - s)
    noise = rng.standard_normal((e - s, d)).astype(np.float32)
    if law == "gauss_nrz":
      x = centres[pick] + np.float32(0.5) * noise
      x /= np.linalg.norm(x, axis=1, keepdims=True)
    elif law == "sift":
      x = np.rint(np.clip(centres[pick] + np.float32(20.0) * noise, 0.0, 218.0))
    else:
      x = np.clip(centres[pick] + np.float32(0.05) * noise, 0.0, 1.0)
    out[s:e] = x
  return out


def make(name, n=None, nq=None):
  """Returns (data, queries, spec) of a named config; n / nq shrink it (same law,
  same centres) for tests."""
  spec = dict(CONFIGS[name])
  n = spec["n"] if n is None else n
  nq = spec["nq"] if nq is None else nq
  rng = np.random.default_rng(1000 + spec["cfg"])
  centres = _centres(rng, spec["law"], spec["centres"], spec["d"])
  data = _draw(rng, centres, spec["law"], n)
  qrng = np.random.default_rng(2000 + spec["cfg"])
  if spec.get("query_law") == "unit_normal":
    queries = qrng.standard_normal((nq, spec["d"])).astype(np.float32)
    queries /= np.linalg.norm(queries, axis=1, keepdims=True)
  else:
    queries = _draw(qrng, centres, spec["law"], nq)
  spec["n"], spec["nq"] = n, nq
  return data, queries, spec


def more_queries(name, nq, draw):
  """Another draw of nq queries from the law of a named config's own queries (draw = 0, 1, ...: the seed)."""
  spec = CONFIGS[name]
  qrng = np.random.default_rng(9000 + draw)
  if spec.get("query_law") == "unit_normal":
    queries = qrng.standard_normal((nq, spec["d"])).astype(np.float32)
    return queries / np.linalg.norm(queries, axis=1, keepdims=True)
  centres = _centres(np.random.default_rng(1000 + spec["cfg"]), spec["law"], spec["centres"], spec["d"])
  return _draw(qrng, centres, spec["law"], nq)


def random_levels(n, level_mult, seed=777):
  """Level stream of the Python wrapper (cuhnsw/pyhnsw.py:65-71 in the
  reference): legacy MT19937 uniform draws, truncated -ln(u) * mult."""
  np.random.seed(seed)
  u = np.maximum(np.random.uniform(size=n), 1e-10)
  return (-np.log(u) * level_mult).astype(np.int32)
