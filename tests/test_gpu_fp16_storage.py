"""Vectors stored as fp16 in device memory (the reference's switched-off HALF_PRECISION idea,
cpp/include/types.hpp:9-28).  Parity definition: the index is an index over the vectors ROUNDED
to fp16 (round to nearest even), queries stay fp32 and all arithmetic stays fp32 in the
canonical order — so the CPU oracle searching the rounded vectors must return the same ids,
distances and counters bit for bit.  The saved file holds the rounded vectors as fp32."""
import numpy as np
import pytest

from conftest import write_options
from helpers import gauss_mixture, integer_vectors, recall
from test_gpu_search import _check_parity, _engine, _levels

pytestmark = pytest.mark.gpu


def _half_engine(tmp_path, **opt):
  e = _engine(tmp_path, **opt)
  e.set_tunable("fp16_storage", 1)
  return e


CASES = [
    ("dot50", 12000, 50, "dot", 12, 24, "gauss"),          # one 64-element block, 14 of 16 chunks of a row in use
    ("l2_128_int", 8000, 128, "l2", 16, 32, "int"),        # integers below 2048: fp16 holds them exactly
    ("l2_24", 6000, 24, "l2", 8, 16, "gauss_raw"),         # rows shorter than one block, L2 (masked tail)
    ("dot96", 6000, 96, "dot", 16, 32, "gauss"),           # one and a half blocks
    ("l2_960", 2500, 960, "l2", 16, 32, "gauss_raw"),      # long rows: query in LDS
]


def _data(kind, n, d, seed):
  if kind == "gauss":
    return gauss_mixture(n, d, centres=150, seed=seed)
  if kind == "gauss_raw":
    return gauss_mixture(n, d, centres=100, seed=seed, normalise=False)
  return integer_vectors(n, d, seed=seed, hi=219)


@pytest.mark.parametrize("name,n,d,dist,max_m,max_m0,kind", CASES, ids=[c[0] for c in CASES])
def test_fp16_storage_build_and_search_match_the_oracle_on_rounded_vectors(oracle, tmp_path, name, n, d, dist, max_m, max_m0, kind):
  x = _data(kind, n, d, 71)
  q = _data(kind, 300, d, 72)
  mult = 1.0 / np.log(max_m)
  levels = _levels(n, mult, 73)
  e = _half_engine(tmp_path, dist_type=dist, max_m=max_m, max_m0=max_m0, ef_construction=80, heuristic_coef=0.0)
  e.set_data(x)
  e.set_random_levels(levels)
  e.build_graph()
  p = str(tmp_path / "h.idx")
  e.save_index(p)
  ix = oracle.OracleIndex(dist).load(p)
  assert ix.validate() == 0
  rounded = x.astype(np.float16).astype(np.float32)
  assert (ix.vectors() == rounded).all()            # the file holds what the kernels see
  if kind == "int":
    assert (rounded == x).all()
  for k, ef in ((10, 100), (1, 10), (50, 64), (10, 300)):
    _check_parity(oracle, ix, e, q, k, ef)
  # quality: against brute force over the ORIGINAL vectors, and against the fp32 build
  gt, _ = oracle.bruteforce(x, q, 10, dist)
  r_half = recall(e.search_knn(q, 10, 300)[0], gt)
  e32 = _engine(tmp_path, dist_type=dist, max_m=max_m, max_m0=max_m0, ef_construction=80, heuristic_coef=0.0)
  e32.set_data(x)
  e32.set_random_levels(levels)
  e32.build_graph()
  r_full = recall(e32.search_knn(q, 10, 300)[0], gt)
  print("recall@10 fp16 storage %.4f fp32 storage %.4f" % (r_half, r_full))
  assert r_half >= r_full - 0.01 and r_half >= 0.93


def test_fp16_storage_of_a_loaded_fp32_index(oracle, tmp_path):
  """An index file written with fp32 vectors, loaded into an engine with fp16 storage: the
  graph is kept, the vectors are rounded, and the oracle over the same graph with rounded
  vectors gives the same answers."""
  n, d = 5000, 40
  x = gauss_mixture(n, d, seed=81)
  q = gauss_mixture(200, d, seed=82)
  levels = _levels(n, 0.4, 83)
  base = oracle.OracleIndex("dot").build(x, levels, 8, 16, 50, 0.4)
  p = str(tmp_path / "f32.idx")
  base.save(p)
  e = _half_engine(tmp_path, dist_type="dot", max_m=8, max_m0=16)
  e.load_index(p)
  p2 = str(tmp_path / "f16.idx")
  e.save_index(p2)
  ix = oracle.OracleIndex("dot").load(p2)
  assert (ix.vectors() == x.astype(np.float16).astype(np.float32)).all()
  a, b = ix.links0(), base.links0()
  used = np.arange(1, a.shape[1])[None, :] <= b[:, :1]          # slots past the count are undefined in the format
  assert (a[:, 0] == b[:, 0]).all() and (a[:, 1:][used] == b[:, 1:][used]).all()
  _check_parity(oracle, ix, e, q, 10, 80)


def test_fp16_storage_is_chosen_before_the_vectors_arrive(tmp_path):
  e = _engine(tmp_path, dist_type="dot")
  e.set_data(gauss_mixture(100, 8, seed=1))
  with pytest.raises(RuntimeError, match="before"):
    e.set_tunable("fp16_storage", 1)
  e.set_tunable("fp16_storage", 0)                  # no change: accepted


def test_fp16_storage_through_the_python_class(oracle, tmp_path):
  from cuhnsw_amd import CuHNSW
  x = gauss_mixture(8000, 50, centres=100, seed=91)
  q = gauss_mixture(100, 50, centres=100, seed=92)
  h = CuHNSW({"dist_type": "dot", "max_m": 12, "max_m0": 24, "ef_construction": 100, "heuristic_coef": 0.0,
              "py_log_level": 1})
  h.obj.set_tunable("fp16_storage", 1)
  h.set_data(x)
  h.build()
  p = str(tmp_path / "py16.idx")
  h.save_index(p)
  ix = oracle.OracleIndex("dot").load(p)
  assert (ix.vectors() == x.astype(np.float16).astype(np.float32)).all()
  nns, dist, found = h.search_knn(q, 10, 200)
  o_ids, o_d, o_f = ix.search(q, 10, 200)
  assert (nns == o_ids).all() and (dist == o_d).all() and (found == o_f).all()
  gt, _ = oracle.bruteforce(x, q, 10, "dot")
  assert recall(nns, gt) >= 0.95
