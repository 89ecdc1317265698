"""Host-side behaviour that needs no GPU: option handling of the Python wrapper
(cuhnsw/pyhnsw.py:23-48 and cuhnsw/proto/config.proto:10-26 of the reference), the
level stream (pyhnsw.py:65-71), level/entry-point logic (cuhnsw_base.cu:130-156), the
C ABI's exports and error codes."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

from conftest import ROOT, write_options
from cuhnsw_amd import aux, capi, datasets


def test_library_exports_every_declared_symbol():
  header = open(os.path.join(ROOT, "include", "cuhnsw_amd.h")).read()
  declared = set(re.findall(r"\b(cuhnsw_[a-z0-9_]+)\s*\(", header))
  assert declared == set(capi.SYMBOLS)
  lib = ctypes.CDLL(capi.LIB_PATH)
  for name in declared:
    assert hasattr(lib, name), name


def test_option_defaults_and_aliases():
  opt = aux.get_opt_as_proto({})
  assert (opt.seed, opt.max_m, opt.max_m0, opt.ef_construction, opt.block_dim) == (777, 12, 24, 150, 32)
  assert opt.dist_type == "dot" and opt.heuristic_coef == 0.25 and opt.hyper_threads == 10.0
  assert opt.visited_list_size == 8192 and opt.visited_table_size == 0
  assert opt.save_remains is False and opt.nrz is False and opt.reverse_cand is False
  with pytest.raises(ValueError, match="unknown option"):
    aux.get_opt_as_proto({"ef_search": 50})
  with pytest.raises(ValueError):
    aux.get_opt_as_proto({"max_m": "12"})
  with pytest.raises(ValueError):
    aux.get_opt_as_proto({"nrz": 1})


def test_wrapper_init_rules():
  from cuhnsw_amd import CuHNSW
  h = CuHNSW({"max_m": 16})
  assert h.opt.level_mult == pytest.approx(1.0 / np.log(16))
  assert CuHNSW({"dist_type": "euclidean"}).opt.dist_type == "l2"
  c = CuHNSW({"dist_type": "cosine"})
  assert c.opt.dist_type == "dot" and c.opt.nrz is False  # alias first: nrz is not switched on (pyhnsw.py:31-33)
  assert CuHNSW({"dist_type": "ip"}).opt.dist_type == "dot"
  with pytest.raises(AssertionError):
    CuHNSW({"dist_type": "hamming"})
  with pytest.raises(AssertionError, match="invalid block dim"):
    CuHNSW({"block_dim": 48})
  assert repr(h.obj) == "<CuHNSWBind>"


def test_c_init_error_codes(tmp_path):
  e = capi.Engine()
  assert e.init(str(tmp_path / "nope.json")) == 1
  bad = str(tmp_path / "bad.json")
  open(bad, "w").write("{ not json")
  assert e.init(bad) == 1
  path, opt = write_options(tmp_path)
  assert e.init(path) == 0
  assert e._l.cuhnsw_last_error(e._h) == b""    # a successful call leaves no stale message behind
  opt["dist_type"] = "cosine"  # only dot / l2 reach the engine; anything else is an error there
  json.dump(opt, open(path, "w"))
  assert e.init(path) == 2
  assert e._l.cuhnsw_last_error(e._h) == b"invalid dist type cosine"   # the offending value, not the previous one
  opt["dist_type"] = "l2"
  for key, value in (("max_m", 65536), ("max_m0", 70000), ("max_m", 0), ("ef_construction", 0)):
    json.dump(dict(opt, **{key: value}), open(path, "w"))   # link counts are 16 bits wide in the index file
    assert e.init(path) == 1
    assert b"max_m" in e._l.cuhnsw_last_error(e._h) or b"ef_construction" in e._l.cuhnsw_last_error(e._h)
  json.dump(dict(opt, max_m=65535, max_m0=65535), open(path, "w"))
  assert e.init(path) == 0


def test_level_stream_is_numpy_legacy_mt19937():
  lv = datasets.random_levels(1000, 1.0 / np.log(12))
  np.random.seed(777)
  u = np.random.uniform(size=1000)
  assert (lv == (-np.log(np.maximum(u, 1e-10)) / np.log(12)).astype(np.int32)).all()
  # frozen values of the legacy stream (numpy guarantees RandomState's stream)
  assert u[0] == pytest.approx(0.15266373, abs=1e-8) and u[1] == pytest.approx(0.30235661, abs=1e-8)
  assert lv.dtype == np.int32 and lv.min() == 0 and lv.max() >= 2
  # population of level >= 1 is N / max_m on average
  big = datasets.random_levels(200000, 1.0 / np.log(12))
  assert abs((big >= 1).mean() - 1.0 / 12) < 0.003


def test_levels_and_entry_point(tmp_path):
  e = capi.Engine()
  path, _ = write_options(tmp_path, max_m=4, max_m0=8)
  assert e.init(path) == 0
  with pytest.raises(RuntimeError, match="set_data first"):
    e.set_random_levels(np.zeros(3, np.int32))
  e.set_data(np.zeros((6, 3), np.float32))
  with pytest.raises(RuntimeError, match="length"):
    e.set_random_levels(np.zeros(5, np.int32))
  e.set_random_levels(np.array([0, 2, 1, 2, 0, 1], np.int32))
  assert e.max_level == 2 and e.enter_point == 1  # first node reaching the maximum
  e.set_random_levels(np.zeros(6, np.int32))
  assert e.max_level == 0 and e.enter_point == 0  # all-zero levels: node 0 (undefined in the reference)
  with pytest.raises(RuntimeError, match="non-negative"):
    e.set_random_levels(np.array([0, -1, 0, 0, 0, 0], np.int32))
  with pytest.raises(RuntimeError, match="2d"):
    e.set_data(np.zeros(4, np.float32))


@pytest.mark.skipif(capi.has_device(), reason="checks the no-GPU error path")
def test_compute_calls_fail_loudly_without_gpu(tmp_path):
  e = capi.Engine()
  path, _ = write_options(tmp_path)
  assert e.init(path) == 0
  e.set_data(np.ones((4, 3), np.float32))
  e.set_random_levels(np.zeros(4, np.int32))
  with pytest.raises(RuntimeError, match="no HIP device"):
    e.build_graph()
  with pytest.raises(RuntimeError, match="no HIP device"):
    e.search_knn(np.ones((1, 3), np.float32), 1, 1)


def test_datasets_are_seeded_and_shaped():
  a, qa, spec = datasets.make("C1", n=2000, nq=50)
  b, qb, _ = datasets.make("C1", n=2000, nq=50)
  assert a.shape == (2000, 50) and qa.shape == (50, 50) and a.dtype == np.float32
  assert (a == b).all() and (qa == qb).all()
  np.testing.assert_allclose(np.linalg.norm(a, axis=1), 1.0, rtol=1e-5)
  s, _, _ = datasets.make("C3", n=1000, nq=10)
  assert s.shape == (1000, 128) and (s == np.rint(s)).all() and s.min() >= 0 and s.max() <= 218
  g, _, _ = datasets.make("C4", n=100, nq=10)
  assert g.shape == (100, 960) and g.min() >= 0 and g.max() <= 1
  assert spec["opt"]["level_mult"] == pytest.approx(1 / np.log(24))
  # the reference README's run shape: the C2 data (same seed), queries uniform on the unit sphere
  r, qr, rs = datasets.make("R1", n=500, nq=40)
  c2, _, _ = datasets.make("C2", n=500, nq=1)
  assert (r == c2).all() and qr.shape == (40, 50) and rs["topk"] == 100
  np.testing.assert_allclose(np.linalg.norm(qr, axis=1), 1.0, rtol=1e-5)
  assert abs(float(qr.mean())) < 0.05
