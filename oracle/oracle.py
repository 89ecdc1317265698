"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module; the shipped package never does.  The C++ side (hnsw_oracle.cpp) says
which reference file:line every function restates.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "build", "liboracle.so")
DIST = {"dot": 0, "l2": 1}

_c_float_p = ctypes.POINTER(ctypes.c_float)
_c_int_p = ctypes.POINTER(ctypes.c_int)
_c_uint_p = ctypes.POINTER(ctypes.c_uint)
_c_ll_p = ctypes.POINTER(ctypes.c_longlong)
_c_u64_p = ctypes.POINTER(ctypes.c_uint64)


def build_lib():
  """Compile the oracle with g++ (a few seconds)."""
  subprocess.check_call(["make", "-C", _HERE, "-B", "build/liboracle.so"],
                        stdout=subprocess.DEVNULL)


_lib = None


def lib():
  global _lib
  if _lib is None:
    if not os.path.exists(_LIB_PATH):
      build_lib()
    l = ctypes.CDLL(_LIB_PATH)
    l.orc_create.restype = ctypes.c_void_p
    l.orc_free.argtypes = [ctypes.c_void_p]
    l.orc_error.restype = ctypes.c_char_p
    l.orc_error.argtypes = [ctypes.c_void_p]
    l.orc_load.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int]
    l.orc_save.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
    l.orc_from_arrays.argtypes = [
        ctypes.c_void_p, _c_float_p, ctypes.c_int, ctypes.c_int, _c_int_p,
        _c_uint_p, _c_uint_p, _c_u64_p, ctypes.c_int, ctypes.c_int,
        ctypes.c_int, ctypes.c_uint, ctypes.c_int, ctypes.c_double,
        ctypes.c_int]
    l.orc_build.argtypes = [
        ctypes.c_void_p, _c_float_p, ctypes.c_int, ctypes.c_int, _c_int_p,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_double, ctypes.c_int]
    l.orc_mark_deleted.argtypes = [ctypes.c_void_p, _c_uint_p, ctypes.c_int, ctypes.c_int]
    for name in ("orc_num_data", "orc_num_dims", "orc_maxlevel", "orc_max_m",
                 "orc_max_m0", "orc_validate", "orc_num_deleted"):
      getattr(l, name).argtypes = [ctypes.c_void_p]
    l.orc_enterpoint.argtypes = [ctypes.c_void_p]
    l.orc_enterpoint.restype = ctypes.c_uint
    l.orc_get_levels.argtypes = [ctypes.c_void_p, _c_int_p]
    l.orc_get_vectors.argtypes = [ctypes.c_void_p, _c_float_p]
    l.orc_get_labels.argtypes = [ctypes.c_void_p, _c_u64_p]
    l.orc_get_links.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                _c_uint_p]
    l.orc_get_links0.argtypes = [ctypes.c_void_p, _c_uint_p]
    l.orc_distance.restype = ctypes.c_float
    l.orc_distance.argtypes = [_c_float_p, _c_float_p, ctypes.c_int,
                               ctypes.c_int]
    l.orc_api_distance.restype = ctypes.c_float
    l.orc_api_distance.argtypes = [_c_float_p, _c_float_p, ctypes.c_int,
                                   ctypes.c_int]
    l.orc_search.argtypes = [
        ctypes.c_void_p, _c_float_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        _c_int_p, _c_float_p, _c_int_p, _c_ll_p, ctypes.c_int, ctypes.c_int]
    l.orc_search_far.argtypes = l.orc_search.argtypes
    l.orc_search_meets_ties.argtypes = [ctypes.c_void_p, _c_float_p, ctypes.c_int, ctypes.c_int,
                                        ctypes.POINTER(ctypes.c_ubyte), ctypes.c_int]
    l.orc_descend.argtypes = [ctypes.c_void_p, _c_float_p, ctypes.c_int,
                              _c_int_p]
    l.orc_select.argtypes = [ctypes.c_void_p, _c_uint_p, _c_float_p,
                             ctypes.c_int, ctypes.c_int, _c_uint_p]
    l.orc_select_ref.argtypes = [ctypes.c_void_p, _c_uint_p, _c_float_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                 ctypes.c_int, ctypes.c_int, _c_uint_p, _c_float_p, _c_ll_p]
    l.orc_set_vectors.argtypes = [ctypes.c_void_p, _c_float_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    l.orc_check_link_keys0.argtypes = [ctypes.c_void_p, _c_float_p, ctypes.c_int]
    l.orc_check_link_keys0.restype = ctypes.c_longlong
    l.orc_bruteforce.argtypes = [
        _c_float_p, ctypes.c_int, ctypes.c_int, _c_float_p, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, _c_int_p, _c_float_p, ctypes.c_int]
    _lib = l
  return _lib


def _f32(a):
  return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t):
  return a.ctypes.data_as(t)


def host_threads():
  """Host cores this process may use (container cpu share, not the machine's)."""
  try:
    return max(1, len(os.sched_getaffinity(0)))
  except AttributeError:
    return os.cpu_count() or 1


def distance(a, b, dist_type="dot"):
  """Ordering key of the search: 1 - dot (hnswlib convention) or squared L2."""
  a, b = _f32(a), _f32(b)
  return float(lib().orc_distance(_p(a, _c_float_p), _p(b, _c_float_p),
                                  a.shape[0], DIST[dist_type]))


def api_distance(a, b, dist_type="dot"):
  """Value returned by the cuhnsw API: -dot or squared L2."""
  a, b = _f32(a), _f32(b)
  return float(lib().orc_api_distance(_p(a, _c_float_p), _p(b, _c_float_p),
                                      a.shape[0], DIST[dist_type]))


def bruteforce(data, queries, k, dist_type="dot", threads=None):
  data, queries = _f32(data), _f32(queries)
  nq = queries.shape[0]
  ids = np.empty((nq, k), dtype=np.int32)
  dists = np.empty((nq, k), dtype=np.float32)
  lib().orc_bruteforce(_p(data, _c_float_p), data.shape[0], data.shape[1],
                       _p(queries, _c_float_p), nq, k, DIST[dist_type],
                       _p(ids, _c_int_p), _p(dists, _c_float_p),
                       threads or host_threads())
  return ids, dists


class OracleIndex:
  """hnswlib-semantics index: load/save (hnswlib file format), CPU build, search."""

  def __init__(self, dist_type="dot"):
    self._l = lib()
    self._h = ctypes.c_void_p(self._l.orc_create())
    self.dist_type = dist_type

  def __del__(self):
    if getattr(self, "_h", None):
      self._l.orc_free(self._h)
      self._h = None

  def load(self, path):
    if not self._l.orc_load(self._h, os.fsencode(path), DIST[self.dist_type]):
      raise RuntimeError(self._l.orc_error(self._h).decode())
    return self

  def save(self, path):
    if not self._l.orc_save(self._h, os.fsencode(path)):
      raise RuntimeError("oracle: cannot write " + str(path))

  def from_arrays(self, vectors, levels, links0, links_upper, max_m, max_m0,
                  maxlevel, enterpoint, labels=None, mult=0.0, efc=0):
    vectors = _f32(vectors)
    levels = np.ascontiguousarray(levels, dtype=np.int32)
    links0 = np.ascontiguousarray(links0, dtype=np.uint32)
    links_upper = np.ascontiguousarray(links_upper, dtype=np.uint32)
    n, d = vectors.shape
    assert links0.shape == (n, 1 + max_m0)
    assert links_upper.size == int(levels.sum()) * (1 + max_m)
    lab = None
    if labels is not None:
      labels = np.ascontiguousarray(labels, dtype=np.uint64)
      lab = _p(labels, _c_u64_p)
    self._l.orc_from_arrays(
        self._h, _p(vectors, _c_float_p), n, d, _p(levels, _c_int_p),
        _p(links0, _c_uint_p), _p(links_upper, _c_uint_p), lab, max_m, max_m0,
        maxlevel, enterpoint, DIST[self.dist_type], mult, efc)
    return self

  def build(self, data, levels, max_m, max_m0, ef_construction, mult,
            threads=None):
    data = _f32(data)
    levels = np.ascontiguousarray(levels, dtype=np.int32)
    self._l.orc_build(self._h, _p(data, _c_float_p), data.shape[0],
                      data.shape[1], _p(levels, _c_int_p),
                      DIST[self.dist_type], max_m, max_m0, ef_construction,
                      mult, threads or host_threads())
    return self

  num_data = property(lambda s: s._l.orc_num_data(s._h))
  num_dims = property(lambda s: s._l.orc_num_dims(s._h))
  maxlevel = property(lambda s: s._l.orc_maxlevel(s._h))
  enterpoint = property(lambda s: s._l.orc_enterpoint(s._h))
  max_m = property(lambda s: s._l.orc_max_m(s._h))
  max_m0 = property(lambda s: s._l.orc_max_m0(s._h))
  num_deleted = property(lambda s: s._l.orc_num_deleted(s._h))

  def mark_deleted(self, ids, mark=True):
    """hnswlib markDelete (unmarkDelete with mark=False) on internal ids; the marks are written by save()
    and honoured by search(): walked through, never returned."""
    ids = np.ascontiguousarray(ids, dtype=np.uint32).ravel()
    n = self._l.orc_mark_deleted(self._h, _p(ids, _c_uint_p), ids.size, 1 if mark else 0)
    if n < 0:
      raise ValueError("mark_deleted: id out of range")
    return n

  def levels(self):
    out = np.empty(self.num_data, dtype=np.int32)
    self._l.orc_get_levels(self._h, _p(out, _c_int_p))
    return out

  def vectors(self):
    out = np.empty((self.num_data, self.num_dims), dtype=np.float32)
    self._l.orc_get_vectors(self._h, _p(out, _c_float_p))
    return out

  def labels(self):
    out = np.empty(self.num_data, dtype=np.uint64)
    self._l.orc_get_labels(self._h, _p(out, _c_u64_p))
    return out

  def links(self, node, level):
    buf = np.empty(max(self.max_m0, self.max_m), dtype=np.uint32)
    n = self._l.orc_get_links(self._h, node, level, _p(buf, _c_uint_p))
    if n < 0:
      raise IndexError("node %d has no level %d" % (node, level))
    return buf[:n].copy()

  def links0(self):
    out = np.empty((self.num_data, 1 + self.max_m0), dtype=np.uint32)
    self._l.orc_get_links0(self._h, _p(out, _c_uint_p))
    return out

  def validate(self):
    return self._l.orc_validate(self._h)

  def descend(self, queries):
    queries = _f32(queries)
    out = np.empty(queries.shape[0], dtype=np.int32)
    self._l.orc_descend(self._h, _p(queries, _c_float_p), queries.shape[0],
                        _p(out, _c_int_p))
    return out

  def select(self, cand_ids, cand_dists, m):
    cand_ids = np.ascontiguousarray(cand_ids, dtype=np.uint32)
    cand_dists = _f32(cand_dists)
    out = np.empty(max(m, 1), dtype=np.uint32)
    n = self._l.orc_select(self._h, _p(cand_ids, _c_uint_p),
                           _p(cand_dists, _c_float_p), cand_ids.shape[0], m,
                           _p(out, _c_uint_p))
    return out[:n].copy()

  def set_vectors(self, vectors):
    """Vectors without a graph: enough for select_ref and distances by id."""
    vectors = _f32(vectors)
    self._l.orc_set_vectors(self._h, _p(vectors, _c_float_p), vectors.shape[0], vectors.shape[1],
                            DIST[self.dist_type])
    return self

  def select_ref(self, cand_ids, cand_keys, max_m, nn_num=0, save_remains=False, new_comer=-1):
    """The reference's SearchHeuristic on candidates given in ascending order of their key to the
    target.  Returns (ids, keys, pair_tests): the new link row and how many candidate-pick distances
    were evaluated."""
    cand_ids = np.ascontiguousarray(cand_ids, dtype=np.uint32)
    cand_keys = _f32(cand_keys)
    out_ids = np.empty(max(max_m, 1), dtype=np.uint32)
    out_keys = np.empty(max(max_m, 1), dtype=np.float32)
    tests = ctypes.c_longlong(0)
    deg = self._l.orc_select_ref(self._h, _p(cand_ids, _c_uint_p), _p(cand_keys, _c_float_p), cand_ids.shape[0],
                                 max_m, nn_num, int(bool(save_remains)), new_comer, _p(out_ids, _c_uint_p),
                                 _p(out_keys, _c_float_p), ctypes.byref(tests))
    return out_ids[:deg].copy(), out_keys[:deg].copy(), tests.value

  def check_link_keys0(self, keys0, threads=None):
    """Number of level-0 links whose stored key (keys0: N x max_m0) is not bitwise the canonical
    distance between the link's end points."""
    keys0 = _f32(keys0)
    assert keys0.shape == (self.num_data, self.max_m0)
    return int(self._l.orc_check_link_keys0(self._h, _p(keys0, _c_float_p), threads or host_threads()))

  def meets_ties(self, queries, ef_search, threads=None):
    """Per query: does the hnswlib search meet equal distances in its result set?"""
    queries = _f32(queries)
    out = np.zeros(queries.shape[0], dtype=np.uint8)
    self._l.orc_search_meets_ties(self._h, _p(queries, _c_float_p), queries.shape[0], ef_search,
                                  out.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), threads or host_threads())
    return out.astype(bool)

  def search(self, queries, topk, ef_search, threads=None, convention="api",
             counters=False, reverse_cand=False):
    """Returns (ids, distances, found[, counters]); rows ascending by
    (distance, label); entries beyond found[i] are undefined.
    counters columns: n_dist, n_hops, n_dist_upper, n_sweeps_upper, max_cand."""
    queries = _f32(queries)
    if queries.ndim == 1:
      queries = queries[None, :]
    nq = queries.shape[0]
    ids = np.full((nq, topk), -1, dtype=np.int32)
    dists = np.full((nq, topk), np.inf, dtype=np.float32)
    found = np.zeros(nq, dtype=np.int32)
    cnt = np.zeros((nq, 5), dtype=np.int64)
    fn = self._l.orc_search_far if reverse_cand else self._l.orc_search
    fn(self._h, _p(queries, _c_float_p), nq, topk, ef_search,
                       _p(ids, _c_int_p), _p(dists, _c_float_p),
                       _p(found, _c_int_p), _p(cnt, _c_ll_p),
                       threads or host_threads(),
                       1 if convention == "api" else 0)
    if counters:
      return ids, dists, found, cnt
    return ids, dists, found
