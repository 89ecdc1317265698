"""ctypes binding of the C ABI (include/cuhnsw_amd.h) — the same entry points the
pybind11 module wraps, reachable without pybind11 (foreign-function callers, the
benchmark's device-pointer search)."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("CUHNSW_AMD_LIB") or os.path.join(_HERE, "libcuhnsw_amd.so")

SYMBOLS = [
    "cuhnsw_create", "cuhnsw_destroy", "cuhnsw_last_error", "cuhnsw_init",
    "cuhnsw_set_data", "cuhnsw_set_random_levels", "cuhnsw_build_graph",
    "cuhnsw_save_index", "cuhnsw_load_index", "cuhnsw_search_knn",
    "cuhnsw_search_knn_device", "cuhnsw_num_data", "cuhnsw_num_dims",
    "cuhnsw_max_level", "cuhnsw_enter_point", "cuhnsw_has_device",
    "cuhnsw_last_build_seconds", "cuhnsw_last_search_repeats", "cuhnsw_set_tunable",
    "cuhnsw_search_knn_device_noalloc", "cuhnsw_last_build_dropped_links", "cuhnsw_debug_link_keys0",
    "cuhnsw_last_build_counters", "cuhnsw_debug_gather_probe", "cuhnsw_last_search_trails",
    "cuhnsw_last_search_side_by_side", "cuhnsw_literal_fallbacks", "cuhnsw_trails_available",
    "cuhnsw_num_deleted",
]

_lib = None


def load():
  """Loads libcuhnsw_amd.so; raises OSError if it has not been built."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise OSError("libcuhnsw_amd.so is not built; run `python -m cuhnsw_amd.build`")
  l = ctypes.CDLL(LIB_PATH)
  vp, ci, cd = ctypes.c_void_p, ctypes.c_int, ctypes.c_double
  l.cuhnsw_create.argtypes = [ctypes.POINTER(vp)]
  l.cuhnsw_destroy.argtypes = [vp]
  l.cuhnsw_destroy.restype = None
  l.cuhnsw_last_error.argtypes = [vp]
  l.cuhnsw_last_error.restype = ctypes.c_char_p
  l.cuhnsw_init.argtypes = [vp, ctypes.c_char_p]
  l.cuhnsw_set_data.argtypes = [vp, vp, ci, ci]
  l.cuhnsw_set_random_levels.argtypes = [vp, vp, ci]
  l.cuhnsw_build_graph.argtypes = [vp]
  l.cuhnsw_save_index.argtypes = [vp, ctypes.c_char_p]
  l.cuhnsw_load_index.argtypes = [vp, ctypes.c_char_p]
  l.cuhnsw_search_knn.argtypes = [vp, vp, ci, ci, ci, vp, vp, vp]
  l.cuhnsw_search_knn_device.argtypes = [vp, vp, ci, ci, ci, vp, vp, vp, vp, ctypes.POINTER(ctypes.c_float)]
  l.cuhnsw_search_knn_device_noalloc.argtypes = [vp, vp, ci, ci, ci, vp, vp, vp, ctypes.POINTER(ctypes.c_float)]
  l.cuhnsw_last_build_dropped_links.argtypes = [vp]
  l.cuhnsw_debug_link_keys0.argtypes = [vp, vp, ctypes.c_longlong]
  l.cuhnsw_last_build_counters.argtypes = [vp, vp, ci]
  l.cuhnsw_debug_gather_probe.argtypes = [vp, ci, ci, ci, ctypes.POINTER(cd), ctypes.POINTER(ctypes.c_float)]
  for name in ("cuhnsw_num_data", "cuhnsw_num_dims", "cuhnsw_max_level", "cuhnsw_enter_point"):
    getattr(l, name).argtypes = [vp]
  l.cuhnsw_has_device.argtypes = []
  l.cuhnsw_last_build_seconds.argtypes = [vp]
  l.cuhnsw_last_build_seconds.restype = cd
  l.cuhnsw_last_search_repeats.argtypes = [vp]
  l.cuhnsw_last_search_trails.argtypes = [vp]
  l.cuhnsw_last_search_side_by_side.argtypes = [vp]
  l.cuhnsw_literal_fallbacks.argtypes = [vp]
  l.cuhnsw_trails_available.argtypes = [vp]
  l.cuhnsw_num_deleted.argtypes = [vp]
  l.cuhnsw_set_tunable.argtypes = [vp, ctypes.c_char_p, cd]
  _lib = l
  return l


def has_device():
  return bool(load().cuhnsw_has_device())


class Engine:
  """One engine handle; methods map 1:1 onto the C entry points and raise
  RuntimeError with the engine's message on failure."""

  def __init__(self):
    self._l = load()
    self._h = ctypes.c_void_p()
    if self._l.cuhnsw_create(ctypes.byref(self._h)) != 0:
      raise RuntimeError("cuhnsw_create failed: " + self._l.cuhnsw_last_error(None).decode())

  def close(self):
    if self._h:
      self._l.cuhnsw_destroy(self._h)
      self._h = ctypes.c_void_p()

  def __del__(self):
    try:
      self.close()
    except Exception:  # pylint: disable=broad-except
      pass

  def _check(self, rc):
    if rc != 0:
      raise RuntimeError(self._l.cuhnsw_last_error(self._h).decode())

  def init(self, opt_path):
    """0 ok, 1 unreadable option file, 2 invalid dist_type (no exception, like the C call)."""
    return self._l.cuhnsw_init(self._h, os.fsencode(opt_path))

  def set_data(self, data):
    data = np.ascontiguousarray(data, dtype=np.float32)
    if data.ndim != 2:
      raise RuntimeError("data must be 2d array")
    self._check(self._l.cuhnsw_set_data(self._h, data.ctypes.data, data.shape[0], data.shape[1]))

  def set_random_levels(self, levels):
    levels = np.ascontiguousarray(levels, dtype=np.int32)
    self._check(self._l.cuhnsw_set_random_levels(self._h, levels.ctypes.data, levels.shape[0]))

  def build_graph(self):
    self._check(self._l.cuhnsw_build_graph(self._h))

  def save_index(self, path):
    self._check(self._l.cuhnsw_save_index(self._h, os.fsencode(path)))

  def load_index(self, path):
    self._check(self._l.cuhnsw_load_index(self._h, os.fsencode(path)))

  def search_knn(self, queries, topk, ef_search):
    queries = np.ascontiguousarray(queries, dtype=np.float32)
    if queries.ndim == 1:
      queries = queries[None, :]
    if queries.shape[1] != self.num_dims:
      raise RuntimeError("query dimension differs from the index dimension")
    nq = queries.shape[0]
    nns = np.empty((nq, topk), dtype=np.int32)
    dists = np.empty((nq, topk), dtype=np.float32)
    found = np.empty(nq, dtype=np.int32)
    self._check(self._l.cuhnsw_search_knn(self._h, queries.ctypes.data, nq, topk, ef_search,
                                          nns.ctypes.data, dists.ctypes.data, found.ctypes.data))
    return nns, dists, found

  def search_knn_device(self, q_ptr, nq, topk, ef_search, nns_ptr, dist_ptr, found_ptr, stats_ptr=None):
    """All pointers are device addresses (ints).  Returns the kernel time in ms."""
    ms = ctypes.c_float(0.0)
    self._check(self._l.cuhnsw_search_knn_device(self._h, q_ptr, nq, topk, ef_search, nns_ptr, dist_ptr,
                                                 found_ptr, stats_ptr, ctypes.byref(ms)))
    return ms.value

  def search_knn_device_noalloc(self, q_ptr, nq, topk, ef_search, nns_ptr, dist_ptr, found_ptr):
    """The search that allocates nothing (device addresses as ints).  Returns the kernel time in ms."""
    ms = ctypes.c_float(0.0)
    self._check(self._l.cuhnsw_search_knn_device_noalloc(self._h, q_ptr, nq, topk, ef_search, nns_ptr, dist_ptr,
                                                         found_ptr, ctypes.byref(ms)))
    return ms.value

  def link_keys0(self, max_m0):
    """Keys stored with the level-0 links by the last build (needs tunable keep_link_keys)."""
    out = np.empty((self.num_data, max_m0), dtype=np.float32)
    self._check(self._l.cuhnsw_debug_link_keys0(self._h, out.ctypes.data, out.size))
    return out

  def gather_probe(self, waves_per_cu, rows_in_flight, dependent=True):
    """Random row gathers over the resident vectors alone: returns (rows fetched, kernel ms)."""
    rows, ms = ctypes.c_double(0.0), ctypes.c_float(0.0)
    self._check(self._l.cuhnsw_debug_gather_probe(self._h, waves_per_cu, rows_in_flight, int(bool(dependent)),
                                                  ctypes.byref(rows), ctypes.byref(ms)))
    return rows.value, ms.value

  def build_counters(self):
    """Work of the last build counted on the device (needs tunable build_counters): dict of two lists
    [evaluations, link rows read, heuristic pair tests, heuristic candidate rows, link rows written]."""
    out = np.zeros(10, dtype=np.uint64)
    if self._l.cuhnsw_last_build_counters(self._h, out.ctypes.data, 10) != 0:
      raise RuntimeError("cuhnsw_last_build_counters failed")
    return {"level0": [int(v) for v in out[:5]], "upper": [int(v) for v in out[5:]]}

  def set_tunable(self, name, value):
    rc = self._l.cuhnsw_set_tunable(self._h, name.encode(), float(value))
    if rc == -2:
      raise RuntimeError("tunable " + name + " has to be set before set_data / load_index")
    if rc != 0:
      raise RuntimeError("unknown tunable " + name)

  num_data = property(lambda s: s._l.cuhnsw_num_data(s._h))
  num_dims = property(lambda s: s._l.cuhnsw_num_dims(s._h))
  max_level = property(lambda s: s._l.cuhnsw_max_level(s._h))
  enter_point = property(lambda s: s._l.cuhnsw_enter_point(s._h))
  num_deleted = property(lambda s: s._l.cuhnsw_num_deleted(s._h))
  last_build_seconds = property(lambda s: s._l.cuhnsw_last_build_seconds(s._h))
  last_search_repeats = property(lambda s: s._l.cuhnsw_last_search_repeats(s._h))
  last_search_trails = property(lambda s: s._l.cuhnsw_last_search_trails(s._h))
  last_search_side_by_side = property(lambda s: bool(s._l.cuhnsw_last_search_side_by_side(s._h)))
  literal_fallbacks = property(lambda s: s._l.cuhnsw_literal_fallbacks(s._h))
  trails_available = property(lambda s: bool(s._l.cuhnsw_trails_available(s._h)))
  last_build_dropped_links = property(lambda s: s._l.cuhnsw_last_build_dropped_links(s._h))
