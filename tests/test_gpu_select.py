"""Neighbour selection on the GPU (select_neighbors in cuhnsw_amd/csrc/kernels.h, the counterpart of the
reference's SearchHeuristic, cpp/include/cuda_build_kernels.cuh:68-162) against the CPU oracle's
statement of the same rule: the link row (ids and keys, slot by slot) and the degree must be equal on
random candidate lists — plain Alg. 4, with nn_num free picks (heuristic_coef) and with the
save_remains tail fill — for the three query layouts of the kernels (one / two float4 registers per
lane, LDS copy), dot and L2, fp32 and fp16 vector storage.  The harness kernel calls the very device
function the build kernels call.  And the shortcut for newcomers to a row the rule produced before (the
reference's new_comer, cpp/include/cuda_build_kernels.cuh:109-138): same row as the full rule on the merged
list, for one newcomer (where it is also the oracle's statement of the reference's shortcut) and for several."""
import ctypes
import os

import numpy as np
import pytest

from helpers import gauss_mixture, integer_vectors

pytestmark = pytest.mark.gpu
LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpu_harness", "libselect_replay.so")


def _cases(oracle, x, dist, n_cases, seed):
  rng = np.random.default_rng(seed)
  n = x.shape[0]
  ix = oracle.OracleIndex(dist).set_vectors(x)
  ids, keys, off, ms, nns, saves, want = [], [], [0], [], [], [], []
  for _ in range(n_cases):
    target = int(rng.integers(0, n))
    t = int(rng.integers(1, 201))                       # what a construction search hands over: up to ef_construction
    # candidates as a search returns them (the target's neighbourhood, chosen by an approximate distance)
    # plus a few far ones; their keys are the oracle's canonical fp32 values
    approx = (1.0 - x @ x[target]) if dist == "dot" else ((x - x[target]) ** 2).sum(1)
    approx[target] = np.inf
    near = np.argsort(approx, kind="stable")[:max(1, t - 3)]
    far = rng.choice(n, size=3, replace=False)
    c_ids = np.unique(np.concatenate([near, far[far != target]])).astype(np.uint32)
    c_keys = np.array([oracle.distance(x[target], x[c], dist) for c in c_ids], np.float32)
    order = np.lexsort((c_ids, c_keys))
    c_ids, c_keys = c_ids[order], c_keys[order]
    m = int(rng.choice([12, 24, 16, 32, 5]))
    nn_num = int(np.float32(m) * np.float32(rng.choice([0.0, 0.0, 0.25, 0.5])))
    save = int(rng.random() < 0.3)
    ids.append(c_ids); keys.append(c_keys); off.append(off[-1] + len(c_ids))
    ms.append(m); nns.append(nn_num); saves.append(save)
    want.append(ix.select_ref(c_ids, c_keys, m, nn_num=nn_num, save_remains=bool(save))[:2])
  return (np.concatenate(ids), np.concatenate(keys), np.array(off, np.int32), np.array(ms, np.int32),
          np.array(nns, np.int32), np.array(saves, np.int32), want)


@pytest.mark.parametrize("dist,d,kind,half", [
    ("dot", 50, "gauss", 0), ("l2", 50, "gauss_raw", 0), ("dot", 128, "gauss", 0), ("l2", 128, "int", 0),
    ("dot", 960, "gauss", 0), ("l2", 960, "gauss_raw", 0), ("dot", 50, "gauss", 1), ("l2", 128, "int", 1),
    ("l2", 960, "gauss_raw", 1),
], ids=lambda v: str(v))
def test_select_neighbors_matches_the_oracle(oracle, dist, d, kind, half):
  if not os.path.exists(LIB):
    pytest.fail("tests/gpu_harness/libselect_replay.so is not built (run __graft_entry__.build())")
  lib = ctypes.CDLL(LIB)
  n = 3000
  if kind == "int":
    x = integer_vectors(n, d, seed=d, hi=219)           # equal keys and equal pair distances are common
  else:
    x = gauss_mixture(n, d, centres=20, seed=d, sigma=0.3, normalise=(kind == "gauss"))
  if half:
    x = x.astype(np.float16).astype(np.float32)         # the index IS an index over the rounded vectors
  n_cases = 1200
  c_ids, c_keys, off, ms, nns, saves, want = _cases(oracle, x, dist, n_cases, seed=7 * d + half)
  cap = 32
  out_ids = np.zeros((n_cases, cap), np.uint32)
  out_keys = np.zeros((n_cases, cap), np.float32)
  out_deg = np.zeros(n_cases, np.int32)
  vp, ci = ctypes.c_void_p, ctypes.c_int
  lib.select_replay.argtypes = [vp, ci, ci, ci, ci, ci, vp, vp, vp, vp, vp, vp, vp, ci, vp, vp, vp]
  x = np.ascontiguousarray(x)
  new_from = np.zeros(n_cases, np.uint32)
  print("select_replay", dist, d, kind, "half" if half else "fp32", n_cases, "cases", flush=True)
  rc = lib.select_replay(x.ctypes.data, n, d, 0 if dist == "dot" else 1, half, n_cases, c_ids.ctypes.data,
                         c_keys.ctypes.data, off.ctypes.data, ms.ctypes.data, nns.ctypes.data, saves.ctypes.data,
                         new_from.ctypes.data, cap, out_ids.ctypes.data, out_keys.ctypes.data, out_deg.ctypes.data)
  assert rc == 0
  pruned_somewhere = 0
  for i, (w_ids, w_keys) in enumerate(want):
    assert out_deg[i] == len(w_ids), "case %d" % i
    assert (out_ids[i, :len(w_ids)] == w_ids).all(), "case %d" % i
    assert (out_keys[i, :len(w_ids)] == w_keys).all(), "case %d" % i
    pruned_somewhere += len(w_ids) < min(ms[i], off[i + 1] - off[i])
  assert pruned_somewhere > n_cases // 10                # the heuristic did prune: the comparison is not vacuous


@pytest.mark.parametrize("dist,d,kind,half", [
    ("dot", 50, "gauss", 0), ("l2", 128, "int", 0), ("l2", 960, "gauss_raw", 0), ("dot", 96, "gauss", 1),
], ids=lambda v: str(v))
def test_newcomer_shortcut_gives_the_row_of_the_full_rule(oracle, dist, d, kind, half):
  """A row the rule produced, plus newcomers (the ids from new_from on): select_neighbors with new_from tests an old
  candidate only against the newcomers picked before it.  The row must be the one the full rule selects from the
  merged list — and, for a single newcomer, the one the oracle's statement of the reference's own shortcut selects."""
  if not os.path.exists(LIB):
    pytest.fail("tests/gpu_harness/libselect_replay.so is not built (run __graft_entry__.build())")
  lib = ctypes.CDLL(LIB)
  n, split = 3000, 2600                                   # ids from `split` on play the newcomers
  if kind == "int":
    x = integer_vectors(n, d, seed=d + 1, hi=219)
  else:
    x = gauss_mixture(n, d, centres=20, seed=d + 1, sigma=0.3, normalise=(kind == "gauss"))
  if half:
    x = x.astype(np.float16).astype(np.float32)
  rng = np.random.default_rng(11 * d + half)
  ix = oracle.OracleIndex(dist).set_vectors(x)
  n_cases = 600
  ids, keys, off, ms, want = [], [], [0], [], []
  took_shortcut = changed = 0
  for i in range(n_cases):
    target = int(rng.integers(0, split))
    approx = (1.0 - x @ x[target]) if dist == "dot" else ((x - x[target]) ** 2).sum(1)
    approx[target] = np.inf
    m = int(rng.choice([12, 24, 16, 32]))
    old = np.argsort(np.where(np.arange(n) < split, approx, np.inf), kind="stable")[:int(rng.integers(m, 4 * m))].astype(np.uint32)
    o_keys = np.array([oracle.distance(x[target], x[c], dist) for c in old], np.float32)
    order = np.lexsort((old, o_keys))
    row_ids, row_keys, _ = ix.select_ref(old[order], o_keys[order], m)          # the row as the rule left it
    n_new = 1 if i % 2 == 0 else int(rng.integers(2, 6))
    pool = np.argsort(np.where(np.arange(n) >= split, approx, np.inf), kind="stable")[:12]
    new = rng.choice(pool, size=n_new, replace=False).astype(np.uint32)
    n_keys = np.array([oracle.distance(x[target], x[c], dist) for c in new], np.float32)
    c_ids = np.concatenate([row_ids, new])
    c_keys = np.concatenate([row_keys, n_keys])
    order = np.lexsort((c_ids, c_keys))
    c_ids, c_keys = c_ids[order], c_keys[order]
    w_ids, w_keys, full_tests = ix.select_ref(c_ids, c_keys, m)                  # the full rule on the merged list
    if n_new == 1:
      r_ids, r_keys, short_tests = ix.select_ref(c_ids, c_keys, m, new_comer=int(new[0]))
      assert (r_ids == w_ids).all() and (r_keys == w_keys).all(), "case %d: the reference's shortcut differs from the full rule" % i
      took_shortcut += short_tests < full_tests
    changed += len(w_ids) != len(row_ids) or (w_ids != row_ids[:len(w_ids)]).any()
    ids.append(c_ids); keys.append(c_keys); off.append(off[-1] + len(c_ids)); ms.append(m); want.append((w_ids, w_keys))
  c_ids, c_keys = np.concatenate(ids), np.concatenate(keys)
  off, ms = np.array(off, np.int32), np.array(ms, np.int32)
  zeros = np.zeros(n_cases, np.int32)
  new_from = np.full(n_cases, split, np.uint32)
  cap = 32
  out_ids = np.zeros((n_cases, cap), np.uint32)
  out_keys = np.zeros((n_cases, cap), np.float32)
  out_deg = np.zeros(n_cases, np.int32)
  vp, ci = ctypes.c_void_p, ctypes.c_int
  lib.select_replay.argtypes = [vp, ci, ci, ci, ci, ci, vp, vp, vp, vp, vp, vp, vp, ci, vp, vp, vp]
  x = np.ascontiguousarray(x)
  print("select_replay with newcomers", dist, d, kind, "half" if half else "fp32", n_cases, "cases", flush=True)
  rc = lib.select_replay(x.ctypes.data, n, d, 0 if dist == "dot" else 1, half, n_cases, c_ids.ctypes.data,
                         c_keys.ctypes.data, off.ctypes.data, ms.ctypes.data, zeros.ctypes.data, zeros.ctypes.data,
                         new_from.ctypes.data, cap, out_ids.ctypes.data, out_keys.ctypes.data, out_deg.ctypes.data)
  assert rc == 0
  for i, (w_ids, w_keys) in enumerate(want):
    assert out_deg[i] == len(w_ids), "case %d" % i
    assert (out_ids[i, :len(w_ids)] == w_ids).all(), "case %d" % i
    assert (out_keys[i, :len(w_ids)] == w_keys).all(), "case %d" % i
  assert changed > n_cases // 10 and took_shortcut > n_cases // 10     # newcomers do get in, and the shortcut does save tests
