"""Pins the oracle's descent and level-0 search (restating
cpp/include/cuda_search_kernels.cuh:22-66 and :99-164 of the reference with
hnswlib's two-queue order): brute force on connected graphs, a hand-walked tiny
graph, invariants, and a literal Python model of libstdc++ heaps for tie cases."""
import numpy as np
import pytest

from helpers import gauss_mixture, integer_vectors, ring_graph


def flat_index(oracle, vectors, links0, dist_type, max_m0, labels=None):
  n = vectors.shape[0]
  return oracle.OracleIndex(dist_type).from_arrays(
      vectors, np.zeros(n, np.int32), links0, np.zeros(0, np.uint32), max_m=4,
      max_m0=max_m0, maxlevel=0, enterpoint=0, labels=labels)


@pytest.mark.parametrize("dist_type", ["dot", "l2"])
def test_ef_ge_n_equals_brute_force(oracle, dist_type):
  n, d, k = 300, 17, 10
  x = gauss_mixture(n, d, seed=5, normalise=(dist_type == "dot"))
  q = gauss_mixture(20, d, seed=6, normalise=(dist_type == "dot"))
  ix = flat_index(oracle, x, ring_graph(n, 8), dist_type, 8)
  ids, dists, found = ix.search(q, k, n, convention="hnswlib")
  bf_ids, bf_d = oracle.bruteforce(x, q, k, dist_type)
  assert (found == k).all()
  assert (ids == bf_ids).all()
  assert (dists == bf_d).all()


def test_hand_walked_descent_and_search(oracle):
  # 1-d points on a line, L2.  level 1: 0 - 4 - 8; level 0: chain i <-> i+1
  pts = np.arange(10, dtype=np.float32)[:, None]
  levels = np.zeros(10, np.int32)
  levels[[0, 4, 8]] = 1
  max_m, max_m0 = 2, 2
  links0 = np.zeros((10, 3), np.uint32)
  for i in range(10):
    nb = [j for j in (i - 1, i + 1) if 0 <= j < 10]
    links0[i, 0] = len(nb)
    links0[i, 1:1 + len(nb)] = nb
  up = np.zeros((3, 3), np.uint32)
  up[0] = [1, 4, 0]       # node 0 -> 4
  up[1] = [2, 0, 8]       # node 4 -> 0, 8
  up[2] = [1, 4, 0]       # node 8 -> 4
  ix = oracle.OracleIndex("l2").from_arrays(pts, levels, links0, up.reshape(-1), max_m, max_m0,
                                            maxlevel=1, enterpoint=0)
  # query 6.2: level 1 walk 0 -> 4 (d 4.84) -> 8 (3.24): stops at 8
  assert ix.descend(np.array([[6.2]], np.float32))[0] == 8
  # query 5.9: 0 -> 4 (3.61); 8 is 4.41: stays at 4
  assert ix.descend(np.array([[5.9]], np.float32))[0] == 4
  ids, dists, found, cnt = ix.search(np.array([[6.2]], np.float32), 3, 3, counters=True)
  assert list(ids[0]) == [6, 7, 5] and found[0] == 3
  np.testing.assert_allclose(dists[0], [0.04, 0.64, 1.44], rtol=1e-5)
  # ef = 3 from entry 8: expands 8, 7, 6, 5 (4 hops); evaluates 8,7,9,6,5,4
  assert cnt[0, 1] == 4 and cnt[0, 0] == 6


def test_upper_counters_hand_count(oracle):
  pts = np.arange(10, dtype=np.float32)[:, None]
  levels = np.zeros(10, np.int32)
  levels[[0, 4, 8]] = 1
  links0 = ring_graph(10, 2, hops=(1,))
  up = np.array([[1, 4, 0], [2, 0, 8], [1, 4, 0]], np.uint32)
  ix = oracle.OracleIndex("l2").from_arrays(pts, levels, links0, up.reshape(-1), 2, 2, 1, 0)
  _, _, _, cnt = ix.search(np.array([[6.2]], np.float32), 1, 1, counters=True)
  # sweeps: at node 0 (1 evaluation), at node 4 (2), at node 8 (1) -> 3 sweeps, 4 evaluations
  assert cnt[0, 3] == 3 and cnt[0, 2] == 4


@pytest.mark.parametrize("dist_type", ["dot", "l2"])
def test_invariants(oracle, dist_type):
  n, d = 2000, 24
  x = gauss_mixture(n, d, seed=1, normalise=(dist_type == "dot"))
  q = gauss_mixture(50, d, seed=2, normalise=(dist_type == "dot"))
  levels = np.zeros(n, np.int32)
  ix = oracle.OracleIndex(dist_type).build(x, levels, 8, 16, 40, 0.0, threads=1)
  assert ix.validate() == 0
  for k, ef in ((1, 1), (10, 10), (10, 50), (25, 5)):
    ids, dists, found = ix.search(q, k, ef)
    assert (found == k).all()
    assert (np.diff(dists, axis=1) >= 0).all()
    for row, drow, qq in zip(ids, dists, q):
      assert len(set(row)) == k
      for i, dd in zip(row, drow):
        assert dd == oracle.api_distance(qq, x[i], dist_type)


def test_found_less_than_topk_on_small_component(oracle):
  # two components: {0,1,2} reachable from the entry, {3,4} not
  pts = np.arange(5, dtype=np.float32)[:, None]
  links0 = np.zeros((5, 3), np.uint32)
  links0[0] = [2, 1, 2]; links0[1] = [2, 0, 2]; links0[2] = [2, 0, 1]
  links0[3] = [1, 4, 0]; links0[4] = [1, 3, 0]
  ix = flat_index(oracle, pts, links0, "l2", 2)
  ids, dists, found = ix.search(np.array([[3.6]], np.float32), 5, 10)
  assert found[0] == 3 and list(ids[0, :3]) == [2, 1, 0]


def test_labels_are_returned_and_break_ties(oracle):
  # two nodes at the same distance: the lower LABEL comes first, whatever the internal id
  pts = np.array([[0.0], [1.0], [-1.0]], np.float32)
  links0 = np.array([[2, 1, 2], [2, 0, 2], [2, 0, 1]], np.uint32)
  ix = flat_index(oracle, pts, links0, "l2", 2, labels=np.array([100, 70, 50], np.uint64))
  ids, dists, found = ix.search(np.array([[0.0]], np.float32), 3, 3)
  assert list(ids[0]) == [100, 50, 70]
  ix = flat_index(oracle, pts, links0, "l2", 2, labels=np.array([100, 50, 70], np.uint64))
  ids, _, _ = ix.search(np.array([[0.0]], np.float32), 3, 3)
  assert list(ids[0]) == [100, 50, 70]


# ---- literal Python model of libstdc++ heaps + hnswlib search, for tie-rich inputs ----
def _push_heap(a, value, less):
  a.append(value)
  hole = len(a) - 1
  parent = (hole - 1) // 2
  while hole > 0 and less(a[parent], value):
    a[hole] = a[parent]
    hole = parent
    parent = (hole - 1) // 2
  a[hole] = value


def _pop_heap(a, less):
  if len(a) > 1:
    value = a[-1]
    ln = len(a) - 1
    hole = child = 0
    while child < (ln - 1) // 2:
      child = 2 * (child + 1)
      if less(a[child], a[child - 1]):
        child -= 1
      a[hole] = a[child]
      hole = child
    if ln % 2 == 0 and child == (ln - 2) // 2:
      child = 2 * (child + 1)
      a[hole] = a[child - 1]
      hole = child - 1
    parent = (hole - 1) // 2
    while hole > 0 and less(a[parent], value):
      a[hole] = a[parent]
      hole = parent
      parent = (hole - 1) // 2
    a[hole] = value
  a.pop()


def _model_search(vectors, links0, q, k, ef, ep=0):
  less = lambda x, y: x[0] < y[0]
  dist = lambda i: float(np.sum((q.astype(np.float64) - vectors[i].astype(np.float64)) ** 2))  # exact on small ints
  top, cand = [], []
  d0 = dist(ep)
  _push_heap(top, (d0, ep), less)
  _push_heap(cand, (-d0, ep), less)
  lower = d0
  seen = {ep}
  while cand:
    c = cand[0]
    if -c[0] > lower:
      break
    _pop_heap(cand, less)
    row = links0[c[1]]
    for n in row[1:1 + row[0]]:
      n = int(n)
      if n in seen:
        continue
      seen.add(n)
      d = dist(n)
      if len(top) < ef or lower > d:
        _push_heap(cand, (-d, n), less)
        _push_heap(top, (d, n), less)
        if len(top) > ef:
          _pop_heap(top, less)
        lower = top[0][0]
  while len(top) > k:
    _pop_heap(top, less)
  return sorted(top)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_tie_rich_search_matches_literal_model(oracle, seed):
  n, d, k, ef = 400, 6, 10, 24
  x = integer_vectors(n, d, seed=seed, hi=4)  # few distinct distances -> ties everywhere
  links0 = ring_graph(n, 8, hops=(1, 2, 7, 31))
  ix = flat_index(oracle, x, links0, "l2", 8)
  q = integer_vectors(25, d, seed=100 + seed, hi=4)
  ids, dists, found = ix.search(q, k, ef)
  for qi in range(q.shape[0]):
    want = _model_search(x, links0, q[qi], k, ef)
    assert [i for _, i in want] == list(ids[qi, :found[qi]])
    assert [dd for dd, _ in want] == [float(v) for v in dists[qi, :found[qi]]]


# ---- the reverse_cand search (farthest waiting entry first; cuda_utils_kernels.cuh:104-151) ----

def _far_model(x, rows, q, ep, k, ef, dist):
  """Plain-Python statement of the same search on a level-0-only index: a list kept sorted by
  a stable insert, the last entry not yet expanded goes next, a full list drops its last."""
  import bisect
  keys, ids, done = [dist(q, x[ep])], [ep], [False]
  seen = {ep}
  hops = 0
  while True:
    pick = next((i for i in range(len(ids) - 1, -1, -1) if not done[i]), -1)
    if pick < 0:
      break
    done[pick] = True
    hops += 1
    for nb in rows[ids[pick]]:
      if nb in seen:
        continue
      seen.add(nb)
      d = dist(q, x[nb])
      if len(ids) < ef or keys[-1] > d:
        pos = bisect.bisect_right(keys, d)
        keys.insert(pos, d); ids.insert(pos, nb); done.insert(pos, False)
        if len(ids) > ef:
          keys.pop(); ids.pop(); done.pop()
  return ids[:k], keys[:k], hops, len(seen)


@pytest.mark.parametrize("kind", ["gauss", "tiny_int"])
def test_reverse_cand_search_matches_plain_model(oracle, kind):
  n, d = 400, 6
  x = gauss_mixture(n, d, seed=31, normalise=False) if kind == "gauss" else integer_vectors(n, d, seed=31, hi=4)
  q = gauss_mixture(25, d, seed=32, normalise=False) if kind == "gauss" else integer_vectors(25, d, seed=32, hi=4)
  links0 = ring_graph(n, 6)
  rows = [list(r[1:1 + r[0]]) for r in links0]
  ix = flat_index(oracle, x, links0, "l2", 6)
  dist = lambda a, b: oracle.distance(a, b, "l2")
  for k, ef in ((5, 5), (10, 40), (3, 17)):
    ids, dists, found, cnt = ix.search(q, k, ef, convention="hnswlib", counters=True, reverse_cand=True)
    for r in range(q.shape[0]):
      m_ids, m_keys, hops, seen = _far_model(x, rows, q[r], 0, k, ef, dist)
      assert list(ids[r, :found[r]]) == m_ids and list(dists[r, :found[r]]) == m_keys
      assert cnt[r, 1] == hops and cnt[r, 0] == seen


def test_reverse_cand_search_with_ef_ge_n_is_brute_force(oracle):
  n, d, k = 300, 17, 10
  x = gauss_mixture(n, d, seed=5)
  q = gauss_mixture(20, d, seed=6)
  ix = flat_index(oracle, x, ring_graph(n, 8), "dot", 8)
  ids, dists, found = ix.search(q, k, n, convention="hnswlib", reverse_cand=True)
  bf_ids, bf_d = oracle.bruteforce(x, q, k, "dot")
  assert (found == k).all() and (ids == bf_ids).all() and (dists == bf_d).all()


def test_meets_ties_flags_exactly_the_queries_with_equal_keys(oracle):
  # tie-free data: nothing flagged; data on a coarse grid: everything flagged; and the flag
  # agrees with a direct look at the distances of all nodes a full search (ef >= N) accepts
  n, d = 300, 5
  x = gauss_mixture(n, d, seed=41, normalise=False)
  q = gauss_mixture(30, d, seed=42, normalise=False)
  ix = flat_index(oracle, x, ring_graph(n, 8), "l2", 8)
  assert not ix.meets_ties(q, n).any()
  xi = integer_vectors(n, 2, seed=43, hi=3)
  qi = integer_vectors(30, 2, seed=44, hi=3)
  ixi = flat_index(oracle, xi, ring_graph(n, 8), "l2", 8)
  assert ixi.meets_ties(qi, n).all()
  # one duplicated point: only queries are flagged for which it matters, i.e. all (ef >= N
  # accepts every node, the duplicate's key repeats)
  xd = x.copy(); xd[17] = xd[200]
  ixd = flat_index(oracle, xd, ring_graph(n, 8), "l2", 8)
  assert ixd.meets_ties(q, n).all()
