"""Pins the oracle's neighbour selection: the reference's SearchHeuristic
(cpp/include/cuda_build_kernels.cuh:68-162: HNSW Alg. 4 + nn_num free picks + save_remains tail
fill + the new_comer shortcut) and the hnswlib form the CPU build uses.

Nothing here repeats the oracle's loop.  The checks are (a) point sets whose answer follows from
geometry, each chosen so that one plausible mistake (comparing against the pick's distance to the
target instead of the candidate's, a non-strict comparison, an off-by-one in nn_num, a tail fill
in the wrong direction) gives another row; (b) a brute-force statement of Alg. 4 as a fixed
point ("c is kept iff no earlier kept r is strictly closer to c than the target is") evaluated with
exact integer arithmetic; (c) the properties that determine the output uniquely on tie-free data."""
import numpy as np
import pytest

from helpers import gauss_mixture, integer_vectors, recall


def _index(oracle, vectors, dist="l2"):
  return oracle.OracleIndex(dist).set_vectors(np.asarray(vectors, np.float32))


def _keys(oracle, vectors, target, ids, dist):
  return np.array([oracle.distance(vectors[target], vectors[i], dist) for i in ids], np.float32)


def _sorted_candidates(oracle, vectors, target, ids, dist):
  keys = _keys(oracle, vectors, target, ids, dist)
  order = np.lexsort((ids, keys))
  return np.asarray(ids, np.uint32)[order], keys[order]


# ---------------------------------------------------------------- (a) geometry
def test_collinear_points_keep_only_the_nearest(oracle):
  # target at 0, candidates at 1, 2, 3, 5 on a line: each later one is closer to the pick at 1
  pts = np.zeros((5, 3), np.float32)
  pts[1:, 0] = [1, 2, 3, 5]
  ix = _index(oracle, pts)
  ids, keys = _sorted_candidates(oracle, pts, 0, [1, 2, 3, 4], "l2")
  assert list(keys) == [1.0, 4.0, 9.0, 25.0]
  got, gk, tests = ix.select_ref(ids, keys, 3)
  assert list(got) == [1] and list(gk) == [1.0] and tests == 3
  # nn_num = 2: the two nearest pass untested, the third is tested against both
  got, _, tests = ix.select_ref(ids, keys, 3, nn_num=2)
  assert list(got) == [1, 2] and tests == 2          # candidate 3 is pruned by the first pick already
  # nn_num counts picks, so nn_num = 1 is plain Alg. 4 (the first pick is never tested anyway)
  assert list(ix.select_ref(ids, keys, 3, nn_num=1)[0]) == [1]
  # save_remains: pruned candidates fill the row from the back, in the order they were pruned
  got, gk, _ = ix.select_ref(ids, keys, 3, save_remains=True)
  assert list(got) == [1, 3, 2] and list(gk) == [1.0, 9.0, 4.0]
  got, _, _ = ix.select_ref(ids, keys, 4, save_remains=True)
  assert list(got) == [1, 4, 3, 2]
  got, _, _ = ix.select_ref(ids, keys, 2, save_remains=True)
  assert list(got) == [1, 2]                          # room for one pruned candidate only: the first


def test_orthogonal_axes_keep_everything_up_to_the_cap(oracle):
  # candidates a_i * e_i: D(c_i, c_j) = a_i^2 + a_j^2 > a_i^2 = D(c_i, target)
  d = 8
  pts = np.zeros((d + 1, d), np.float32)
  for i in range(d):
    pts[i + 1, i] = i + 1
  ix = _index(oracle, pts)
  ids, keys = _sorted_candidates(oracle, pts, 0, list(range(1, d + 1)), "l2")
  for m in (1, 3, 8, 12):
    got, gk, tests = ix.select_ref(ids, keys, m)
    h = min(m, d)
    assert list(got) == list(range(1, h + 1))
    assert list(gk) == [float(i * i) for i in range(1, h + 1)]
    assert tests == h * (h - 1) // 2                  # every pick was tested against all earlier picks
    got_sr, _, _ = ix.select_ref(ids, keys, m, save_remains=True)
    assert list(got_sr) == list(got)                  # nothing pruned, nothing to fill


def test_the_comparison_uses_the_candidates_distance_to_the_target(oracle):
  # r = (1,0): key 1; c = (2,1): key 5; D(c,r) = 2.  Pruned (2 < 5).  Comparing with the PICK's key
  # (2 < 1 is false) would keep it.
  pts = np.array([[0, 0], [1, 0], [2, 1]], np.float32)
  ix = _index(oracle, pts)
  ids, keys = _sorted_candidates(oracle, pts, 0, [1, 2], "l2")
  assert list(ix.select_ref(ids, keys, 4)[0]) == [1]
  # r = (3,0): key 9; c = (0,4): key 16; D(c,r) = 25: kept (25 > 16).  A reversed comparison would prune it.
  pts = np.array([[0, 0], [3, 0], [0, 4]], np.float32)
  ix = _index(oracle, pts)
  ids, keys = _sorted_candidates(oracle, pts, 0, [1, 2], "l2")
  assert list(ix.select_ref(ids, keys, 4)[0]) == [1, 2]


def test_equal_distances_do_not_prune(oracle):
  # target (0,0), pick r = (2,0): key 4; c = (1,2): key 5 and D(c,r) = 1 + 4 = 5: equal, so c is kept (the
  # reference prunes only on strictly greater, cuda_build_kernels.cuh:126, as hnswlib does).
  pts = np.array([[0, 0], [2, 0], [1, 2]], np.float32)
  ix = _index(oracle, pts)
  ids, keys = _sorted_candidates(oracle, pts, 0, [1, 2], "l2")
  assert list(keys) == [4.0, 5.0]
  assert list(ix.select_ref(ids, keys, 4)[0]) == [1, 2]
  assert list(ix.select(ids, keys, 2)) == [1, 2]     # hnswlib form, same rule


def test_new_comer_shortcut(oracle):
  # line again: target 0, existing links at 1 and 4, newcomer at 2 (ids: 1 -> x=1, 2 -> x=4, 3 -> x=2, 4 -> x=7)
  pts = np.zeros((5, 2), np.float32)
  pts[1:, 0] = [1, 4, 2, 7]
  ix = _index(oracle, pts)
  ids, keys = _sorted_candidates(oracle, pts, 0, [1, 2, 3, 4], "l2")
  assert list(ids) == [1, 3, 2, 4]
  # candidates ahead of the newcomer pass untested (1); the newcomer (x=2) is tested against the picks and
  # pruned (D = 1 < 4); it was never inserted, so everything after it passes untested as well
  got, _, tests = ix.select_ref(ids, keys, 4, new_comer=3)
  assert list(got) == [1, 2, 4] and tests == 1
  # newcomer first in the list: accepted, then every later candidate is tested against the newcomer alone
  pts2 = np.zeros((4, 2), np.float32)
  pts2[1:, 0] = [1, 3, -2]                             # newcomer id 1 at x=1; x=3 is closer to it (4 < 9): pruned;
  ix2 = _index(oracle, pts2)                           # x=-2 is not (9 > 4): kept
  ids2, keys2 = _sorted_candidates(oracle, pts2, 0, [1, 2, 3], "l2")
  got, _, tests = ix2.select_ref(ids2, keys2, 4, new_comer=1)
  assert list(ids2) == [1, 3, 2] and list(got) == [1, 3] and tests == 2
  # without the shortcut the same list gives the same picks here, by testing against all picks
  assert list(ix2.select_ref(ids2, keys2, 4)[0]) == [1, 3]


# ---------------------------------------------------------------- (b) brute force, exact integers
def _alg4_fixed_point(vectors, target, cand_ids, m):
  """HNSW Alg. 4 (keepPrunedConnections off, no extendCandidates) stated on exact integers:
  walk the candidates nearest first; c is kept iff fewer than m are kept and no kept r has
  D(c, r) < D(c, target)."""
  v = vectors.astype(np.int64)
  def d(a, b):
    return int(((v[a] - v[b]) ** 2).sum())
  order = sorted(cand_ids, key=lambda c: (d(c, target), c))
  kept = []
  for c in order:
    if len(kept) < m and all(d(c, r) >= d(c, target) for r in kept):
      kept.append(c)
  return kept


@pytest.mark.parametrize("seed", range(12))
def test_alg4_brute_force_on_integer_data(oracle, seed):
  rng = np.random.default_rng(seed)
  n, dim = 60, int(rng.integers(2, 9))
  x = integer_vectors(n, dim, seed=100 + seed, hi=int(rng.integers(4, 40)))
  ix = _index(oracle, x)
  checked_hnswlib_form = [0]
  for _ in range(40):
    target = int(rng.integers(0, n))
    pool = [i for i in range(n) if i != target]
    cand = [int(c) for c in rng.choice(pool, size=int(rng.integers(1, 21)), replace=False)]
    m = int(rng.integers(1, 13))
    ids, keys = _sorted_candidates(oracle, x, target, cand, "l2")
    want = _alg4_fixed_point(x, target, cand, m)
    got, gk, _ = ix.select_ref(ids, keys, m)
    assert list(got) == want
    assert list(gk) == [float(((x[c] - x[target]) ** 2).sum()) for c in want]
    # hnswlib's form returns its input untouched below m candidates and Alg. 4 otherwise (it
    # orders its candidates through a priority queue, which leaves the order among equal keys
    # to the heap: compared only where the keys are distinct)
    if len(set(keys.tolist())) == len(keys):
      hn = list(ix.select(ids, keys, m))
      assert hn == (want if len(cand) >= m else list(ids))
      checked_hnswlib_form[0] += 1
  assert checked_hnswlib_form[0] > 0 or dim < 4


# ---------------------------------------------------------------- (c) characterising properties
def _float64_dist(x, a, b, dist):
  if dist == "dot":
    return 1.0 - float(np.dot(x[a].astype(np.float64), x[b].astype(np.float64)))
  return float(((x[a].astype(np.float64) - x[b].astype(np.float64)) ** 2).sum())


@pytest.mark.parametrize("dist,dim", [("dot", 50), ("l2", 128), ("l2", 17), ("dot", 96)])
def test_properties_that_determine_the_row(oracle, dist, dim):
  rng = np.random.default_rng(dim)
  n = 400
  x = gauss_mixture(n, dim, centres=6, seed=dim, normalise=(dist == "dot"))
  ix = _index(oracle, x, dist)
  margin = 1e-4  # float64 closed form vs canonical fp32: comparisons closer than this are not judged
  for trial in range(60):
    target = int(rng.integers(0, n))
    cand = [int(c) for c in rng.choice([i for i in range(n) if i != target], size=int(rng.integers(2, 80)), replace=False)]
    m = int(rng.integers(1, 33))
    coef = float(rng.choice([0.0, 0.25, 0.5]))
    nn_num = int(np.float32(m) * np.float32(coef))
    ids, keys = _sorted_candidates(oracle, x, target, cand, dist)
    picks, pk, _ = ix.select_ref(ids, keys, m, nn_num=nn_num)
    picks = [int(p) for p in picks]
    # the picks are a subsequence of the candidate list: nearest first, each with its own key
    pos = [list(ids).index(p) for p in picks]
    assert pos == sorted(pos) and len(set(picks)) == len(picks) <= m
    assert list(pk) == [float(keys[p]) for p in pos]
    # the first nn_num picks are the first nn_num candidates
    assert picks[:nn_num] == [int(i) for i in ids[:min(nn_num, len(picks))]]
    # soundness: beyond the free picks nobody has an earlier pick strictly closer than the target
    for a, p in enumerate(picks):
      if a < nn_num:
        continue
      dt = _float64_dist(x, p, target, dist)
      assert all(_float64_dist(x, p, r, dist) >= dt - margin for r in picks[:a])
    # completeness: every candidate passed over while there was room has such a pick
    for j, c in enumerate(ids):
      c = int(c)
      if c in picks:
        continue
      before = [p for p, q in zip(picks, pos) if q < j]
      if len(before) >= m:
        continue
      dt = _float64_dist(x, c, target, dist)
      assert any(_float64_dist(x, c, r, dist) < dt + margin for r in before), (trial, c)
    # save_remains: same picks in front, then the first pruned candidates, last slot first
    row, _, _ = ix.select_ref(ids, keys, m, nn_num=nn_num, save_remains=True)
    row = [int(r) for r in row]
    assert len(row) == min(m, len(cand))
    assert row[:len(picks)] == picks
    pruned = [int(c) for c in ids if int(c) not in picks]
    assert row[len(picks):] == pruned[:len(row) - len(picks)][::-1]


def test_cpu_build_is_a_sane_quality_bar(oracle):
  """The hnswlib-style CPU build serves as the recall bar of the GPU build tests: it has to be a
  good graph itself (every invariant, recall@10 >= 0.95 at ef 300 against brute force)."""
  n, d = 6000, 32
  x = gauss_mixture(n, d, centres=50, seed=7)
  q = gauss_mixture(200, d, centres=50, seed=8)
  mult = 1.0 / np.log(12)
  levels = (-np.log(np.maximum(np.random.default_rng(9).uniform(size=n), 1e-10)) * mult).astype(np.int32)
  ix = oracle.OracleIndex("dot").build(x, levels, 12, 24, 100, mult)
  assert ix.validate() == 0
  gt, _ = oracle.bruteforce(x, q, 10, "dot")
  assert recall(ix.search(q, 10, 300)[0], gt) >= 0.95
