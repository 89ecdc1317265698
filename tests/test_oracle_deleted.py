"""Pins the oracle's search on an index with deleted elements (hnswlib markDelete: bit 0 of the third byte of
the level-0 count word; searchBaseLayerST in its has_deletions form).  The reference knows no deleted elements
(it reads the count word as a plain count, cpp/src/cuhnsw_base.cu:311-312); hnswlib is not available offline, so
the rule is pinned by what the mathematics fixes: with ef >= N on a connected level 0 the search walks the whole
graph, deleted elements included, and returns the exact top-k of the others; tiny graphs whose only bridge is a
deleted element (nearer or farther than the bound) tell the stop rule and the walk-through apart from the plain
search; and the marks survive the file format bit for bit."""
import struct

import numpy as np
import pytest

from helpers import gauss_mixture, integer_vectors, ring_graph


def flat_index(oracle, vectors, links0, dist_type, max_m0, enterpoint=0):
  n = vectors.shape[0]
  return oracle.OracleIndex(dist_type).from_arrays(
      vectors, np.zeros(n, np.int32), links0, np.zeros(0, np.uint32), max_m=4,
      max_m0=max_m0, maxlevel=0, enterpoint=enterpoint)


def chain_links(n):
  links0 = np.zeros((n, 3), np.uint32)
  for i in range(n):
    nb = [j for j in (i - 1, i + 1) if 0 <= j < n]
    links0[i, 0] = len(nb)
    links0[i, 1:1 + len(nb)] = nb
  return links0


@pytest.mark.parametrize("dist_type", ["dot", "l2"])
@pytest.mark.parametrize("share", [0.02, 0.4, 0.95])
def test_ef_ge_n_equals_brute_force_over_the_others(oracle, dist_type, share):
  n, d, k = 300, 17, 10
  x = gauss_mixture(n, d, seed=5, normalise=(dist_type == "dot"))
  q = gauss_mixture(20, d, seed=6, normalise=(dist_type == "dot"))
  ix = flat_index(oracle, x, ring_graph(n, 8), dist_type, 8)
  rng = np.random.default_rng(int(share * 100))
  dead = rng.choice(n, int(n * share), replace=False)
  assert ix.mark_deleted(dead) == dead.size
  alive = np.setdiff1d(np.arange(n), dead)
  ids, dists, found = ix.search(q, k, n, convention="hnswlib")
  bf_ids, bf_d = oracle.bruteforce(x[alive], q, k, dist_type)
  assert (found == k).all()
  assert (ids == alive[bf_ids]).all()
  assert (dists == bf_d).all()


def test_walks_through_a_deleted_bridge_nearer_than_the_bound(oracle):
  # points 0..5 on a line, chain links, entry 0, query beside 5: the walk has to pass the deleted 2 and 3
  pts = np.arange(6, dtype=np.float32)[:, None]
  ix = flat_index(oracle, pts, chain_links(6), "l2", 2)
  ix.mark_deleted([2, 3])
  ids, dists, found, cnt = ix.search(np.array([[5.2]], np.float32), 2, 1, counters=True)
  assert found[0] == 2 and list(ids[0]) == [5, 4]  # ef = max(ef, k) = 2
  # every element is evaluated once and expanded once: entry 0, then 1..5
  assert cnt[0, 0] == 6 and cnt[0, 1] == 6
  ids, _, found = ix.search(np.array([[5.2]], np.float32), 1, 1)
  assert found[0] == 1 and ids[0, 0] == 5


def test_a_short_result_queue_never_stops_the_search(oracle):
  # entry 0 at 0.0; its only link is the deleted X far away (10.0); behind X sits the element nearest to the
  # query.  The plain rule would stop at X (its key lies beyond the bound); with deleted elements hnswlib
  # stops only once the result queue is full.
  pts = np.array([[0.0], [10.0], [0.2], [0.3]], np.float32)
  links0 = np.zeros((4, 3), np.uint32)
  links0[0] = [1, 1, 0]
  links0[1] = [2, 0, 2]
  links0[2] = [2, 1, 3]
  links0[3] = [1, 2, 0]
  q = np.array([[0.21]], np.float32)
  ix = flat_index(oracle, pts, links0, "l2", 2)
  plain_ids, _, plain_found = ix.search(q, 3, 3)
  assert plain_found[0] == 3 and list(plain_ids[0]) == [2, 3, 0]  # (nothing deleted: everything is reachable)
  ix.mark_deleted([1])
  ids, _, found = ix.search(q, 3, 3)
  assert found[0] == 3 and list(ids[0]) == [2, 3, 0]
  # a full queue does stop it: ef = 1, result queue {0} is full when X's turn comes
  ids, _, found = ix.search(q, 1, 1)
  assert found[0] == 1 and ids[0, 0] == 0


def test_deleted_entry_point_and_nothing_left(oracle):
  pts = np.arange(6, dtype=np.float32)[:, None]
  ix = flat_index(oracle, pts, chain_links(6), "l2", 2)
  ix.mark_deleted([0])
  ids, _, found = ix.search(np.array([[0.1]], np.float32), 3, 3)
  assert found[0] == 3 and list(ids[0]) == [1, 2, 3]
  ix.mark_deleted(np.arange(6))
  assert ix.num_deleted == 6
  ids, _, found = ix.search(np.array([[0.1]], np.float32), 3, 10)
  assert found[0] == 0
  ix.mark_deleted(np.arange(6), mark=False)
  assert ix.num_deleted == 0
  ids, _, found = ix.search(np.array([[0.1]], np.float32), 3, 3)
  assert list(ids[0]) == [0, 1, 2]


def test_deleted_elements_on_the_upper_levels_are_walked_like_any_other(oracle):
  # level 1: 0 - 4 - 8, all three deleted: the descent still ends at 8 for a query at 6.2 (hnswlib's upper
  # loop looks at no mark); level 0 starts there and returns the others
  pts = np.arange(10, dtype=np.float32)[:, None]
  levels = np.zeros(10, np.int32)
  levels[[0, 4, 8]] = 1
  up = np.array([[1, 4, 0], [2, 0, 8], [1, 4, 0]], np.uint32)
  ix = oracle.OracleIndex("l2").from_arrays(pts, levels, chain_links(10), up.reshape(-1), 2, 2, maxlevel=1, enterpoint=0)
  ix.mark_deleted([0, 4, 8])
  q = np.array([[6.2]], np.float32)
  assert ix.descend(q)[0] == 8
  ids, _, found = ix.search(q, 3, 3)
  assert found[0] == 3 and list(ids[0]) == [6, 7, 5]


@pytest.mark.parametrize("dist_type", ["dot", "l2"])
def test_no_mark_is_the_plain_search_and_marks_survive_the_file(oracle, dist_type, tmp_path):
  n, d = 1500, 20
  x = gauss_mixture(n, d, seed=11, normalise=(dist_type == "dot"))
  q = gauss_mixture(40, d, seed=12, normalise=(dist_type == "dot"))
  mult = 1 / np.log(8)
  rng = np.random.default_rng(3)
  levels = (-np.log(np.maximum(rng.uniform(size=n), 1e-10)) * mult).astype(np.int32)
  ix = oracle.OracleIndex(dist_type).build(x, levels, 8, 16, 60, mult, threads=1)
  plain = ix.search(q, 10, 50, counters=True)
  dead = rng.choice(n, n // 3, replace=False)
  ix.mark_deleted(dead)
  marked = ix.search(q, 10, 50, counters=True)
  assert not np.isin(marked[0], dead).any() and (marked[2] == 10).all()
  # quality against brute force over the others
  alive = np.setdiff1d(np.arange(n), dead)
  bf_ids, _ = oracle.bruteforce(x[alive], q, 10, dist_type)
  hit = np.mean([len(set(marked[0][i]) & set(alive[bf_ids[i]])) / 10 for i in range(q.shape[0])])
  assert hit >= 0.9
  # the file: bit 16 of the count word of exactly the marked elements; load reads them back
  path = str(tmp_path / "marked.idx")
  ix.save(path)
  raw = open(path, "rb").read()
  rec = 16 * 4 + 4 + d * 4 + 8
  words = np.array([struct.unpack_from("<I", raw, 96 + i * rec)[0] for i in range(n)])
  assert (((words >> 16) & 1) == np.isin(np.arange(n), dead)).all()
  assert ((words >> 17) == 0).all()
  back = oracle.OracleIndex(dist_type).load(path)
  assert back.num_deleted == dead.size
  again = back.search(q, 10, 50, counters=True)
  for a, b in zip(marked, again):
    assert (a == b).all()
  # unmarked again: the plain search, bit for bit (the other form of the loop with nothing to skip)
  ix.mark_deleted(dead, mark=False)
  for a, b in zip(plain, ix.search(q, 10, 50, counters=True)):
    assert (a == b).all()


def test_ties_and_deleted_elements(oracle):
  """Integer data (equal keys everywhere): the answer never holds a deleted element, holds k others, and its
  keys are the k smallest keys among the others whenever ef covers the graph."""
  n, d = 400, 6
  x = integer_vectors(n, d, seed=2, hi=4)
  q = integer_vectors(30, d, seed=3, hi=4)
  ix = flat_index(oracle, x, ring_graph(n, 8), "l2", 8)
  dead = np.arange(0, n, 3)
  ix.mark_deleted(dead)
  alive = np.setdiff1d(np.arange(n), dead)
  ids, dists, found = ix.search(q, 10, n, convention="hnswlib")
  _, bf_d = oracle.bruteforce(x[alive], q, 10, "l2")
  assert (found == 10).all() and not np.isin(ids, dead).any()
  assert (dists == bf_d).all()
