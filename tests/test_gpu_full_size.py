"""Every benchmark configuration at its full size, checked through properties that do not need the
CPU oracle to search millions of points in a test: graph invariants of the saved file (the oracle's
validator reads it), found counts, ascending distances, distinct ids, returned distance == recomputed
distance, recall against an exact top-k (GPU matmul, harness only), the same answers from both search
paths and after a save / load round trip — and, on a sample of the queries, the oracle's search of the
very file the GPU wrote: ids, distances and found counts bit for bit, split into the queries whose
search meets equal distances and the rest."""
import os
import time

import numpy as np
import pytest

from conftest import write_options

pytestmark = pytest.mark.gpu


def _exact_topk(data, queries, k, dist):
  import torch
  dd = torch.from_numpy(data).cuda()
  qq = torch.from_numpy(queries).cuda()
  best_v = best_i = None
  cols = 1 << 19                       # score blocks of 2^28 elements at most
  rows = max(1, (1 << 28) // cols)
  out = []
  for r in range(0, queries.shape[0], rows):
    qs = qq[r:r + rows]
    best_v = best_i = None
    for c in range(0, data.shape[0], cols):
      blk = dd[c:c + cols]
      score = -(qs @ blk.T)
      if dist == "l2":
        score = (blk * blk).sum(1)[None, :] + 2.0 * score
      tv, ti = torch.topk(score, k, dim=1, largest=False)
      ti = ti + c
      if best_v is not None:
        tv, ti = torch.cat([best_v, tv], 1), torch.cat([best_i, ti], 1)
        tv, sel = torch.topk(tv, k, dim=1, largest=False)
        ti = torch.gather(ti, 1, sel)
      best_v, best_i = tv, ti
    out.append(best_i.cpu().numpy())
  del dd, qq
  torch.cuda.empty_cache()
  return np.concatenate(out)


def _recompute(data, queries, ids, dist):
  v = data[ids].astype(np.float64)
  q = queries[:, None, :].astype(np.float64)
  return -(q * v).sum(2) if dist == "dot" else ((q - v) ** 2).sum(2)


def _full_size(oracle, tmp_path, name, shape, efs, recall_bars, n_oracle=500, n_recall=1000, n_literal=None,
               min_repeats=1):
  from cuhnsw_amd import capi, datasets
  t0 = time.time()
  data, queries, spec = datasets.make(name)
  o = spec["opt"]
  n, d = data.shape
  assert (n, d) == shape and queries.shape[0] == spec["nq"]
  dist, k = o["dist_type"], spec["topk"]
  mult = o.get("level_mult") or 1.0 / np.log(o["max_m"])
  levels = datasets.random_levels(n, mult)
  print("%s: data %.1f s" % (name, time.time() - t0), flush=True)
  e = capi.Engine()
  path, _ = write_options(tmp_path, dist_type=dist, max_m=o["max_m"], max_m0=o["max_m0"],
                          ef_construction=o["ef_construction"], level_mult=mult, heuristic_coef=0.0)
  assert e.init(path) == 0
  e.set_data(data)
  e.set_random_levels(levels)
  e.build_graph()
  print("%s: built in %.2f s, %d reverse links beyond the inboxes" % (name, e.last_build_seconds,
                                                                     e.last_build_dropped_links), flush=True)
  assert e.max_level == levels.max() and e.enter_point == int(np.argmax(levels))

  p = str(tmp_path / (name + ".idx"))
  e.save_index(p)
  ix = oracle.OracleIndex(dist).load(p)
  assert ix.validate() == 0                            # ids in range, no self loops / duplicates, degree caps, levels
  deg0 = ix.links0()[:, 0]
  assert deg0.min() >= 1 and deg0.max() <= o["max_m0"]
  print("%s: file validated, %.1f s so far" % (name, time.time() - t0), flush=True)

  nq = queries.shape[0]
  gt = _exact_topk(data, queries[:n_recall], k, dist)
  n_literal = nq if n_literal is None else n_literal
  answers = {}
  for ef in efs:
    ids, dv, found = e.search_knn(queries, k, ef)
    repeats = e.last_search_repeats
    assert (found == k).all()
    # ascending by the ordering key: squared L2 itself, or hnswlib's 1 - dot (fp32), under which two dot
    # products one ulp apart can tie (below 0.5 the subtraction rounds) and are then listed by label, so
    # the returned -dot values themselves may step back by that ulp
    order_key = dv if dist == "l2" else np.float32(1.0) + dv
    assert (np.diff(order_key, axis=1) >= 0).all()
    assert (np.diff(dv, axis=1) >= -1e-7).all()
    assert ids.min() >= 0 and ids.max() < n
    srt = np.sort(ids, axis=1)
    assert (np.diff(srt, axis=1) > 0).all()            # distinct ids in every row
    rows = np.arange(0, nq, max(1, nq // 1500))
    ref = _recompute(data, queries[rows], ids[rows], dist)
    np.testing.assert_allclose(dv[rows], ref, rtol=1e-5, atol=1e-5)   # reference's convention, fp32 sums
    rec = float(np.mean([len(set(a) & set(b)) / k for a, b in zip(ids[:n_recall], gt)]))
    print("%s ef %d: recall@%d %.4f, %d queries answered by the literal pass" % (name, ef, k, rec, repeats), flush=True)
    assert rec >= recall_bars[ef], (ef, rec)
    assert repeats >= min_repeats                      # both passes took part
    # the oracle on the same file: bit-exact ids, distances, found counts
    o_ids, o_d, o_f = ix.search(queries[:n_oracle], k, ef)
    tied = ix.meets_ties(queries[:n_oracle], ef)
    bad = (o_ids != ids[:n_oracle]).any(axis=1) | (o_f != found[:n_oracle])
    print("%s ef %d: oracle check on %d queries, %d of them meet equal distances; mismatches among those %d, among the "
          "rest %d" % (name, ef, n_oracle, int(tied.sum()), int((bad & tied).sum()), int((bad & ~tied).sum())), flush=True)
    assert not bad.any()
    assert (o_d == dv[:n_oracle]).all()
    # literal queues only: same answers
    e.set_tunable("fast_path", 0)
    ids0, d0, f0 = e.search_knn(queries[:n_literal], k, ef)
    e.set_tunable("fast_path", 1)
    assert (ids0 == ids[:n_literal]).all() and (d0 == dv[:n_literal]).all() and (f0 == found[:n_literal]).all()
    if min_repeats == 0:
      # a batch of one round is answered by the literal queues by default: force the sorted-set pass as well
      e.set_tunable("fast_path", 2)
      ids1, d1, f1 = e.search_knn(queries, k, ef)
      e.set_tunable("fast_path", 1)
      assert (ids1 == ids).all() and (d1 == dv).all() and (f1 == found).all()
    answers[ef] = (ids, dv)
  del ix
  # a second engine loads the file: same answers
  e2 = capi.Engine()
  assert e2.init(path) == 0
  e2.load_index(p)
  os.remove(p)
  ef = efs[-1]
  ids2, d2, _ = e2.search_knn(queries, k, ef)
  assert (ids2 == answers[ef][0]).all() and (d2 == answers[ef][1]).all()
  print("%s: done in %.1f s" % (name, time.time() - t0), flush=True)


def test_c1_full_size(oracle, tmp_path):
  # 1 000 queries fit one round of wavefronts: the default path answers them with the literal queues alone
  _full_size(oracle, tmp_path, "C1", (100_000, 50), [300], {300: 0.95}, n_oracle=1000, min_repeats=0)


def test_c2_full_size(oracle, tmp_path):
  _full_size(oracle, tmp_path, "C2", (1_183_514, 50), [300], {300: 0.95}, n_recall=2000)


def test_c3_full_size(oracle, tmp_path):
  # integer-valued data: nine queries in ten meet equal distances; every ef of the configuration's sweep
  _full_size(oracle, tmp_path, "C3", (1_000_000, 128), [64, 128, 300], {64: 0.95, 128: 0.95, 300: 0.95}, n_oracle=700)


def test_c4_full_size(oracle, tmp_path):
  # 3 840-byte rows, query staged in LDS; 1 000 queries: one round of wavefronts
  _full_size(oracle, tmp_path, "C4", (1_000_000, 960), [300], {300: 0.95}, min_repeats=0)


def test_c5_full_size(oracle, tmp_path):
  # 10 M points (64-bit row offsets), topk 100, eight keys per lane at ef 512; the literal-only comparison
  # runs on a fifth of the batch (its visited bitmaps are 1.25 MB per wavefront)
  _full_size(oracle, tmp_path, "C5", (10_000_000, 96), [128, 512], {128: 0.95, 512: 0.95}, n_literal=20_000)
