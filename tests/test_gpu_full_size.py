"""The 1.18M-point benchmark configuration at its full size, checked through properties that
do not need the CPU oracle to search a million points in a test: graph invariants of the
saved file (the oracle's validator reads it), found counts, ascending distances, distinct
ids, returned distance == recomputed distance, recall against an exact top-k, the same
answers from both search paths and after a save / load round trip."""
import numpy as np
import pytest

from conftest import write_options

pytestmark = pytest.mark.gpu


def _exact_topk(data, queries, k):
  import torch
  dd = torch.from_numpy(data).cuda()
  qq = torch.from_numpy(queries).cuda()
  best_v = best_i = None
  cols = 1 << 19                       # score blocks of 2^28 elements at most
  for c in range(0, data.shape[0], cols):
    score = -(qq @ dd[c:c + cols].T)
    tv, ti = torch.topk(score, k, dim=1, largest=False)
    ti = ti + c
    if best_v is not None:
      tv, ti = torch.cat([best_v, tv], 1), torch.cat([best_i, ti], 1)
      tv, sel = torch.topk(tv, k, dim=1, largest=False)
      ti = torch.gather(ti, 1, sel)
    best_v, best_i = tv, ti
  return best_i.cpu().numpy()


def test_c2_full_size_properties(oracle, tmp_path):
  from cuhnsw_amd import capi, datasets
  data, queries, spec = datasets.make("C2", nq=10_000)
  o = spec["opt"]
  n, d = data.shape
  assert (n, d) == (1_183_514, 50)
  mult = 1.0 / np.log(o["max_m"])
  levels = datasets.random_levels(n, mult)
  e = capi.Engine()
  path, _ = write_options(tmp_path, dist_type="dot", max_m=o["max_m"], max_m0=o["max_m0"],
                          ef_construction=o["ef_construction"], heuristic_coef=0.0)
  assert e.init(path) == 0
  e.set_data(data)
  e.set_random_levels(levels)
  e.build_graph()
  assert e.max_level == levels.max() and e.enter_point == int(np.argmax(levels))

  k, ef = 10, 300
  ids, dist, found = e.search_knn(queries, k, ef)
  assert e.last_search_repeats > 0                     # both passes took part
  assert (found == k).all()
  assert (np.diff(dist, axis=1) >= 0).all()            # ascending
  assert all(len(set(r)) == k for r in ids)            # distinct ids
  assert ids.min() >= 0 and ids.max() < n
  rows = np.arange(0, 10_000, 7)
  ref = -(queries[rows, None, :] * data[ids[rows]]).sum(2)
  np.testing.assert_allclose(dist[rows], ref, rtol=1e-5, atol=1e-6)   # -dot convention, fp32 sums

  gt = _exact_topk(data, queries[:2000], k)
  rec = np.mean([len(set(a) & set(b)) / k for a, b in zip(ids[:2000], gt)])
  assert rec >= 0.95, rec                              # the benchmark's bar for this configuration

  e.set_tunable("fast_path", 0)                        # literal queues only: same answers
  ids0, dist0, found0 = e.search_knn(queries, k, ef)
  assert (ids0 == ids).all() and (dist0 == dist).all() and (found0 == found).all()
  e.set_tunable("fast_path", 1)

  p = str(tmp_path / "c2.idx")
  e.save_index(p)
  ix = oracle.OracleIndex("dot").load(p)
  assert ix.validate() == 0                            # ids in range, no self loops / duplicates, degree caps, levels
  deg0 = ix.links0()[:, 0]
  assert deg0.min() >= 1 and deg0.max() <= o["max_m0"]
  o_ids, o_d, o_f = ix.search(queries[:500], k, ef)    # the oracle on the same file: bit-exact ids
  assert (o_ids == ids[:500]).all() and (o_d == dist[:500]).all()
  e2 = capi.Engine()
  assert e2.init(path) == 0
  e2.load_index(p)
  ids2, dist2, found2 = e2.search_knn(queries, k, ef)
  assert (ids2 == ids).all() and (dist2 == dist).all()
