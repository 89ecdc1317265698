"""The search entry point that allocates nothing (cuhnsw_search_knn_device_noalloc) through the C ABI
against the allocating entry point (cuhnsw_search_knn_device) on the same index and queries: ids,
distances and found counts bit-equal on two calls in a row, the second with a smaller batch (the
static scratch array keeps the first call's contents), on tie-free and on tie-heavy data (the latter
sends many queries through the literal pass, which is the part that uses the scratch areas), plus the
limits the call must reject."""
import numpy as np
import pytest

from conftest import write_options
from helpers import gauss_mixture, integer_vectors

pytestmark = pytest.mark.gpu


def _levels(n, mult, seed):
  rng = np.random.default_rng(seed)
  return (-np.log(np.maximum(rng.uniform(size=n), 1e-10)) * mult).astype(np.int32)


def _search(e, q, k, ef, no_alloc):
  import torch
  nq = q.shape[0]
  qq = torch.from_numpy(np.ascontiguousarray(q, dtype=np.float32)).cuda()
  nns = torch.full((nq, k), -7, dtype=torch.int32, device="cuda")
  dist = torch.full((nq, k), -7.0, dtype=torch.float32, device="cuda")
  found = torch.full((nq,), -7, dtype=torch.int32, device="cuda")
  torch.cuda.synchronize()
  fn = e.search_knn_device_noalloc if no_alloc else e.search_knn_device
  args = (qq.data_ptr(), nq, k, ef, nns.data_ptr(), dist.data_ptr(), found.data_ptr())
  if no_alloc:
    # (the first launch of a kernel shape may make the HIP runtime size its own spill area for the
    # launch: what is checked is that a repeated call leaves the device's free memory where it was)
    fn(*args)
    free_before = torch.cuda.mem_get_info()[0]
    nns.fill_(-7); dist.fill_(-7.0); found.fill_(-7)
    torch.cuda.synchronize()
    fn(*args)
    assert torch.cuda.mem_get_info()[0] == free_before
  else:
    fn(*args, None)
  return nns.cpu().numpy(), dist.cpu().numpy(), found.cpu().numpy(), e.last_search_repeats


@pytest.mark.parametrize("kind", ["gauss", "int"])
def test_no_alloc_search_equals_the_allocating_search(tmp_path, kind):
  from cuhnsw_amd import capi
  n, d = 20000, 24
  if kind == "gauss":
    x, q, dist = gauss_mixture(n, d, centres=100, seed=71), gauss_mixture(3000, d, centres=100, seed=72), "dot"
  else:
    x, q, dist = integer_vectors(n, d, seed=73, hi=12), integer_vectors(3000, d, seed=74, hi=12), "l2"
  e = capi.Engine()
  path, _ = write_options(tmp_path, dist_type=dist, max_m=8, max_m0=16, ef_construction=60, heuristic_coef=0.0)
  assert e.init(path) == 0
  e.set_data(x)
  e.set_random_levels(_levels(n, 1 / np.log(8), 75))
  e.build_graph()
  e.set_tunable("fast_path", 2)   # the allocating call takes the same two passes
  print("no_alloc", kind, "first call: 3000 queries", flush=True)
  for nq, k, ef in ((3000, 10, 100), (700, 10, 100), (700, 100, 300), (64, 5, 512), (1, 1, 1)):
    want = _search(e, q[:nq], k, ef, False)
    got = _search(e, q[:nq], k, ef, True)
    assert (got[2] == want[2]).all()
    assert (got[0] == want[0]).all(), (kind, nq, k, ef)
    assert (got[1] == want[1]).all()
    if kind == "int" and nq >= 700:
      assert got[3] > 20                          # queries went through the literal pass: the scratch areas were in use
  # limits
  for nq, k, ef, what in ((200000, 10, 100, "at most"), (10, 10, 600, "must not exceed"), (10, 600, 10, "must not exceed")):
    with pytest.raises(RuntimeError, match=what):
      e.search_knn_device_noalloc(0, nq, k, ef, 0, 0, 0)
  # the allocating entry point is untouched by all this
  want = _search(e, q[:500], 10, 100, False)
  again = _search(e, q[:500], 10, 100, False)
  assert (want[0] == again[0]).all()
