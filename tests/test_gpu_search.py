"""GPU search parity: the HIP search (through the C ABI) against the CPU oracle on the
same index file and queries — ids bit-exact, distances within 1e-5 relative (in fact
bit-equal, both sides use the same canonical fp32 order), found counts and the
per-query distance-evaluation / hop counters identical."""
import numpy as np
import pytest

from conftest import write_options
from helpers import gauss_mixture, integer_vectors, ring_graph

pytestmark = pytest.mark.gpu


def _engine(tmp_path, **opt):
  from cuhnsw_amd import capi
  e = capi.Engine()
  path, _ = write_options(tmp_path, **opt)
  assert e.init(path) == 0
  return e


def _levels(n, mult, seed):
  rng = np.random.default_rng(seed)
  return (-np.log(np.maximum(rng.uniform(size=n), 1e-10)) * mult).astype(np.int32)


def _device_search(e, q, k, ef):
  import torch
  nq = q.shape[0]
  qq = torch.from_numpy(np.ascontiguousarray(q, dtype=np.float32)).cuda()
  nns = torch.empty((nq, k), dtype=torch.int32, device="cuda")
  dist = torch.empty((nq, k), dtype=torch.float32, device="cuda")
  found = torch.empty(nq, dtype=torch.int32, device="cuda")
  stats = torch.zeros((nq, 4), dtype=torch.int32, device="cuda")
  torch.cuda.synchronize()
  e.search_knn_device(qq.data_ptr(), nq, k, ef, nns.data_ptr(), dist.data_ptr(), found.data_ptr(), stats.data_ptr())
  return nns.cpu().numpy(), dist.cpu().numpy(), found.cpu().numpy(), stats.cpu().numpy()


def _check_parity(oracle, ix, e, q, k, ef, counters=True, dup_bound=3.0):
  """Both search paths against the oracle: the default one (sorted set in registers with an
  LDS-only visited filter; queries that meet equal keys are repeated with literal queues)
  and the literal queues alone (fast_path = 0)."""
  o_ids, o_d, o_f, o_cnt = ix.search(q, k, ef, counters=True)
  # 2 = sorted-set pass whatever the batch size; 1 = default (a batch this small goes to the literal
  # pass on the sorted set with ids and the LDS filter); 0 = literal queues with the exact bitmap
  for fast in (2, 1, 0):
    e.set_tunable("fast_path", fast)
    e.set_tunable("lean_literal", 2 if fast else 1)   # small test indexes would otherwise choose the bitmap
    g_ids, g_d, g_f = e.search_knn(q, k, ef)
    assert (g_f == o_f).all()
    for r in range(q.shape[0]):
      f = o_f[r]
      assert (g_ids[r, :f] == o_ids[r, :f]).all(), "query %d fast_path %d" % (r, fast)
      np.testing.assert_allclose(g_d[r, :f], o_d[r, :f], rtol=1e-5, atol=0)
      assert (g_d[r, :f] == o_d[r, :f]).all()
    if counters:
      d_ids, d_d, d_f, stats = _device_search(e, q, k, ef)
      assert (d_ids == g_ids).all() and (d_f == g_f).all()
      # expansions and upper-level work are the oracle's in both paths; the lossy filter of
      # the default path may evaluate a forgotten neighbour again, the literal path never
      assert (stats[:, 1:] == o_cnt[:, 1:4]).all()
      if fast:
        assert (stats[:, 0] >= o_cnt[:, 0]).all()
        if dup_bound:
          assert stats[:, 0].sum() <= dup_bound * o_cnt[:, 0].sum() + 64
      else:
        assert (stats[:, 0] == o_cnt[:, 0]).all()
        assert e.last_search_repeats == 0
  e.set_tunable("fast_path", 1)
  e.set_tunable("lean_literal", 1)


CASES = [
    # name, n, d, dist, max_m, max_m0, data kind
    ("dot50", 6000, 50, "dot", 12, 24, "gauss"),        # one float4 per lane
    ("dot96", 4000, 96, "dot", 16, 32, "gauss"),        # two
    ("l2_128_int", 5000, 128, "l2", 16, 32, "int"),     # integer data: exact sums, many ties
    ("l2_200", 3000, 200, "l2", 8, 16, "gauss_raw"),    # four
    ("l2_960", 1500, 960, "l2", 16, 32, "gauss_raw"),   # query staged in LDS
    ("dot7", 3000, 7, "dot", 5, 10, "gauss"),           # odd small dimension, odd degrees
    ("l2_tiny_int", 4000, 6, "l2", 6, 12, "tiny_int"),  # almost everything ties
]


def _data(kind, n, d, seed):
  if kind == "gauss":
    return gauss_mixture(n, d, seed=seed)
  if kind == "gauss_raw":
    return gauss_mixture(n, d, seed=seed, normalise=False)
  if kind == "int":
    return integer_vectors(n, d, seed=seed, hi=219)
  return integer_vectors(n, d, seed=seed, hi=4)


@pytest.mark.parametrize("name,n,d,dist,max_m,max_m0,kind", CASES, ids=[c[0] for c in CASES])
def test_search_parity_on_oracle_built_index(oracle, tmp_path, name, n, d, dist, max_m, max_m0, kind):
  x = _data(kind, n, d, 1)
  q = _data(kind, 200, d, 2)
  mult = 1.0 / np.log(max_m)
  ix = oracle.OracleIndex(dist).build(x, _levels(n, mult, 3), max_m, max_m0, 60, mult)
  p = str(tmp_path / "i.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type=dist, max_m=max_m, max_m0=max_m0)
  e.load_index(p)
  assert (e.num_data, e.num_dims, e.max_level, e.enter_point) == (n, d, ix.maxlevel, ix.enterpoint)
  # ef <= 128: result keys in 2 registers per lane; < 320: 5; <= 512: 8; < 1024: 16; beyond: literal LDS heap
  for k, ef in ((10, 300), (1, 1), (10, 10), (100, 64), (100, 120), (7, 33), (128, 128), (10, 129), (10, 400),
                (100, 512), (10, 513),
                (50, 1023), (10, 1100)):
    _check_parity(oracle, ix, e, q, k, ef)


@pytest.mark.parametrize("kind,d,dist,max_m,half", [
    ("gauss", 50, "dot", 8, False), ("int", 24, "l2", 8, False),
    ("gauss_raw", 100, "l2", 20, False),   # two register chunks per lane; upper-level rows longer than 16 ids
    ("int", 128, "l2", 16, True),          # fp16 rows (integers below 2048 are exact in fp16), full upper-level rows
    ("gauss", 160, "dot", 8, False),       # rows too long for registers: the descents one query per wavefront
], ids=["dot50", "l2_int_ties", "l2_100_m20", "l2_128_fp16", "dot160"])
def test_longest_queries_first_changes_nothing_but_the_order(oracle, tmp_path, kind, d, dist, max_m, half):
  """A batch of several rounds of wavefronts does its upper-level descents first (four queries per wavefront
  where the rows fit registers) and takes its queries by descending entry distance.  Answers, found counts and
  every counter (the descent's evaluations and sweeps come from the separate kernel) are those of the caller's
  order, and the oracle's."""
  n, nq, k = 8000, 12000, 10
  x = _data(kind, n, d, 11)
  q = _data(kind, nq, d, 12)
  ix = oracle.OracleIndex(dist).build(x, _levels(n, 0.4, 13), max_m, 2 * max_m, 60, 0.4)
  p = str(tmp_path / "i.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type=dist, max_m=max_m, max_m0=2 * max_m)
  if half:
    e.set_tunable("fp16_storage", 1)
  e.load_index(p)
  for ef in (150, 64):
    got = {}
    for order in (2, 0):          # 2: in order whenever the batch is more than one round of wavefronts
      e.set_tunable("query_order", order)
      got[order] = _device_search(e, q, k, ef)
    for a, b in zip(got[2], got[0]):
      assert (a == b).all()
    e.set_tunable("concurrent_literal", 0)   # the literal pass after the first one instead of beside it
    e.set_tunable("query_order", 2)
    for a, b in zip(_device_search(e, q, k, ef), got[0]):
      assert (a == b).all()
    e.set_tunable("concurrent_literal", 1)
    o_ids, o_d, o_f, o_cnt = ix.search(q[:1500], k, ef, counters=True)
    g_ids, g_d, g_f, stats = got[2]
    assert (g_f[:1500] == o_f).all() and (g_ids[:1500] == o_ids).all() and (g_d[:1500] == o_d).all()
    assert (stats[:1500, 1:] == o_cnt[:, 1:4]).all()
  e.set_tunable("query_order", 1)


def test_tight_rows_layout_and_gather_probe(oracle, tmp_path):
  """Vector rows padded to 16-byte chunks only (tunable tight_rows; rows then start off the 128-byte lines):
  same answers as the oracle, for a dimension with a partial last chunk too.  And the memory-pattern probe
  runs on the resident vectors and reports a sane rate."""
  for d, dist in ((50, "dot"), (7, "l2"), (100, "l2")):
    n = 3000
    x = gauss_mixture(n, d, seed=41, normalise=(dist == "dot"))
    q = gauss_mixture(100, d, seed=42, normalise=(dist == "dot"))
    mult = 1 / np.log(8)
    ix = oracle.OracleIndex(dist).build(x, _levels(n, mult, 43), 8, 16, 60, mult)
    p = str(tmp_path / "tight.idx")
    ix.save(p)
    e = _engine(tmp_path, dist_type=dist, max_m=8, max_m0=16)
    e.set_tunable("tight_rows", 1)
    e.load_index(p)
    with pytest.raises(RuntimeError, match="before set_data"):
      e.set_tunable("tight_rows", 0)
    _check_parity(oracle, ix, e, q, 10, 100)
    _check_parity(oracle, ix, e, q, 10, 300)
    rows, ms = e.gather_probe(8, 4, True)
    assert rows > 0 and rows % (8 * 4 * 2048) == 0 and 0.0 < ms < 1000.0


def test_labels_from_file_are_returned(oracle, tmp_path):
  n, d = 3000, 20
  x = gauss_mixture(n, d, seed=4)
  q = gauss_mixture(64, d, seed=5)
  levels = _levels(n, 0.4, 6)
  base = oracle.OracleIndex("dot").build(x, levels, 8, 16, 40, 0.4)
  labels = np.random.default_rng(0).permutation(n).astype(np.uint64) * 3 + 5
  l0 = base.links0()
  up = np.concatenate([np.concatenate([[len(base.links(i, l))], np.pad(base.links(i, l), (0, 8 - len(base.links(i, l))))])
                       for i in range(n) for l in range(1, levels[i] + 1)]).astype(np.uint32)
  ix = oracle.OracleIndex("dot").from_arrays(x, levels, l0, up, 8, 16, base.maxlevel, base.enterpoint, labels=labels)
  p = str(tmp_path / "lab.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="dot", max_m=8, max_m0=16)
  e.load_index(p)
  _check_parity(oracle, ix, e, q, 10, 50, counters=False)
  g_ids, _, _ = e.search_knn(q, 10, 50)
  assert set(np.unique(g_ids)) <= set(labels.astype(np.int64))


def test_single_query_1d_and_tiny_indexes(oracle, tmp_path):
  # N = 1
  one = oracle.OracleIndex("l2").from_arrays(np.array([[1.0, 2.0]], np.float32), np.zeros(1, np.int32),
                                             np.zeros((1, 5), np.uint32), np.zeros(0, np.uint32), 2, 4, 0, 0)
  p = str(tmp_path / "one.idx")
  one.save(p)
  e = _engine(tmp_path, dist_type="l2", max_m=2, max_m0=4)
  e.load_index(p)
  ids, d, f = e.search_knn(np.array([0.0, 0.0], np.float32), 3, 10)  # 1-d query = one query
  assert ids.shape == (1, 3) and f[0] == 1 and ids[0, 0] == 0 and d[0, 0] == 5.0
  assert ids[0, 1] == -1 and np.isinf(d[0, 1])
  # two components: found < topk
  pts = np.arange(5, dtype=np.float32)[:, None]
  links0 = np.zeros((5, 3), np.uint32)
  links0[0] = [2, 1, 2]; links0[1] = [2, 0, 2]; links0[2] = [2, 0, 1]
  links0[3] = [1, 4, 0]; links0[4] = [1, 3, 0]
  ix = oracle.OracleIndex("l2").from_arrays(pts, np.zeros(5, np.int32), links0, np.zeros(0, np.uint32), 2, 2, 0, 0)
  p = str(tmp_path / "comp.idx")
  ix.save(p)
  e.load_index(p)
  ids, d, f = e.search_knn(np.array([[3.6]], np.float32), 5, 10)
  assert f[0] == 3 and list(ids[0, :3]) == [2, 1, 0]
  _check_parity(oracle, ix, e, np.array([[3.6], [0.2], [-5.0]], np.float32), 5, 10)


def test_ef_ge_n_is_exact_brute_force(oracle, tmp_path):
  n, d, k = 500, 12, 10
  x = gauss_mixture(n, d, seed=8)
  q = gauss_mixture(40, d, seed=9)
  ix = oracle.OracleIndex("dot").from_arrays(x, np.zeros(n, np.int32), ring_graph(n, 8), np.zeros(0, np.uint32),
                                             4, 8, 0, 0)
  p = str(tmp_path / "ring.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="dot", max_m=4, max_m0=8)
  e.load_index(p)
  e.set_tunable("hnswlib_dist", 1)
  ids, dists, found = e.search_knn(q, k, n)
  bf_ids, bf_d = oracle.bruteforce(x, q, k, "dot")
  assert (found == k).all() and (ids == bf_ids).all() and (dists == bf_d).all()


def test_candidate_queue_spills_to_global_memory(oracle, tmp_path):
  """A tiny LDS share for the candidate queue forces the global-memory overflow path;
  results must not change."""
  n, d = 8000, 32
  x = gauss_mixture(n, d, seed=10)
  q = gauss_mixture(100, d, seed=11)
  mult = 1 / np.log(8)
  ix = oracle.OracleIndex("dot").build(x, _levels(n, mult, 12), 8, 16, 60, mult)
  p = str(tmp_path / "s.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="dot", max_m=8, max_m0=16)
  e.load_index(p)
  e.set_tunable("cand_lds", 64)
  _check_parity(oracle, ix, e, q, 10, 400)
  e.set_tunable("search_slots", 3)  # many queries per resident wavefront: visited sets must be clean between queries
  _check_parity(oracle, ix, e, q, 10, 100)
  for entries in (-1, 256, 8192):   # without / tiny / large LDS visited cache: same answers
    e.set_tunable("visited_cache", entries)
    _check_parity(oracle, ix, e, q, 10, 100)
  e.set_tunable("concurrent_literal", 0)   # literal pass after the sorted-set pass instead of beside it
  _check_parity(oracle, ix, e, q, 10, 100)
  e.set_tunable("concurrent_literal", 1)
  for entries in (256, 16384):      # tiny / large visited filter of the sorted-set search
    e.set_tunable("filter_entries", entries)
    _check_parity(oracle, ix, e, q, 10, 100, dup_bound=None)


def test_literal_pass_schedules_on_tie_heavy_data(oracle, tmp_path):
  """Integer data: most queries meet equal distances in the sorted-set pass and are answered by
  the literal pass — beside the first pass (default), after it, and after it because the
  waiting wavefronts were told from the host to give up at once (a bound of zero polls: every
  kernel still ends normally)."""
  n, d = 5000, 16
  x = integer_vectors(n, d, seed=21, hi=30)
  q = integer_vectors(150, d, seed=22, hi=30)
  mult = 1 / np.log(8)
  ix = oracle.OracleIndex("l2").build(x, _levels(n, mult, 23), 8, 16, 60, mult)
  p = str(tmp_path / "t.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="l2", max_m=8, max_m0=16)
  e.load_index(p)
  e.set_tunable("fast_path", 2)
  e.search_knn(q, 10, 100)
  assert e.last_search_repeats > 50
  for tunable, value in (("concurrent_literal", 1), ("concurrent_literal", 0), ("literal_spin_limit", 0),
                         ("literal_per_cu", 1)):
    e.set_tunable("concurrent_literal", 1)
    e.set_tunable("literal_spin_limit", -1)
    e.set_tunable(tunable, value)
    _check_parity(oracle, ix, e, q, 10, 100)
    _check_parity(oracle, ix, e, q, 100, 100)


def test_fallback_schedule_is_temporary_and_trails_are_optional(oracle, tmp_path):
  """A literal wavefront whose wait runs out (forced from the host: a bound of zero polls) makes the engine answer
  the batch after its first pass and run the next 8 searches one pass after the other; then the side-by-side
  schedule is back, the caller's concurrent_literal setting untouched throughout.  A new index forgets all of it.
  And trail buffers that cannot be allocated (a trail_cap of 2^30 entries) switch the trails off, not the search."""
  n, d = 5000, 16
  x = integer_vectors(n, d, seed=21, hi=30)
  q = integer_vectors(150, d, seed=22, hi=30)
  mult = 1 / np.log(8)
  ix = oracle.OracleIndex("l2").build(x, _levels(n, mult, 23), 8, 16, 60, mult)
  p = str(tmp_path / "t.idx")
  ix.save(p)
  o_ids, o_d, o_f = ix.search(q, 10, 100)
  e = _engine(tmp_path, dist_type="l2", max_m=8, max_m0=16)
  e.load_index(p)
  assert e.trails_available and e.literal_fallbacks == 0
  e.set_tunable("fast_path", 2)
  e.set_tunable("lean_literal", 2)

  def search():
    g_ids, g_d, g_f = e.search_knn(q, 10, 100)
    assert (g_f == o_f).all() and (g_ids == o_ids).all() and (g_d == o_d).all()
    assert e.last_search_repeats > 0

  search()
  assert e.last_search_side_by_side and e.last_search_trails > 0
  e.set_tunable("literal_spin_limit", 0)
  search()                                         # beside the first pass, every waiting wavefront gives up at once
  assert e.last_search_side_by_side and e.literal_fallbacks == 1
  e.set_tunable("literal_spin_limit", -1)
  for _ in range(8):
    search()
    assert not e.last_search_side_by_side
  search()
  assert e.last_search_side_by_side and e.literal_fallbacks == 1
  e.set_tunable("literal_spin_limit", 0)
  search()
  assert e.literal_fallbacks == 2
  e.set_tunable("literal_spin_limit", -1)
  e.load_index(p)                                  # another index: nothing of that is carried over
  assert e.literal_fallbacks == 0
  search()
  assert e.last_search_side_by_side
  # trails that cannot be allocated
  e.set_tunable("trail_cap", 1 << 30)
  search()
  assert not e.trails_available and e.last_search_trails == 0
  e.set_tunable("trail_cap", 2048)
  search()
  assert e.trails_available and e.last_search_trails > 0


@pytest.mark.parametrize("d,hi", [(16, 30), (12, 60), (80, 6)], ids=["many_ties", "fewer_ties", "two_chunks_per_lane"])
def test_handed_over_queries_start_from_the_first_pass_trail(oracle, tmp_path, d, hi):
  """The first pass leaves the entries it accepted, hop by hop, and the literal pass (on the tag filter) replays
  its queue operations from them instead of searching a handed-over query from the entry point: same answers and
  hop counters as the oracle — with a trail for every handed-over query, for a few only (no spare buffers after
  three), with trails that overflow (16 entries), and with none."""
  n = 5000
  x = integer_vectors(n, d, seed=61, hi=hi)
  q = integer_vectors(250, d, seed=62, hi=hi)   # (under 256 queries: the engine keeps trying the first pass however many tie)
  mult = 1 / np.log(8)
  ix = oracle.OracleIndex("l2").build(x, _levels(n, mult, 63), 8, 16, 60, mult)
  p = str(tmp_path / "t.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="l2", max_m=8, max_m0=16)
  e.load_index(p)
  e.set_tunable("fast_path", 2)
  e.set_tunable("lean_literal", 2)
  for k, ef in ((10, 100), (100, 100), (10, 300)):
    o_ids, o_d, o_f, o_cnt = ix.search(q, k, ef, counters=True)
    # (eight wavefronts: each answers some thirty queries and needs a spare buffer after every hand-over; trails = 2:
    # also in a batch of many rounds of wavefronts)
    for name, settings in (("all", {}), ("eight", {"search_slots": 8, "trails": 2}), ("three", {"search_slots": 8, "trails": 2, "trail_spares": 3}),
                           ("short", {"trail_cap": 16}), ("after", {"concurrent_literal": 0}), ("none", {"trails": 0})):
      for key, value in {"trails": 1, "trail_cap": 2048, "trail_spares": 1024, "concurrent_literal": 1, "search_slots": 0,
                         **settings}.items():
        e.set_tunable(key, value)
      g_ids, g_d, g_f, stats = _device_search(e, q, k, ef)
      assert (g_f == o_f).all()
      for r in range(q.shape[0]):
        f = o_f[r]
        assert (g_ids[r, :f] == o_ids[r, :f]).all() and (g_d[r, :f] == o_d[r, :f]).all(), (name, k, ef, r)
      assert (stats[:, 1:] == o_cnt[:, 1:4]).all()
      handed, trails = e.last_search_repeats, e.last_search_trails
      assert handed > 0, (name, k, ef, handed, trails)
      if name in ("all", "after", "eight"):
        assert trails == handed
      elif name == "three":
        assert trails <= 8 + 3 and (trails < handed or handed <= 11)   # the wavefronts' own buffers and the spares
      elif name == "short":
        assert trails <= handed
      else:
        assert trails == 0
  for key, value in (("trails", 1), ("trail_cap", 2048), ("trail_spares", 1024), ("concurrent_literal", 1),
                     ("search_slots", 0)):
    e.set_tunable(key, value)


def test_overflowing_scratch_areas_are_retried(oracle, tmp_path):
  """Accept log and queue overflow area start far too small: the engine must notice, grow
  them and repeat the search with unchanged answers."""
  n, d = 6000, 24
  x = gauss_mixture(n, d, seed=13)
  q = gauss_mixture(80, d, seed=14)
  mult = 1 / np.log(8)
  ix = oracle.OracleIndex("dot").build(x, _levels(n, mult, 15), 8, 16, 60, mult)
  p = str(tmp_path / "r.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="dot", max_m=8, max_m0=16)
  e.load_index(p)
  e.set_tunable("spill_cap", 8)
  _check_parity(oracle, ix, e, q, 10, 300)
  _check_parity(oracle, ix, e, q, 10, 1200)   # literal-heap path


def test_search_on_a_file_with_spare_capacity_and_flag_bits(oracle, tmp_path):
  """An index file as hnswlib writes it from an index that was not filled up (max_elements >
  cur_element_count: extra level-0 records of arbitrary content) and with unknown flag bits set above
  the 16-bit link counts: loaded on the GPU it must answer exactly as the oracle does on the compact
  file; so must the same file with elements marked deleted (hnswlib markDelete), against the oracle that
  read the same marks."""
  import struct
  n, d = 4000, 20
  x = gauss_mixture(n, d, seed=31)
  q = gauss_mixture(100, d, seed=32)
  levels = _levels(n, 0.4, 33)
  ix = oracle.OracleIndex("dot").build(x, levels, 8, 16, 40, 0.4)
  p = str(tmp_path / "compact.idx")
  ix.save(p)
  raw = bytearray(open(p, "rb").read())
  rec = 16 * 4 + 4 + d * 4 + 8
  spare = 37
  struct.pack_into("<Q", raw, 8, n + spare)                        # max_elements
  for i in range(0, n, 3):                                         # flag bits above the count, never the delete mark
    (word,) = struct.unpack_from("<I", raw, 96 + i * rec)
    struct.pack_into("<I", raw, 96 + i * rec, word | (1 << 17) | (1 << 30))
  junk = np.random.default_rng(5).integers(0, 256, spare * rec, dtype=np.uint8).tobytes()
  body_end = 96 + n * rec
  hnsw_like = bytes(raw[:body_end]) + junk + bytes(raw[body_end:])
  p2 = str(tmp_path / "spare.idx")
  open(p2, "wb").write(hnsw_like)
  e = _engine(tmp_path, dist_type="dot", max_m=8, max_m0=16)
  e.load_index(p2)
  assert e.num_data == n
  _check_parity(oracle, ix, e, q, 10, 80)
  marked = bytearray(hnsw_like)
  (word,) = struct.unpack_from("<I", marked, 96 + 5 * rec)
  struct.pack_into("<I", marked, 96 + 5 * rec, word | (1 << 16))   # hnswlib's markDelete on element 5
  open(p2, "wb").write(bytes(marked))
  e.load_index(p2)
  assert e.num_deleted == 1
  ix.mark_deleted([5])
  _check_deleted_parity(ix, e, q, 10, 80)


def _check_deleted_parity(ix, e, q, k, ef):
  """Engine against oracle on an index with deleted elements: ids, distances, found counts and every
  counter (the search on the literal queues evaluates exactly what hnswlib's loop evaluates)."""
  o_ids, o_d, o_f, o_cnt = ix.search(q, k, ef, counters=True)
  g_ids, g_d, g_f, stats = _device_search(e, q, k, ef)
  assert (g_f == o_f).all()
  for r in range(q.shape[0]):
    f = o_f[r]
    assert (g_ids[r, :f] == o_ids[r, :f]).all(), "query %d" % r
    assert (g_d[r, :f] == o_d[r, :f]).all()
    assert (g_ids[r, f:] == -1).all()
  assert (stats == o_cnt[:, :4]).all()
  h_ids, h_d, h_f = e.search_knn(q, k, ef)
  assert (h_ids == g_ids).all() and (h_f == g_f).all()


@pytest.mark.parametrize("dist_type", ["dot", "l2"])
def test_search_on_an_index_with_deleted_elements(oracle, tmp_path, dist_type):
  """hnswlib's delete marks in a loaded file: walked through, never returned.  Shares from one element to
  nearly all, the entry point among them, more results asked for than elements are left, the marks written
  back by save_index; calls that cannot honour the marks fail with a message."""
  n, d = 5000, 24
  x = gauss_mixture(n, d, seed=41, normalise=(dist_type == "dot"))
  q = gauss_mixture(200, d, seed=42, normalise=(dist_type == "dot"))
  levels = _levels(n, 0.4, 43)
  ix = oracle.OracleIndex(dist_type).build(x, levels, 8, 16, 60, 0.4)
  rng = np.random.default_rng(44)
  e = _engine(tmp_path, dist_type=dist_type, max_m=8, max_m0=16)
  for share in (0.0002, 0.05, 0.5, 0.97, 0.999):
    ix.mark_deleted(np.arange(n), mark=False)
    dead = rng.choice(n, max(1, int(n * share)), replace=False)
    dead = np.union1d(dead, [ix.enterpoint]) if share >= 0.05 else dead
    ix.mark_deleted(dead)
    p = str(tmp_path / ("m%g.idx" % share))
    ix.save(p)
    e.load_index(p)
    assert e.num_deleted == dead.size
    for k, ef in ((10, 64), (1, 1), (10, 300), (40, 20), (10, 1100)):
      _check_deleted_parity(ix, e, q, k, ef)
    ids, _, found = e.search_knn(q, 10, 64)
    assert not np.isin(ids[ids >= 0], dead).any()
    if share == 0.999:
      # five elements are left: a search finds those of them that can be reached from the entry point (the
      # parity check above says: the same ones as the oracle's)
      assert (found <= n - dead.size).all() and (found >= 1).all()
    p2 = str(tmp_path / "back.idx")
    e.save_index(p2)
    assert open(p2, "rb").read() == open(p, "rb").read()
  with pytest.raises(RuntimeError, match="deleted elements"):
    e.search_knn_device_noalloc(0, 8, 10, 64, 0, 0, 0)   # (fails before any pointer is used)
  # everything marked: nothing is found
  ix.mark_deleted(np.arange(n))
  p = str(tmp_path / "all.idx")
  ix.save(p)
  e.load_index(p)
  ids, dist, found = e.search_knn(q[:50], 5, 40)
  assert (found == 0).all() and (ids == -1).all()
  # a graph built anew holds every element again
  e.set_random_levels(levels)
  e.build_graph()
  assert e.num_deleted == 0
  _, _, found = e.search_knn(q[:50], 5, 40)
  assert (found == 5).all()


def test_deleted_elements_and_equal_keys(oracle, tmp_path):
  """Integer data: nearly every search meets equal keys, the order the literal heaps give them is the
  answer; a third of the elements deleted."""
  n, d = 6000, 8
  x = integer_vectors(n, d, seed=51, hi=6)
  q = integer_vectors(300, d, seed=52, hi=6)
  levels = _levels(n, 0.4, 53)
  ix = oracle.OracleIndex("l2").build(x, levels, 8, 16, 60, 0.4)
  ix.mark_deleted(np.arange(1, n, 3))
  p = str(tmp_path / "ties.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="l2", max_m=8, max_m0=16)
  e.load_index(p)
  for k, ef in ((10, 100), (1, 30), (50, 50), (10, 400)):
    _check_deleted_parity(ix, e, q, k, ef)


def test_reverse_cand_refuses_an_index_with_deleted_elements(oracle, tmp_path):
  n, d = 1000, 8
  x = gauss_mixture(n, d, seed=61)
  ix = oracle.OracleIndex("dot").build(x, _levels(n, 0.4, 62), 8, 16, 40, 0.4)
  ix.mark_deleted([3])
  p = str(tmp_path / "r.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type="dot", max_m=8, max_m0=16, reverse_cand=True)
  e.load_index(p)
  with pytest.raises(RuntimeError, match="reverse_cand is not defined"):
    e.search_knn(x[:4], 3, 20)


def test_tiny_batches_on_long_rows(oracle, tmp_path):
  """Vectors of more than 256 dimensions (the query in LDS): every batch takes the first pass, a single query
  too, and a query handed over out of a batch of one is answered by the literal pass beside it.  Integer data:
  nearly every query is handed over.  Dimensions that end inside a fetch round, on one, and just past one."""
  for case, d in enumerate((300, 512, 1030)):
    n = 2500
    x = integer_vectors(n, d, seed=70 + case, hi=3)
    q = integer_vectors(12, d, seed=80 + case, hi=3)
    ix = oracle.OracleIndex("l2").build(x, _levels(n, 0.4, 90 + case), 8, 16, 60, 0.4)
    p = str(tmp_path / ("long%d.idx" % d))
    ix.save(p)
    (tmp_path / ("e%d" % d)).mkdir()
    e = _engine(tmp_path / ("e%d" % d), dist_type="l2", max_m=8, max_m0=16)
    e.load_index(p)
    handed = 0
    for nq in (1, 2, 12):
      for k, ef in ((10, 100), (1, 1), (5, 300)):
        for start in (0, 3):
          qq = q[start:start + nq]
          o_ids, o_d, o_f, o_cnt = ix.search(qq, k, ef, counters=True)
          g_ids, g_d, g_f, stats = _device_search(e, qq, k, ef)
          assert (g_f == o_f).all()
          for r in range(qq.shape[0]):
            assert (g_ids[r, :o_f[r]] == o_ids[r, :o_f[r]]).all() and (g_d[r, :o_f[r]] == o_d[r, :o_f[r]]).all()
          assert (stats[:, 1:] == o_cnt[:, 1:4]).all()
          handed += e.last_search_repeats
    assert handed > 0


def test_errors(tmp_path):
  e = _engine(tmp_path)
  e.set_data(np.zeros((8, 4), np.float32))
  with pytest.raises(RuntimeError, match="no index"):
    e.search_knn(np.zeros((1, 4), np.float32), 1, 1)
  with pytest.raises(RuntimeError, match="set_random_levels first"):
    e.build_graph()


@pytest.mark.parametrize("name,n,d,dist,max_m,max_m0,kind", [CASES[0], CASES[2], CASES[4], CASES[6]],
                         ids=[CASES[i][0] for i in (0, 2, 4, 6)])
def test_reverse_cand_search_parity(oracle, tmp_path, name, n, d, dist, max_m, max_m0, kind):
  """The reference's reverse_cand option (the farthest waiting candidate is expanded first)
  against the oracle's statement of it: ids, distances, found counts and expansion counters
  identical, ties included (equal keys keep their order of arrival on both sides), for result sets in
  registers and beyond."""
  x = _data(kind, n, d, 1)
  q = _data(kind, 120, d, 2)
  mult = 1.0 / np.log(max_m)
  ix = oracle.OracleIndex(dist).build(x, _levels(n, mult, 3), max_m, max_m0, 60, mult)
  p = str(tmp_path / "i.idx")
  ix.save(p)
  e = _engine(tmp_path, dist_type=dist, max_m=max_m, max_m0=max_m0, reverse_cand=True)
  e.load_index(p)
  # (from 1024 on the register set is too small: the literal pass keeps a sorted list in LDS)
  for k, ef in ((10, 300), (1, 1), (10, 10), (100, 120), (10, 400), (50, 1023), (10, 1024), (300, 1500), (5, 2500)):
    o_ids, o_d, o_f, o_cnt = ix.search(q, k, ef, counters=True, reverse_cand=True)
    g_ids, g_d, g_f = e.search_knn(q, k, ef)
    assert (g_f == o_f).all()
    for r in range(q.shape[0]):
      f = o_f[r]
      assert (g_ids[r, :f] == o_ids[r, :f]).all(), "query %d k %d ef %d" % (r, k, ef)
      assert (g_d[r, :f] == o_d[r, :f]).all()
    d_ids, d_d, d_f, stats = _device_search(e, q, k, ef)
    assert (d_ids == g_ids).all() and (stats[:, 1:] == o_cnt[:, 1:4]).all() and (stats[:, 0] >= o_cnt[:, 0]).all()
    assert e.last_search_repeats == 0


@pytest.mark.parametrize("seed,d,hi", [(101, 12, 12), (102, 8, 40), (103, 24, 6), (104, 5, 200)])
def test_followed_up_ties_match_the_oracle_on_quantised_data(oracle, tmp_path, seed, d, hi):
  """Quantised data: equal distances everywhere, but most of them harmless.  The sorted-set
  pass follows groups of equal keys up instead of giving every such query to the literal
  queues; ids, distances and expansion counts must still be the oracle's for every query, at
  many (k, ef) shapes, with and without labels that differ from the ids."""
  n = 8000
  x = integer_vectors(n, d, seed=seed, hi=hi)
  q = integer_vectors(700, d, seed=seed + 50, hi=hi)
  mult = 1 / np.log(8)
  levels = _levels(n, mult, seed + 7)
  base = oracle.OracleIndex("l2").build(x, levels, 8, 16, 50, mult)
  # the same graph under labels that reverse the order of the ids: equal distances among the
  # k best are listed by label, so the two answers differ in exactly those places
  labels = (np.uint64(3) * (n - 1 - np.arange(n, dtype=np.uint64)) + np.uint64(7))
  up = np.concatenate([np.concatenate([[len(base.links(i, l))], np.pad(base.links(i, l), (0, 8 - len(base.links(i, l))))])
                       for i in range(n) for l in range(1, levels[i] + 1)]).astype(np.uint32)
  relabelled = oracle.OracleIndex("l2").from_arrays(x, levels, base.links0(), up, 8, 16, base.maxlevel, base.enterpoint,
                                                    labels=labels)
  for tag, ix in (("ids", base), ("labels", relabelled)):
    p = str(tmp_path / ("qd_%s.idx" % tag))
    ix.save(p)
    e = _engine(tmp_path, dist_type="l2", max_m=8, max_m0=16)
    e.load_index(p)
    e.set_tunable("fast_path", 2)
    answered_by_first_pass = 0
    # (600, 600): more answers than the in-place ordering of equal distances has room for
    for k, ef in ((10, 64), (10, 300), (1, 16), (100, 100), (32, 33), (5, 319), (10, 700), (600, 600)):
      o_ids, o_d, o_f, o_cnt = ix.search(q, k, ef, counters=True)
      g_ids, g_d, g_f, stats = _device_search(e, q, k, ef)
      assert (g_f == o_f).all()
      for r in range(q.shape[0]):
        f = o_f[r]
        assert (g_ids[r, :f] == o_ids[r, :f]).all(), "%s query %d k %d ef %d" % (tag, r, k, ef)
        assert (g_d[r, :f] == o_d[r, :f]).all()
      assert (stats[:, 1:] == o_cnt[:, 1:4]).all()
      answered_by_first_pass += q.shape[0] - e.last_search_repeats
    assert answered_by_first_pass > 0
