#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--storage fp32|fp16] [--no-cpu]

Workload (default C2): the GloVe-50-shaped angular configuration — 1 183 514 x 50
float32 vectors from the seeded 1000-centre Gaussian mixture, L2-normalised,
dist_type=dot, max_m=12, max_m0=24, ef_construction=110; 10 000 queries, topk=10,
ef_search=300.  The index is built on the GPU (build seconds reported); one *step* is
one search pass of the whole query batch with queries and outputs resident in HBM.
Other workloads: C1, C3, C4, C5 (the other benchmark configurations) and R1 — the run
the reference's README times: the C2 index, one batch of 1 000 000 random unit queries,
topk=100, ef_search=300 (recall there is measured on the first 20 000 queries).

Prints one JSON line: value = search queries/s over the timed steps; `roofline`
prices the search kernel's algorithmic distance-gather bytes (sum over queries of
level-0 distance evaluations x 4*D, counted on the device) against the kernel time
measured with HIP events on the engine's stream; `cpu_baseline` times the CPU oracle
(hnswlib-semantics search of the same index file, and a bounded CPU build sample) on
this host's cores.
"""
import argparse
import csv
import glob
import hashlib
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "hbm_traffic.json")
KERNEL_SOURCES = ["device_core.h", "heap_coop.h", "kernels.h", "engine.hip"]


def kernel_source_digest():
  """Digest of the kernel sources without their comments and blank space: a traffic figure measured on other
  kernels is not reported."""
  h = hashlib.sha256()
  for name in KERNEL_SOURCES:
    with open(os.path.join(ROOT, "cuhnsw_amd", "csrc", name), "r") as f:
      for line in f:
        code = line.split("//", 1)[0].strip()
        if code:
          h.update(" ".join(code.split()).encode() + b"\n")
  return h.hexdigest()[:16]


def ingest_pmc(fetch_dir, write_dir, workload):
  """Turns two rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE; both with
  --profile --copy-calibration) into profiles/hbm_traffic.json: HBM bytes of one search of the
  batch = the counters summed over the search kernels' dispatches, divided by the number of searches,
  each scaled by what the same counter reads for the 256 MiB device copy of the calibration."""
  def read(directory, counter):
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
      raise SystemExit("no counter_collection.csv under " + directory)
    search, first_pass, copies = 0.0, 0, []
    for row in csv.DictReader(open(files[0])):
      if row["Counter_Name"] != counter:
        continue
      name, value = row["Kernel_Name"], float(row["Counter_Value"])
      if "cuhnsw_amd::search_" in name:
        search += value
        first_pass += "search_fast_kernel" in name
      elif "copyBuffer" in name:
        copies.append(value)
    if not first_pass or not copies:
      raise SystemExit("%s: no first-pass dispatches or no calibration copy in %s" % (counter, files[0]))
    return search / first_pass, max(copies), first_pass
  copy_bytes = 256 * 1024 * 1024
  fetch, copy_fetch, n_f = read(fetch_dir, "FETCH_SIZE")
  write, copy_write, n_w = read(write_dir, "WRITE_SIZE")
  out = {
      "workload": workload,
      "kernel_source_digest": kernel_source_digest(),
      "fetch_size_per_search": fetch, "write_size_per_search": write,
      "fetch_size_of_256MiB_copy": copy_fetch, "write_size_of_256MiB_copy": copy_write,
      "searches_counted": [n_f, n_w],
      "hbm_bytes_per_search": int(fetch * copy_bytes / copy_fetch + write * copy_bytes / copy_write),
      "fetch_bytes_per_search": int(fetch * copy_bytes / copy_fetch),
      "write_bytes_per_search": int(write * copy_bytes / copy_write),
  }
  with open(TRAFFIC_JSON, "w") as f:
    json.dump(out, f, indent=1)
    f.write("\n")
  print(json.dumps(out))


def measured_traffic(workload):
  """HBM bytes per search from profiles/hbm_traffic.json if it was measured on this workload with these
  kernel sources; else None."""
  try:
    with open(TRAFFIC_JSON) as f:
      t = json.load(f)
  except (OSError, ValueError):
    return None
  if t.get("workload") != workload or t.get("kernel_source_digest") != kernel_source_digest():
    return None
  return t.get("hbm_bytes_per_search")


def workload_text(name, n, d, o, nq, k, ef, storage):
  return "%s: %dx%d %s max_m=%d max_m0=%d ef_construction=%d; %d queries topk=%d ef_search=%d" % (
      name, n, d, o["dist_type"], o["max_m"], o["max_m0"], o["ef_construction"], nq, k, ef) + (
          "; vectors stored as fp16 (recall is against the exact neighbours of the unrounded vectors)"
          if storage == "fp16" else "")


def exact_topk(torch, data_dev, sq_dev, queries_dev, k, dot):
  """Exact top-k on the GPU (harness only).  Scores are produced in blocks of at most 2^28 elements (1 GiB):
  larger matmul outputs came back with wrong entries on this stack."""
  n = data_dev.shape[0]
  cols = 1 << 19
  out = []
  for s in range(0, queries_dev.shape[0], 512):
    qs = queries_dev[s:s + 512]
    best_v = best_i = None
    for c in range(0, n, cols):
      score = -(qs @ data_dev[c:c + cols].T)
      if not dot:
        score = sq_dev[None, c:c + cols] + 2.0 * score
      tv, ti = torch.topk(score, min(k, score.shape[1]), dim=1, largest=False)
      ti = ti + c
      if best_v is not None:
        tv, ti = torch.cat([best_v, tv], 1), torch.cat([best_i, ti], 1)
        tv, sel = torch.topk(tv, min(k, tv.shape[1]), dim=1, largest=False)
        ti = torch.gather(ti, 1, sel)
      best_v, best_i = tv, ti
    out.append(best_i.cpu().numpy())
  return np.concatenate(out)


def other_workload_rows(torch, capi, datasets, orc, tmpdir, name, efs, n_check=1000, n_recall=1000, steps=5):
  """One of the other benchmark configurations at its full size, compactly: build seconds, and per ef_search the
  search time of the whole batch (device pointers, HIP events on the engine's stream), QPS, recall, the
  distance-gather roofline fraction counted like the headline's (distinct evaluations of a literal-only pass
  x row bytes), the queries the literal pass answered, and the id rows that differ from the CPU oracle's on the
  first n_check queries of the index file the GPU wrote (orc = None: no CPU check)."""
  data, queries, spec = datasets.make(name)
  o = spec["opt"]
  n, d = data.shape
  nq, k = queries.shape[0], spec["topk"]
  dot = o["dist_type"] == "dot"
  mult = o.get("level_mult") or 1.0 / np.log(o["max_m"])
  levels = datasets.random_levels(n, mult)
  opt = dict(seed=777, c_log_level=2, py_log_level=2, max_m=o["max_m"], max_m0=o["max_m0"],
             ef_construction=o["ef_construction"], level_mult=mult, save_remains=False, hyper_threads=10.0,
             block_dim=32, dist_type=o["dist_type"], visited_table_size=0, visited_list_size=8192, nrz=False,
             reverse_cand=False, heuristic_coef=0.0)
  opt_path = os.path.join(tmpdir, "opt_%s.json" % name)
  with open(opt_path, "w") as f:
    json.dump(opt, f)
  eng = capi.Engine()
  assert eng.init(opt_path) == 0
  # the first launch of a kernel pays for loading its code: a small build and search of the same shape first
  m = min(n, 20000)
  eng.set_data(data[:m])
  eng.set_random_levels(levels[:m])
  eng.build_graph()
  eng.search_knn(queries[:64], k, efs[-1])
  eng.set_data(data)
  eng.set_random_levels(levels)
  eng.build_graph()
  build_s = eng.last_build_seconds
  dd = torch.from_numpy(data).cuda()
  qq = torch.from_numpy(queries).cuda()
  sq = None if dot else (dd * dd).sum(1)
  gt = exact_topk(torch, dd, sq, qq[:n_recall], k, dot)
  del dd, sq
  torch.cuda.empty_cache()
  ix = None
  if orc is not None:
    idx_path = os.path.join(tmpdir, "other_%s.idx" % name)
    eng.save_index(idx_path)
    ix = orc.OracleIndex(o["dist_type"]).load(idx_path)
    os.remove(idx_path)
  nns = torch.empty((nq, k), dtype=torch.int32, device="cuda")
  dist = torch.empty((nq, k), dtype=torch.float32, device="cuda")
  found = torch.empty(nq, dtype=torch.int32, device="cuda")
  stats = torch.zeros((nq, 4), dtype=torch.int32, device="cuda")
  torch.cuda.synchronize()

  def step(ef, with_stats=False):
    return eng.search_knn_device(qq.data_ptr(), nq, k, ef, nns.data_ptr(), dist.data_ptr(), found.data_ptr(),
                                 stats.data_ptr() if with_stats else None)

  rows = []
  for ef in efs:
    ef = max(ef, k)
    eng.set_tunable("fast_path", 0)
    step(ef, with_stats=True)              # literal queues only: the distinct evaluations
    n_dist = int(stats[:, 0].sum().item())
    eng.set_tunable("fast_path", 1)
    step(ef)
    ms = float(np.mean([step(ef) for _ in range(steps)]))
    handed = int(eng.last_search_repeats)
    ids = nns.cpu().numpy()
    recall = float(np.mean([len(set(a) & set(b)) / k for a, b in zip(ids[:n_recall], gt)]))
    gather = n_dist * 4 * d
    row = {"ef_search": ef, "search_ms": ms, "value": nq / (ms * 1e-3), "unit": "queries/s",
           "recall_at_%d" % k: recall, "frac": gather / (ms * 1e-3) / 8e12, "algorithmic_bytes_per_launch": gather,
           "queries_repeated_with_literal_queues": handed}
    if ix is not None:
      n_c = min(nq, n_check)
      o_ids, _, o_f = ix.search(queries[:n_c], k, ef, threads=orc.host_threads())
      row["oracle_rows_checked"] = n_c
      row["rows_with_id_mismatch_vs_oracle"] = int(((o_ids != ids[:n_c]).any(axis=1) |
                                                    (o_f != found[:n_c].cpu().numpy())).sum())
    rows.append(row)
  out = {"workload": "%s: %dx%d %s max_m=%d max_m0=%d ef_construction=%d; %d queries topk=%d" % (
             name, n, d, o["dist_type"], o["max_m"], o["max_m0"], o["ef_construction"], nq, k),
         "build_seconds": build_s, "rows": rows}
  eng.close()
  del ix, qq, nns, dist, found, stats, data, queries
  torch.cuda.empty_cache()
  return out


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=20)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--workload", default="C2")
  ap.add_argument("--n", type=int, default=None, help="shrink the data set (debugging)")
  ap.add_argument("--nq", type=int, default=None)
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
  ap.add_argument("--ef", type=int, default=None, help="ef_search (default: the configuration's headline value)")
  ap.add_argument("--storage", choices=["fp32", "fp16"], default="fp32",
                  help="element type of the vectors in device memory; fp16 = an index over the vectors rounded "
                       "to fp16, arithmetic stays fp32 (the default is the configuration the metric is quoted on)")
  ap.add_argument("--copy-calibration", action="store_true",
                  help="also run a plain 256 MiB device copy (reference point for rocprofv3 FETCH_SIZE / WRITE_SIZE)")
  ap.add_argument("--fast-path", type=int, default=1, choices=[0, 1, 2],
                  help="0 = literal priority queues only, 1 = default, 2 = sorted-set first pass whatever the batch size")
  ap.add_argument("--query-order", type=int, default=1, choices=[0, 1, 2],
                  help="0 = queries in the caller's order, 1 = longest first from one to one and a half rounds of wavefronts on, 2 = from one")
  ap.add_argument("--trails", type=int, default=1, choices=[0, 1, 2],
                  help="0 = the literal pass searches handed-over queries from the entry point, 1 = from the first pass's "
                       "trail in batches of up to two rounds of wavefronts (default), 2 = in every batch")
  ap.add_argument("--no-large", action="store_true", help="skip the extra 4x batch (profiling runs)")
  ap.add_argument("--no-others", action="store_true", help="skip the compact rows of the other benchmark configurations")
  ap.add_argument("--profile", action="store_true",
                  help="profiling run: only searches of the default path are launched (no literal-only counting pass, "
                       "no CPU baseline, no 4x batch); per_query and roofline then use the evaluations performed")
  ap.add_argument("--tight-rows", action="store_true",
                  help="vector rows padded to 16-byte chunks only instead of 128-byte lines (layout experiment)")
  ap.add_argument("--ingest-pmc", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                  help="no benchmark: write profiles/hbm_traffic.json from two rocprofv3 --pmc output directories")
  args = ap.parse_args()
  if args.profile:
    args.no_cpu = args.no_large = args.no_others = True
  if args.ingest_pmc:
    from cuhnsw_amd import datasets
    spec = datasets.CONFIGS[args.workload]
    k = spec["topk"]
    ef = max(args.ef or (300 if args.workload == "C2" else spec["ef"][-1]), k)
    ingest_pmc(args.ingest_pmc[0], args.ingest_pmc[1],
               workload_text(args.workload, args.n or spec["n"], spec["d"], spec["opt"], args.nq or spec["nq"], k, ef,
                             args.storage))
    return
  if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
    print("bench.py: this build runs on ONE GPU (the index and the query batch live on a single "
          "device; there is no multi-GPU path) — run with --gpus 1", file=sys.stderr)
    sys.exit(2)

  import torch  # device buffers only; loaded before the engine so that one HIP runtime is used
  from cuhnsw_amd import capi, datasets
  if not torch.cuda.is_available() or not capi.has_device():
    print("bench.py: no GPU visible", file=sys.stderr)
    sys.exit(3)

  t0 = time.time()
  data, queries, spec = datasets.make(args.workload, n=args.n, nq=args.nq)
  o = dict(spec["opt"])
  n, d = data.shape
  nq, k, ef = queries.shape[0], spec["topk"], spec["ef"][-1] if args.workload != "C2" else 300
  if args.ef:
    ef = max(args.ef, k)
  mult = o.get("level_mult") or 1.0 / np.log(o["max_m"])
  levels = datasets.random_levels(n, mult)
  gen_s = time.time() - t0

  opt = dict(seed=777, c_log_level=2, py_log_level=2, max_m=o["max_m"], max_m0=o["max_m0"],
             ef_construction=o["ef_construction"], level_mult=mult, save_remains=False, hyper_threads=10.0,
             block_dim=32, dist_type=o["dist_type"], visited_table_size=0, visited_list_size=8192, nrz=False,
             reverse_cand=False, heuristic_coef=0.0)
  tmpdir = tempfile.mkdtemp(prefix="cuhnsw_bench_")
  opt_path = os.path.join(tmpdir, "opt.json")
  with open(opt_path, "w") as f:
    json.dump(opt, f)
  eng = capi.Engine()
  assert eng.init(opt_path) == 0
  if args.storage == "fp16":
    eng.set_tunable("fp16_storage", 1)
  if args.tight_rows:
    eng.set_tunable("tight_rows", 1)
  t0 = time.time()
  eng.set_data(data)
  upload_s = time.time() - t0
  eng.set_tunable("build_counters", 1)
  eng.set_random_levels(levels)
  eng.build_graph()                      # warm-up build (first launch pays code loading); its work is counted
  build_work = eng.build_counters()
  eng.set_tunable("build_counters", 0)
  eng.set_random_levels(levels)
  eng.build_graph()                      # the timed build (same graph: the build is deterministic)
  build_s = eng.last_build_seconds
  eng.set_tunable("query_order", args.query_order)
  eng.set_tunable("trails", args.trails)

  # exact top-k on the GPU (harness only) for recall, measured on the first 20 000 queries of larger batches
  dd = torch.from_numpy(data).cuda()
  qq = torch.from_numpy(queries).cuda()
  sq = (dd * dd).sum(1) if o["dist_type"] != "dot" else None
  n_gt = min(nq, 20000)
  gt = exact_topk(torch, dd, sq, qq[:n_gt], k, o["dist_type"] == "dot")
  del dd, sq

  nns = torch.empty((nq, k), dtype=torch.int32, device="cuda")
  dist = torch.empty((nq, k), dtype=torch.float32, device="cuda")
  found = torch.empty(nq, dtype=torch.int32, device="cuda")
  stats = torch.zeros((nq, 4), dtype=torch.int32, device="cuda")
  torch.cuda.synchronize()

  def step(with_stats=False):
    return eng.search_knn_device(qq.data_ptr(), nq, k, ef, nns.data_ptr(), dist.data_ptr(), found.data_ptr(),
                                 stats.data_ptr() if with_stats else None)

  # algorithmic counters (distinct evaluations, expansions) come from a pass with the literal
  # queues only; the timed default path may evaluate a node again after its visited filter
  # has forgotten it, and those repeats must not count as useful bytes
  eng.set_tunable("fast_path", args.fast_path)
  step(with_stats=True)
  st_run = stats.cpu().numpy().astype(np.int64)
  st = st_run
  if not args.profile:
    eng.set_tunable("fast_path", 0)
    step(with_stats=True)
    st = stats.cpu().numpy().astype(np.int64)
    eng.set_tunable("fast_path", args.fast_path)
    step(with_stats=True)
  repeats = eng.last_search_repeats
  from_trails = eng.last_search_trails
  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  kernel_ms = []
  t0 = time.perf_counter()
  for _ in range(args.steps):
    kernel_ms.append(step())             # synchronous: returns after the kernel finished
  torch.cuda.synchronize()
  elapsed = time.perf_counter() - t0
  ids = nns.cpu().numpy()
  recall = float(np.mean([len(set(a) & set(b)) / k for a, b in zip(ids[:n_gt], gt)]))

  if args.copy_calibration:
    src = torch.full((64 * 1024 * 1024,), 1.0, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(3):
      dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

  # the same index with four times the batch (fresh queries of the same law): what the
  # kernels sustain once a launch holds several rounds of wavefronts.  Reported beside the
  # headline figure, never in its place.
  # the entry point most callers use (host pointers: queries staged to the device, results copied back)
  host_calls = 5 if nq <= 100000 else 2
  t0 = time.perf_counter()
  for _ in range(host_calls):
    h_ids, h_d, h_f = eng.search_knn(queries, k, ef)
  host_ms = (time.perf_counter() - t0) / host_calls * 1e3
  host_equal = bool((h_ids == ids).all())

  large = None
  if args.workload == "C2" and args.n is None and args.nq is None and not args.no_large:
    _, q_large, _ = datasets.make(args.workload, n=1, nq=4 * nq)
    ql = torch.from_numpy(q_large).cuda()
    nl = ql.shape[0]
    l_nns = torch.empty((nl, k), dtype=torch.int32, device="cuda")
    l_dist = torch.empty((nl, k), dtype=torch.float32, device="cuda")
    l_found = torch.empty(nl, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    l_ms = [eng.search_knn_device(ql.data_ptr(), nl, k, ef, l_nns.data_ptr(), l_dist.data_ptr(), l_found.data_ptr(), None)
            for _ in range(4)][1:]
    large = {"queries": nl, "search_ms": float(np.mean(l_ms)), "value": nl / (float(np.mean(l_ms)) * 1e-3), "unit": "queries/s"}
    del ql, l_nns, l_dist, l_found

  # The batch's time depends on whether, and when, one of its queries is handed to the literal pass: eight other
  # draws of as many queries from the same law (not part of `value`, which is quoted on the configuration's own queries).
  other_draws = None
  if args.workload == "C2" and args.n is None and args.nq is None and not args.no_large:
    times, handed = [], []
    for draw in range(8):
      qd = torch.from_numpy(datasets.more_queries(args.workload, nq, draw)).cuda()
      torch.cuda.synchronize()
      ms = [eng.search_knn_device(qd.data_ptr(), nq, k, ef, nns.data_ptr(), dist.data_ptr(), found.data_ptr(), None)
            for _ in range(5)][1:]
      times.append(float(np.mean(ms)))
      handed.append(int(eng.last_search_repeats))
    other_draws = {"draws": len(times), "queries": nq, "mean_ms": float(np.mean(times)), "min_ms": float(min(times)),
                   "max_ms": float(max(times)), "ms": [round(t, 3) for t in times],
                   "queries_repeated_with_literal_queues": handed}

  avg_kernel_ms = float(np.mean(kernel_ms))
  row_bytes_stored = (2 if args.storage == "fp16" else 4) * d
  gather_bytes = int(st[:, 0].sum()) * (2 if args.storage == "fp16" else 4) * d
  # HBM bytes of one search of the batch: read from profiles/hbm_traffic.json, which `--ingest-pmc` writes from
  # two rocprofv3 --pmc runs of this script; null when that file was measured on another workload or on
  # other kernel sources (it cannot be measured from inside this process)
  wl = workload_text(args.workload, n, d, o, nq, k, ef, args.storage) + ("; rows padded to 16 bytes" if args.tight_rows else "")
  traffic = measured_traffic(wl) if args.fast_path == 1 else None
  achieved = gather_bytes / (avg_kernel_ms * 1e-3) / 1e9
  out = {
      "metric": "batch search QPS at recall@%d (%s: %dx%d %s), with build seconds" % (
          k, args.workload, n, d, "angular" if o["dist_type"] == "dot" else "l2"),
      "value": nq * args.steps / elapsed,
      "unit": "queries/s",
      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
      "ms_per_step": elapsed / args.steps * 1e3,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
      "dtype": "f32", "data": "synthetic",
      "config": {"workload": wl},
      "build_seconds": build_s,
      "recall_at_k": recall,
      "upload_seconds": upload_s, "datagen_seconds": gen_s,
      "kernel_ms": avg_kernel_ms,
      "per_query": {"n_dist": float(st[:, 0].mean()), "n_hops": float(st[:, 1].mean()),
                    "n_dist_upper": float(st[:, 2].mean()), "n_sweeps_upper": float(st[:, 3].mean()),
                    "n_dist_performed": float(st_run[:, 0].mean()),
                    "queries_repeated_with_literal_queues": int(repeats),
                    "of_them_replayed_from_the_first_pass_trail": int(from_trails)},
      "roofline": {"bound": "hbm", "achieved": achieved, "peak": 8000.0, "unit": "GB/s",
                   "frac": achieved / 8000.0, "traffic": traffic,
                   "kernel": "search_fast_kernel with search_kernel beside it (one search of the batch)"
                             if args.fast_path else "search_kernel (literal priority queues only)",
                   "algorithmic_bytes_per_launch": gather_bytes},
      "host_pointer_search": {"ms_per_call": host_ms, "value": nq / (host_ms * 1e-3), "unit": "queries/s",
                              "same_ids_as_device_pointer_search": host_equal,
                              "note": "cuhnsw_search_knn: queries staged from pageable host memory, results copied back"},
  }
  # build roofline: bytes the build's kernels asked for, from device counters of an identical build
  row_bytes = (2 if args.storage == "fp16" else 4) * d
  lv0, up = build_work["level0"], build_work["upper"]
  s0 = (o["max_m0"] + 31) // 32 * 32 * 4
  su = (o["max_m"] + 15) // 16 * 16 * 4
  build_bytes = ((lv0[0] + lv0[2] + lv0[3] + up[0] + up[2] + up[3]) * row_bytes
                 + (lv0[1] + lv0[4]) * s0 + (up[1] + up[4]) * su)
  out["build_roofline"] = {
      "bound": "hbm", "achieved": build_bytes / build_s / 1e9, "peak": 8000.0, "unit": "GB/s",
      "frac": build_bytes / build_s / 1e9 / 8000.0, "algorithmic_bytes": int(build_bytes),
      "counters": {"names": ["distance evaluations (searches, descents)", "link rows read", "heuristic pair tests",
                             "heuristic candidate rows", "link rows written"], "level0": lv0, "upper_levels": up},
      "note": "vector rows x %d B + link rows x %d B (level 0) / %d B (upper levels), over build_seconds" % (row_bytes, s0, su),
  }

  if large:
    out["large_batch"] = large
  if other_draws:
    out["other_draws_of_the_queries"] = other_draws

  # the memory system alone: random gathers of this index's rows, with as many wavefronts per CU as the first
  # pass holds and as many rows in flight per wavefront as a hop fetches on average (4) and at most (16)
  probes = []
  for waves_per_cu, in_flight in ((28, 4), (28, 16), (8, 4)):
    rows, ms = eng.gather_probe(waves_per_cu, in_flight, True)
    probes.append({"waves_per_cu": waves_per_cu, "rows_in_flight_per_wavefront": in_flight, "rows_per_s": rows / (ms * 1e-3),
                   "GB_per_s": rows * row_bytes_stored / (ms * 1e-3) / 1e9,
                   "us_per_dependent_batch": ms * 1e3 / 2048.0})
  out["gather_ceiling"] = {"probes": probes, "search_rows_per_s": float(st_run[:, 0].sum()) / (avg_kernel_ms * 1e-3),
                           "note": "cuhnsw_debug_gather_probe: dependent batches of random row fetches over the resident vectors, "
                                   "nothing else; search_rows_per_s = evaluations the search performs per second"}

  if not args.no_cpu:
    from oracle import oracle as orc
    cores = orc.host_threads()
    idx_path = os.path.join(tmpdir, "bench.idx")
    eng.save_index(idx_path)
    ix = orc.OracleIndex(o["dist_type"]).load(idx_path)
    os.remove(idx_path)
    n_s = min(nq, 10000)
    passes = 0
    t0 = time.perf_counter()
    while passes < 2 or time.perf_counter() - t0 < 10.0:   # about 10 s of CPU search
      o_ids, o_d, o_f = ix.search(queries[:n_s], k, ef, threads=cores)
      passes += 1
    cpu_search_s = (time.perf_counter() - t0) / passes
    bad_rows = (o_ids != ids[:n_s]).any(axis=1)
    mism = int(bad_rows.sum())
    tied = ix.meets_ties(queries[:n_s], ef, threads=cores)   # queries whose search meets equal distances
    n_b = min(n, 400000)
    t0 = time.perf_counter()
    orc.OracleIndex(o["dist_type"]).build(data[:n_b], levels[:n_b], o["max_m"], o["max_m0"], o["ef_construction"],
                                          mult, threads=cores)
    cpu_build_s = time.perf_counter() - t0
    out["cpu_baseline"] = {
        "value": n_s / cpu_search_s, "unit": "queries/s", "cores": cores, "kind": "port",
        "sample": "CPU oracle (hnswlib-semantics search) on the GPU-built index file, first %d queries x %d passes, "
                  "topk=%d ef_search=%d; build sample: first %d points inserted in %.2f s (%.0f points/s)" % (
                      n_s, passes, k, ef, n_b, cpu_build_s, n_b / cpu_build_s),
        "build_points_per_s": n_b / cpu_build_s,
        "gpu_build_points_per_s": n / build_s,
    }
    out["parity"] = {"queries_checked": n_s, "rows_with_id_mismatch_vs_oracle": mism,
                     "queries_meeting_equal_distances": int(tied.sum()),
                     "id_mismatches_among_them": int((bad_rows & tied).sum()),
                     "id_mismatches_among_the_rest": int((bad_rows & ~tied).sum())}
  # the other benchmark configurations at full size, one compact block (the headline stays the workload above)
  if args.workload == "C2" and args.n is None and args.nq is None and not args.no_others:
    orc_mod = None
    if not args.no_cpu:
      from oracle import oracle as orc_mod
    eng.close()
    del eng, nns, dist, found, stats, qq, data, queries
    torch.cuda.empty_cache()
    t0 = time.time()
    out["other_workloads"] = [
        other_workload_rows(torch, capi, datasets, orc_mod, tmpdir, name, efs)
        for name, efs in (("C1", [300]), ("C3", [64, 128, 300]), ("C4", [300]), ("C5", [64, 128, 256, 512]))]
    out["other_workloads_seconds"] = time.time() - t0
  print(json.dumps(out))


if __name__ == "__main__":
  main()
