#!/usr/bin/env python3
"""Build / search walk-through on the seeded synthetic data sets (counterpart of the
reference's examples/example1.py, which needs downloads, h5py and hnswlib).

  python examples/example_synthetic.py run_gpu_training  --workload C1 --index /tmp/c1.idx
  python examples/example_synthetic.py run_gpu_inference --workload C1 --index /tmp/c1.idx --topk 10 --ef-search 300
  python examples/example_synthetic.py run_experiments   --workload C1
  python examples/example_synthetic.py run_knob_sweep    --workload C2 --ef-list 30 50 300

Recall is measured against exact neighbours computed on the GPU with a plain matmul.
If the `hnswlib` package is importable, `run_cpu_inference` searches the same index file
with it and reports how many result rows are identical.
"""
import argparse
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import torch  # noqa: E402  (exact neighbours only; imported first so that one HIP runtime is loaded)

from cuhnsw_amd import CuHNSW, datasets  # noqa: E402


def exact_neighbours(data, queries, topk, dist_type):
  dd = torch.from_numpy(data).cuda()
  out = []
  for s in range(0, queries.shape[0], 500):
    qs = torch.from_numpy(queries[s:s + 500]).cuda()
    score = -(qs @ dd.T) if dist_type == "dot" else (dd * dd).sum(1)[None, :] - 2.0 * (qs @ dd.T)
    out.append(torch.topk(score, topk, dim=1, largest=False).indices.cpu().numpy())
  return np.concatenate(out)


def recall(found, truth):
  return float(np.mean([len(set(a) & set(b)) / truth.shape[1] for a, b in zip(found, truth)]))


def options(spec):
  return dict(spec["opt"], heuristic_coef=0.0, py_log_level=1)


def run_gpu_training(args):
  data, _, spec = datasets.make(args.workload, n=args.n)
  h = CuHNSW(options(spec))
  h.set_data(data)
  t0 = time.time()
  h.build()
  print("build: %.3f s (%d x %d, ef_construction=%d)" % (time.time() - t0, data.shape[0], data.shape[1],
                                                         spec["opt"]["ef_construction"]))
  h.save_index(args.index)
  print("index written to", args.index)


def run_gpu_inference(args):
  data, queries, spec = datasets.make(args.workload, n=args.n)
  h = CuHNSW(options(spec))
  h.load_index(args.index)
  h.search_knn(queries[:16], args.topk, args.ef_search)  # warm-up
  t0 = time.time()
  nns, dist, found = h.search_knn(queries, args.topk, args.ef_search)
  el = time.time() - t0
  truth = exact_neighbours(data, queries, args.topk, spec["opt"]["dist_type"])
  print("search: %d queries in %.4f s (%.0f QPS incl. transfers), recall@%d = %.4f" % (
      queries.shape[0], el, queries.shape[0] / el, args.topk, recall(nns, truth)))


def run_cpu_inference(args):
  try:
    import hnswlib
  except ImportError:
    print("hnswlib is not installed: nothing to compare with")
    return
  data, queries, spec = datasets.make(args.workload, n=args.n)
  space = "ip" if spec["opt"]["dist_type"] == "dot" else "l2"
  idx = hnswlib.Index(space=space, dim=data.shape[1])
  idx.load_index(args.index)
  idx.set_ef(args.ef_search)
  labels, _ = idx.knn_query(queries, k=args.topk)
  h = CuHNSW(options(spec))
  h.load_index(args.index)
  nns, _, _ = h.search_knn(queries, args.topk, args.ef_search)
  same = int((labels.astype(np.int64) == nns.astype(np.int64)).all(axis=1).sum())
  print("rows identical to hnswlib: %d / %d" % (same, queries.shape[0]))


def run_experiments(args):
  data, queries, spec = datasets.make(args.workload, n=args.n)
  truth = exact_neighbours(data, queries, args.topk, spec["opt"]["dist_type"])
  print("| ef_construction | build s | ef_search | QPS | recall@%d |" % args.topk)
  print("|---|---|---|---|---|")
  for efc in args.ef_construction or [spec["opt"]["ef_construction"]]:
    h = CuHNSW(dict(options(spec), ef_construction=efc))
    h.set_data(data)
    t0 = time.time()
    h.build()
    build_s = time.time() - t0
    for ef in args.ef_list or spec["ef"]:
      h.search_knn(queries[:16], args.topk, ef)
      t0 = time.time()
      nns, _, _ = h.search_knn(queries, args.topk, ef)
      el = time.time() - t0
      print("| %d | %.3f | %d | %.0f | %.4f |" % (efc, build_s, ef, queries.shape[0] / el, recall(nns, truth)))


def run_knob_sweep(args):
  """Build-side knobs the reference took over from n2 (README.md:97-98,104 of the reference): heuristic_coef
  (share of every link row filled with the nearest candidates untested), save_remains (pruned candidates fill
  the row) and reverse_cand (the farthest waiting candidate is expanded first during construction): build time
  and recall at several ef_search, all searched the same (plain) way."""
  data, queries, spec = datasets.make(args.workload, n=args.n)
  truth = exact_neighbours(data, queries, args.topk, spec["opt"]["dist_type"])
  efs = args.ef_list or [30, 50, 300]
  print("| heuristic_coef | save_remains | reverse_cand | build s | " + " | ".join("recall@%d ef %d" % (args.topk, e) for e in efs) + " |")
  print("|---|---|---|---|" + "---|" * len(efs))
  for coef, remains, reverse in ((0.0, False, False), (0.25, False, False), (0.5, False, False), (0.0, True, False),
                                 (0.25, True, False), (0.0, False, True), (0.25, False, True)):
    h = CuHNSW(dict(options(spec), heuristic_coef=coef, save_remains=remains, reverse_cand=reverse))
    h.set_data(data)
    h.build()
    build_s = h.obj.last_build_seconds()
    path = args.index + ".sweep"
    h.save_index(path)
    plain = CuHNSW(options(spec))            # search without reverse_cand, whatever the build used
    plain.load_index(path)
    os.remove(path)
    cells = []
    for ef in efs:
      nns, _, _ = plain.search_knn(queries, args.topk, ef)
      cells.append("%.4f" % recall(nns, truth))
    print("| %.2f | %s | %s | %.3f | %s |" % (coef, remains, reverse, build_s, " | ".join(cells)), flush=True)


def main():
  ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
  ap.add_argument("command", choices=["run_gpu_training", "run_gpu_inference", "run_cpu_inference", "run_experiments",
                                      "run_knob_sweep"])
  ap.add_argument("--workload", default="C1", choices=sorted(datasets.CONFIGS))
  ap.add_argument("--n", type=int, default=None, help="shrink the data set")
  ap.add_argument("--index", default="/tmp/cuhnsw_amd_example.idx")
  ap.add_argument("--topk", type=int, default=10)
  ap.add_argument("--ef-search", type=int, default=300)
  ap.add_argument("--ef-list", type=int, nargs="*")
  ap.add_argument("--ef-construction", type=int, nargs="*")
  args = ap.parse_args()
  globals()[args.command](args)


if __name__ == "__main__":
  main()
