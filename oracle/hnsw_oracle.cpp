// CPU ORACLE — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A from-scratch CPU restatement of the hot path of js1010/cuhnsw (GPU HNSW
// build + batch search) with hnswlib semantics, used only as the checker in
// tests/, in __graft_entry__.smoke() and as the `cpu_baseline` leg of bench.py.
// The shipped library never links, loads or calls anything in this file.
//
// What each part follows (paths relative to the reference checkout):
//   * distance definitions ........ cpp/include/cuda_dist_kernels.cuh:112-124
//       (DOT / squared L2, no sqrt).  The ordering key for DOT is hnswlib's
//       `1.0f - dot`; the value handed back through the cuhnsw API is `-dot`.
//   * upper-level greedy descent .. cpp/include/cuda_search_kernels.cuh:22-66
//       (neighbour list captured once per sweep, strict `<`).
//   * level-0 ef-search ........... cpp/include/cuda_search_kernels.cuh:99-164
//       and cpp/include/cuda_utils_kernels.cuh:153-227 (accept rule
//       `size < ef || top > d`).  The reference claims id-equality with
//       hnswlib (README.md:112-113); because that only holds without distance
//       ties, this oracle restates hnswlib's own two-queue searchBaseLayerST on
//       std::priority_queue (libstdc++), which fixes the behaviour under ties.
//   * levels / entry point ........ cpp/src/cuhnsw_base.cu:130-156
//   * index file format ........... cpp/src/cuhnsw_base.cu:159-365
//   * label remap after load ...... cpp/src/cuhnsw_build.cu:284-286
//   * neighbour-selection heuristic cpp/include/cuda_build_kernels.cuh:68-162
//       (with heuristic_coef = 0, save_remains = false it is HNSW Alg. 4 /
//       hnswlib getNeighborsByHeuristic2).
//   * CPU build ................... hnswlib addPoint / mutuallyConnectNewElement
//       as used by examples/example1.py:64-142 (the reference's CPU
//       comparator).  hnswlib is a third-party dependency of the example
//       harness only (examples/requirements.txt:3, version unpinned) and its
//       source is not available offline; this is a restatement of its
//       published algorithm, kept in this one file.
//
// Parity status of each function:
//   canon_dist ............ pinned (closed form vs float64 numpy; exact on
//                           integer-valued data in any summation order)
//   heaps ................. std::priority_queue itself (libstdc++)
//   descent / search ...... pinned by brute force (ef >= N on a connected level
//                           0 returns the exact top-k), hand-walked tiny graphs
//                           and invariants; bit-parity with a *real* hnswlib
//                           binary is PARITY UNPINNED (not available offline).
//   search_layer_far ...... (reverse_cand, cpp/include/cuda_utils_kernels.cuh:104-151)
//                           pinned by a plain-Python statement of the same rule
//                           incl. hop and evaluation counts, and by brute force
//                           (ef >= N); against the CUDA reference itself PARITY
//                           UNPINNED: it cannot run here and leaves the order
//                           among equal distances to its warp reduction.
//   search_layer_deleted .. (hnswlib searchBaseLayerST on an index with deleted elements; the reference
//                           has no such notion) pinned by brute force over the elements that are left
//                           (ef >= N), by hand-walked chains whose only bridge is deleted and by
//                           "no mark == the plain search" (tests/test_oracle_deleted.py); against a real
//                           hnswlib binary PARITY UNPINNED.
//   file format ........... pinned by closed-form byte layout fixtures
//   select_reference ...... (the reference's SearchHeuristic incl. nn_num, save_remains, new_comer) pinned by
//                           closed-form point sets, by a brute-force statement of HNSW Alg. 4 on integer
//                           data and by the invariants that characterise its output
//                           (tests/test_oracle_heuristic.py)
//   select_neighbors ...... (hnswlib getNeighborsByHeuristic2, used by the CPU build) pinned the same way
//   build ................. quality only (recall vs brute force asserted >= 0.95 where it serves as a bar,
//                           graph invariants); PARITY UNPINNED against real hnswlib.
//
// Canonical fp32 distance arithmetic (shared by this oracle and the HIP
// kernels so that ids are bit-comparable): 64 partial sums, element i goes to
// partial (i mod 64) with one fused multiply-add per element in increasing i;
// the 64 partials are then combined by a pairwise adjacent tree
// (p[j] += p[j+s] for s = 1,2,4,...,32).
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <mutex>
#include <queue>
#include <string>
#include <set>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

enum { DIST_DOT = 0, DIST_L2 = 1 };

typedef std::pair<float, uint32_t> DistId;
struct CompareByFirst {
  bool operator()(const DistId& a, const DistId& b) const noexcept { return a.first < b.first; }
};
typedef std::priority_queue<DistId, std::vector<DistId>, CompareByFirst> MaxQueue;

// raw accumulated value: dot product (DOT) or squared L2
static inline float canon_accumulate(const float* a, const float* b, int D, int type) {
  float p[64];
  for (int j = 0; j < 64; ++j) p[j] = 0.0f;
  int base = 0;
  if (type == DIST_DOT) {
    for (; base + 64 <= D; base += 64)
      for (int j = 0; j < 64; ++j) p[j] = std::fmaf(a[base + j], b[base + j], p[j]);
    for (int j = 0; base + j < D; ++j) p[j] = std::fmaf(a[base + j], b[base + j], p[j]);
  } else {
    for (; base + 64 <= D; base += 64)
      for (int j = 0; j < 64; ++j) {
        float t = a[base + j] - b[base + j];
        p[j] = std::fmaf(t, t, p[j]);
      }
    for (int j = 0; base + j < D; ++j) {
      float t = a[base + j] - b[base + j];
      p[j] = std::fmaf(t, t, p[j]);
    }
  }
  for (int s = 1; s < 64; s <<= 1)
    for (int j = 0; j < 64; j += 2 * s) p[j] = p[j] + p[j + s];
  return p[0];
}

// ordering key: hnswlib convention (1 - dot, or squared L2)
static inline float canon_dist(const float* a, const float* b, int D, int type) {
  float acc = canon_accumulate(a, b, D, type);
  return type == DIST_DOT ? 1.0f - acc : acc;
}
// value returned through the cuhnsw API (cuda_dist_kernels.cuh:117,119)
static inline float api_dist(const float* a, const float* b, int D, int type) {
  float acc = canon_accumulate(a, b, D, type);
  return type == DIST_DOT ? -acc : acc;
}

struct Index {
  int N = 0, D = 0;
  int max_m = 12, max_m0 = 24;  // per-level caps (hnswlib maxM_, maxM0_)
  int M = 12;
  int ef_construction = 150;
  double mult = 0.0;
  int maxlevel = 0;
  uint32_t enterpoint = 0;
  int dist_type = DIST_DOT;
  std::vector<float> vectors;       // N x D
  std::vector<uint64_t> labels;     // N
  std::vector<int> levels;          // N (number of upper levels)
  std::vector<uint32_t> links0;     // N x (1 + max_m0): count, ids
  std::vector<size_t> upper_off;    // N: offset (in uint32) into linksU, valid if levels[i] > 0
  std::vector<uint32_t> linksU;     // sum(levels) x (1 + max_m)
  std::vector<uint8_t> deleted;     // N, or empty: hnswlib's delete marks (markDelete)
  int n_deleted = 0;
  std::string error;

  const float* vec(uint32_t i) const { return &vectors[(size_t)i * D]; }
  bool is_deleted(uint32_t i) const { return n_deleted > 0 && deleted[i] != 0; }
  uint32_t* list(uint32_t i, int level) {
    if (level == 0) return &links0[(size_t)i * (1 + max_m0)];
    return &linksU[upper_off[i] + (size_t)(level - 1) * (1 + max_m)];
  }
  const uint32_t* list(uint32_t i, int level) const {
    return const_cast<Index*>(this)->list(i, level);
  }
  void alloc_links() {
    links0.assign((size_t)N * (1 + max_m0), 0u);
    upper_off.assign(N, 0);
    size_t tot = 0;
    for (int i = 0; i < N; ++i) {
      upper_off[i] = tot;
      tot += (size_t)levels[i] * (1 + max_m);
    }
    linksU.assign(tot, 0u);
  }
};

// ---------------------------------------------------------------- file format
// Layout follows cpp/src/cuhnsw_base.cu:159-247 (writer) and :250-365 (reader).
template <typename T>
static void put(std::vector<char>& buf, const T& v) {
  const char* p = reinterpret_cast<const char*>(&v);
  buf.insert(buf.end(), p, p + sizeof(T));
}

static bool save_index(const Index& ix, const char* path) {
  FILE* f = std::fopen(path, "wb");
  if (!f) return false;
  const size_t size_links_level0 = (size_t)ix.max_m0 * 4 + 4;
  const size_t size_links_per_element = (size_t)ix.max_m * 4 + 4;
  const size_t size_data_per_element = size_links_level0 + (size_t)ix.D * 4 + 8;
  const size_t offsetData = size_links_level0;
  const size_t label_offset = size_links_level0 + (size_t)ix.D * 4;
  std::vector<char> h;
  put<size_t>(h, 0);  // offsetLevel0
  put<size_t>(h, (size_t)ix.N);
  put<size_t>(h, (size_t)ix.N);
  put<size_t>(h, size_data_per_element);
  put<size_t>(h, label_offset);
  put<size_t>(h, offsetData);
  put<int>(h, ix.maxlevel);
  put<uint32_t>(h, ix.enterpoint);
  put<size_t>(h, (size_t)ix.max_m);
  put<size_t>(h, (size_t)ix.max_m0);
  put<size_t>(h, (size_t)ix.M);
  put<double>(h, ix.mult);
  put<size_t>(h, (size_t)ix.ef_construction);
  bool ok = std::fwrite(h.data(), 1, h.size(), f) == h.size();
  std::vector<char> rec(size_data_per_element);
  for (int i = 0; i < ix.N && ok; ++i) {
    std::memset(rec.data(), 0, rec.size());
    const uint32_t* l = ix.list(i, 0);
    std::memcpy(rec.data(), l, 4 + 4 * (size_t)l[0]);
    if (ix.is_deleted((uint32_t)i)) rec[2] |= 0x01;  // hnswlib's DELETE_MARK: bit 0 of the count word's third byte
    std::memcpy(rec.data() + offsetData, ix.vec(i), (size_t)ix.D * 4);
    std::memcpy(rec.data() + label_offset, &ix.labels[i], 8);
    ok = std::fwrite(rec.data(), 1, rec.size(), f) == rec.size();
  }
  std::vector<char> up;
  for (int i = 0; i < ix.N && ok; ++i) {
    uint32_t sz = (uint32_t)(size_links_per_element * (size_t)ix.levels[i]);
    ok = std::fwrite(&sz, 4, 1, f) == 1;
    if (sz && ok) {
      up.assign(sz, 0);
      for (int l = 1; l <= ix.levels[i]; ++l) {
        const uint32_t* ll = ix.list(i, l);
        std::memcpy(up.data() + (size_t)(l - 1) * size_links_per_element, ll, 4 + 4 * (size_t)ll[0]);
      }
      ok = std::fwrite(up.data(), 1, sz, f) == sz;
    }
  }
  std::fclose(f);
  return ok;
}

template <typename T>
static bool get(FILE* f, T& v) { return std::fread(&v, sizeof(T), 1, f) == 1; }

static bool load_index(Index& ix, const char* path) {
  FILE* f = std::fopen(path, "rb");
  if (!f) { ix.error = "cannot open file"; return false; }
  size_t offsetLevel0, max_elements, cur, size_data_per_element, label_offset, offsetData, maxM, maxM0, M, efc;
  int maxlevel; uint32_t ep; double mult;
  bool ok = get(f, offsetLevel0) && get(f, max_elements) && get(f, cur) && get(f, size_data_per_element) &&
            get(f, label_offset) && get(f, offsetData) && get(f, maxlevel) && get(f, ep) && get(f, maxM) &&
            get(f, maxM0) && get(f, M) && get(f, mult) && get(f, efc);
  if (!ok) { std::fclose(f); ix.error = "truncated header"; return false; }
  ix.N = (int)cur; ix.max_m = (int)maxM; ix.max_m0 = (int)maxM0; ix.M = (int)M; ix.mult = mult;
  ix.ef_construction = (int)efc; ix.maxlevel = maxlevel; ix.enterpoint = ep;
  ix.D = (int)((label_offset - offsetData) / 4);
  const size_t size_links_per_element = maxM * 4 + 4;
  ix.vectors.resize((size_t)ix.N * ix.D);
  ix.labels.resize(ix.N);
  ix.levels.assign(ix.N, 0);
  ix.links0.assign((size_t)ix.N * (1 + ix.max_m0), 0u);
  ix.deleted.assign(ix.N, 0);
  ix.n_deleted = 0;
  std::vector<char> rec(size_data_per_element);
  for (int i = 0; i < ix.N; ++i) {
    if (std::fread(rec.data(), 1, rec.size(), f) != rec.size()) { std::fclose(f); ix.error = "truncated level-0 block"; return false; }
    uint32_t* l = &ix.links0[(size_t)i * (1 + ix.max_m0)];
    uint32_t word; std::memcpy(&word, rec.data(), 4);
    uint32_t cnt = word & 0xffffu;  // hnswlib keeps the count in the low 16 bits
    if (cnt > (uint32_t)ix.max_m0) { std::fclose(f); ix.error = "bad link count"; return false; }
    l[0] = cnt;
    if (word & 0x00010000u) { ix.deleted[i] = 1; ix.n_deleted++; }  // (hnswlib counts its marks the same way on load)
    std::memcpy(l + 1, rec.data() + 4, 4 * (size_t)cnt);
    std::memcpy(&ix.vectors[(size_t)i * ix.D], rec.data() + offsetData, (size_t)ix.D * 4);
    std::memcpy(&ix.labels[i], rec.data() + label_offset, 8);
  }
  // skip records of unused capacity (max_elements > cur_element_count)
  if (max_elements > cur) std::fseek(f, (long)((max_elements - cur) * size_data_per_element), SEEK_CUR);
  std::vector<std::vector<uint32_t>> tmp(ix.N);
  for (int i = 0; i < ix.N; ++i) {
    uint32_t sz;
    if (!get(f, sz)) { std::fclose(f); ix.error = "truncated upper block"; return false; }
    if (sz) {
      ix.levels[i] = (int)(sz / size_links_per_element);
      tmp[i].resize(sz / 4);
      if (std::fread(tmp[i].data(), 1, sz, f) != sz) { std::fclose(f); ix.error = "truncated upper block"; return false; }
    }
  }
  std::fclose(f);
  ix.upper_off.assign(ix.N, 0);
  size_t tot = 0;
  for (int i = 0; i < ix.N; ++i) { ix.upper_off[i] = tot; tot += (size_t)ix.levels[i] * (1 + ix.max_m); }
  ix.linksU.assign(tot, 0u);
  for (int i = 0; i < ix.N; ++i)
    for (int l = 1; l <= ix.levels[i]; ++l) {
      const uint32_t* src = &tmp[i][(size_t)(l - 1) * (1 + ix.max_m)];
      uint32_t* dst = ix.list(i, l);
      uint32_t cnt = src[0] & 0xffffu;
      if (cnt > (uint32_t)ix.max_m) { ix.error = "bad upper link count"; return false; }
      dst[0] = cnt;
      std::memcpy(dst + 1, src + 1, 4 * (size_t)cnt);
    }
  return true;
}

// ------------------------------------------------------------------- search
struct Visited {
  std::vector<uint32_t> tag;
  uint32_t epoch = 0;
  void reset(int n) {
    if ((int)tag.size() != n) { tag.assign(n, 0u); epoch = 0; }
    if (++epoch == 0) { std::fill(tag.begin(), tag.end(), 0u); epoch = 1; }
  }
  bool test_and_set(uint32_t i) { if (tag[i] == epoch) return true; tag[i] = epoch; return false; }
};

struct Counters { long long n_dist = 0, n_hops = 0, n_dist_upper = 0, n_sweeps_upper = 0, max_cand = 0; };

// One upper level of greedy descent (cuda_search_kernels.cuh:40-66; hnswlib searchKnn upper loop).
static void descend_level(const Index& ix, const float* q, int level, uint32_t& cur, float& dcur, Counters* c) {
  bool changed = true;
  while (changed) {
    changed = false;
    const uint32_t* l = ix.list(cur, level);  // list captured once per sweep
    uint32_t cnt = l[0];
    if (c) c->n_sweeps_upper++;
    for (uint32_t i = 0; i < cnt; ++i) {
      uint32_t cand = l[1 + i];
      float d = canon_dist(q, ix.vec(cand), ix.D, ix.dist_type);
      if (c) c->n_dist_upper++;
      if (d < dcur) { dcur = d; cur = cand; changed = true; }
    }
  }
}

// hnswlib searchBaseLayerST restated; returns top_candidates (max-queue, <= ef entries).
static MaxQueue search_layer(const Index& ix, const float* q, uint32_t ep, float dep, int level, size_t ef,
                             Visited& vis, Counters* c, int exclude = -1) {
  MaxQueue top, cand;  // cand holds (-dist, id)
  float lowerBound = dep;
  top.emplace(dep, ep);
  cand.emplace(-dep, ep);
  vis.test_and_set(ep);
  if (exclude >= 0) vis.test_and_set((uint32_t)exclude);
  while (!cand.empty()) {
    DistId cur = cand.top();
    if ((-cur.first) > lowerBound) break;
    cand.pop();
    if (c) c->n_hops++;
    const uint32_t* l = ix.list(cur.second, level);
    uint32_t cnt = l[0];
    for (uint32_t j = 0; j < cnt; ++j) {
      uint32_t n = l[1 + j];
      if (vis.test_and_set(n)) continue;
      float d = canon_dist(q, ix.vec(n), ix.D, ix.dist_type);
      if (c) c->n_dist++;
      if (top.size() < ef || lowerBound > d) {
        cand.emplace(-d, n);
        top.emplace(d, n);
        if (top.size() > ef) top.pop();
        if (!top.empty()) lowerBound = top.top().first;
        if (c && (long long)cand.size() > c->max_cand) c->max_cand = (long long)cand.size();
      }
    }
  }
  return top;
}

// hnswlib searchBaseLayerST as it runs on an index that holds deleted elements (its has_deletions /
// non-bare-bone form, no filter): a deleted element is visited, evaluated, queued and expanded like any
// other, but never enters the result queue; the search stops only once the result queue is FULL and the
// nearest candidate lies beyond its largest key (a queue still short of ef never stops it: deleted
// candidates beyond the bound are walked through); the bound moves only while the result queue holds
// something.  A deleted entry point is queued with the largest float as its key and is not evaluated by
// hnswlib; it is the queue's only entry when it is taken, so its key decides nothing, and the evaluation
// is counted here as for any entry point.  The reference itself knows no deleted elements (it reads the
// count word as a plain count, cpp/src/cuhnsw_base.cu:311-312).
static MaxQueue search_layer_deleted(const Index& ix, const float* q, uint32_t ep, float dep, int level, size_t ef,
                                     Visited& vis, Counters* c) {
  MaxQueue top, cand;
  float lowerBound;
  if (!ix.is_deleted(ep)) {
    lowerBound = dep;
    top.emplace(dep, ep);
    cand.emplace(-dep, ep);
  } else {
    lowerBound = std::numeric_limits<float>::max();
    cand.emplace(-lowerBound, ep);
  }
  vis.test_and_set(ep);
  while (!cand.empty()) {
    DistId cur = cand.top();
    if ((-cur.first) > lowerBound && top.size() == ef) break;
    cand.pop();
    if (c) c->n_hops++;
    const uint32_t* l = ix.list(cur.second, level);
    uint32_t cnt = l[0];
    for (uint32_t j = 0; j < cnt; ++j) {
      uint32_t n = l[1 + j];
      if (vis.test_and_set(n)) continue;
      float d = canon_dist(q, ix.vec(n), ix.D, ix.dist_type);
      if (c) c->n_dist++;
      if (top.size() < ef || lowerBound > d) {
        cand.emplace(-d, n);
        if (!ix.is_deleted(n)) top.emplace(d, n);
        if (top.size() > ef) top.pop();
        if (!top.empty()) lowerBound = top.top().first;
        if (c && (long long)cand.size() > c->max_cand) c->max_cand = (long long)cand.size();
      }
    }
  }
  return top;
}

// The reference's reverse_cand search (cuda_search_kernels.cuh:99-164 with GetCand(..., reverse = true),
// cuda_utils_kernels.cuh:104-151): the result set of at most ef entries is also the candidate set; the
// FARTHEST entry not yet expanded is expanded next, until none is left.  Not an hnswlib search.  The
// reference leaves the order among equal distances to its warp reduction; here equal keys keep their
// order of arrival (a stable sorted insert), the entry evicted from a full set is the last one, and the
// result is the first k entries in that order.  Returns the set, ascending.
struct SetEntry { float key; uint32_t id; bool expanded; };
static std::vector<SetEntry> search_layer_far(const Index& ix, const float* q, uint32_t ep, float dep, int level, size_t ef,
                                              Visited& vis, Counters* c) {
  std::vector<SetEntry> set;
  set.push_back({dep, ep, false});
  vis.test_and_set(ep);
  for (;;) {
    int pick = -1;
    for (int i = (int)set.size() - 1; i >= 0; --i) if (!set[i].expanded) { pick = i; break; }
    if (pick < 0) break;
    set[pick].expanded = true;
    if (c) c->n_hops++;
    const uint32_t* l = ix.list(set[pick].id, level);
    uint32_t cnt = l[0];
    for (uint32_t j = 0; j < cnt; ++j) {
      uint32_t n = l[1 + j];
      if (vis.test_and_set(n)) continue;
      float d = canon_dist(q, ix.vec(n), ix.D, ix.dist_type);
      if (c) c->n_dist++;
      if (set.size() < ef || set.back().key > d) {
        size_t pos = set.size();
        while (pos > 0 && set[pos - 1].key > d) --pos;   // after every entry with key <= d
        set.insert(set.begin() + pos, {d, n, false});
        if (set.size() > ef) set.pop_back();
      }
    }
  }
  return set;
}
static int search_one_far(const Index& ix, const float* q, int k, int ef, Visited& vis, Counters* c,
                          int* out_ids, float* out_d, int convention) {
  if (ix.N == 0) return 0;
  uint32_t cur = ix.enterpoint;
  float dcur = canon_dist(q, ix.vec(cur), ix.D, ix.dist_type);
  for (int level = ix.maxlevel; level > 0; --level) descend_level(ix, q, level, cur, dcur, c);
  vis.reset(ix.N);
  if (c) c->n_dist++;
  std::vector<SetEntry> set = search_layer_far(ix, q, cur, dcur, 0, (size_t)std::max(ef, k), vis, c);
  int found = (int)std::min<size_t>(set.size(), (size_t)k);
  for (int i = 0; i < found; ++i) {
    out_ids[i] = (int)ix.labels[set[i].id];
    out_d[i] = convention == 1 ? api_dist(q, ix.vec(set[i].id), ix.D, ix.dist_type) : set[i].key;
  }
  return found;
}

// The same search, only to learn whether the query meets equal distances on its way: true if a key
// accepted into the result set equals a key that is in the result set at that moment.  Those are the
// queries whose answer can depend on how the priority queues lay equal keys out (the reference's README
// claims id-equality with hnswlib, README.md:112-113, which its single-heap kernel can only keep for the
// others).
static bool search_meets_ties(const Index& ix, const float* q, uint32_t ep, float dep, size_t ef, Visited& vis) {
  MaxQueue top, cand;
  std::multiset<float> keys;
  bool met = false;
  float lowerBound = dep;
  top.emplace(dep, ep);
  cand.emplace(-dep, ep);
  keys.insert(dep);
  vis.test_and_set(ep);
  while (!cand.empty()) {
    DistId cur = cand.top();
    if ((-cur.first) > lowerBound) break;
    cand.pop();
    const uint32_t* l = ix.list(cur.second, 0);
    uint32_t cnt = l[0];
    for (uint32_t j = 0; j < cnt; ++j) {
      uint32_t n = l[1 + j];
      if (vis.test_and_set(n)) continue;
      float d = canon_dist(q, ix.vec(n), ix.D, ix.dist_type);
      if (top.size() < ef || lowerBound > d) {
        if (keys.count(d)) met = true;
        keys.insert(d);
        cand.emplace(-d, n);
        top.emplace(d, n);
        if (top.size() > ef) { keys.erase(keys.find(top.top().first)); top.pop(); }
        if (!top.empty()) lowerBound = top.top().first;
      }
    }
  }
  return met;
}

// hnswlib searchKnn restated; results ascending by (distance, label) as the hnswlib python binding emits them.
static int search_one(const Index& ix, const float* q, int k, int ef, Visited& vis, Counters* c,
                      int* out_ids, float* out_d, int convention) {
  if (ix.N == 0) return 0;
  uint32_t cur = ix.enterpoint;
  float dcur = canon_dist(q, ix.vec(cur), ix.D, ix.dist_type);
  for (int level = ix.maxlevel; level > 0; --level) descend_level(ix, q, level, cur, dcur, c);
  vis.reset(ix.N);
  if (c) c->n_dist++;  // the entry's level-0 evaluation is counted once
  // (hnswlib: the bare-bone search while nothing is marked deleted, the other form as soon as something is)
  MaxQueue top = ix.n_deleted > 0 ? search_layer_deleted(ix, q, cur, dcur, 0, (size_t)std::max(ef, k), vis, c)
                                  : search_layer(ix, q, cur, dcur, 0, (size_t)std::max(ef, k), vis, c);
  while ((int)top.size() > k) top.pop();
  std::vector<std::pair<float, uint64_t>> res;
  std::vector<uint32_t> internal;
  while (!top.empty()) { res.emplace_back(top.top().first, ix.labels[top.top().second]); internal.push_back(top.top().second); top.pop(); }
  // the python binding drains a priority_queue<pair<dist,label>> (full pair order) from the back
  std::vector<size_t> ord(res.size());
  for (size_t i = 0; i < ord.size(); ++i) ord[i] = i;
  std::sort(ord.begin(), ord.end(), [&](size_t a, size_t b) { return res[a] < res[b]; });
  int found = (int)res.size();
  for (int i = 0; i < found; ++i) {
    out_ids[i] = (int)res[ord[i]].second;
    out_d[i] = convention == 1 ? api_dist(q, ix.vec(internal[ord[i]]), ix.D, ix.dist_type) : res[ord[i]].first;
  }
  return found;
}

// ------------------------------------------------------------------- build
// hnswlib getNeighborsByHeuristic2 restated (== cuda_build_kernels.cuh:68-162 with
// heuristic_coef = 0, save_remains = false, new_comer = -1).
static void select_neighbors(const Index& ix, MaxQueue& top, size_t M) {
  if (top.size() < M) return;
  MaxQueue closest;
  std::vector<DistId> ret;
  while (!top.empty()) { closest.emplace(-top.top().first, top.top().second); top.pop(); }
  while (!closest.empty()) {
    if (ret.size() >= M) break;
    DistId cur = closest.top();
    float dq = -cur.first;
    closest.pop();
    bool good = true;
    for (const DistId& r : ret) {
      float d = canon_dist(ix.vec(r.second), ix.vec(cur.second), ix.D, ix.dist_type);
      if (d < dq) { good = false; break; }
    }
    if (good) ret.push_back(cur);
  }
  for (const DistId& r : ret) top.emplace(-r.first, r.second);
}

// The reference's SearchHeuristic restated in full (cpp/include/cuda_build_kernels.cuh:68-162): HNSW Alg. 4 plus
// the two n2-style extras and the new_comer shortcut of its reverse-link pass.
//   cand        candidates of `target`, ascending by their key to the target (the reference drains its heap
//               into that order, :82-88)
//   nn_num      the first nn_num picks pass untested (= int(max_m * float(heuristic_coef)), :101,105)
//   save_remains pruned candidates fill the row from its last slot backwards while slots are left (:140-145)
//               and the degree becomes min(max_m, |cand|) instead of the number of picks (:160)
//   new_comer   >= 0: every candidate ahead of the newcomer passes untested, the newcomer itself is tested
//               against all picks so far, and candidates after an accepted newcomer are tested against the
//               newcomer alone (:105-106,120-123,135-136); -1 switches that off
// A candidate c is pruned when its key to the target is strictly greater than its key to a pick (:121,126).
// Returns the degree; row[0..degree) is the new link list with its keys (slots between the picks and the
// tail fill are only meaningful with save_remains, where there are none left over).
static int select_reference(const Index& ix, const std::vector<DistId>& cand, int max_m, int nn_num, bool save_remains,
                            int new_comer, std::vector<DistId>& row, long long* pair_tests = nullptr) {
  const int T = (int)cand.size();
  int head = 0;
  int tail = std::min(max_m, T) - 1;
  const int max_head = tail + 1;
  row.assign((size_t)std::max(max_head, 0), DistId(0.0f, 0xFFFFFFFFu));
  bool inserted = false;
  for (int j = 0; j < T; ++j) {
    if (head >= max_m) break;
    const uint32_t c = cand[j].second;
    const float to_target = cand[j].first;
    const bool freepass = head < nn_num || (new_comer >= 0 && !inserted && c != (uint32_t)new_comer);
    if (freepass) {
      row[head++] = cand[j];
      continue;
    }
    bool skip = false;
    if (new_comer >= 0 && inserted) {
      if (pair_tests) ++*pair_tests;
      skip = to_target > canon_dist(ix.vec(c), ix.vec((uint32_t)new_comer), ix.D, ix.dist_type);
    } else {
      for (int k = 0; k < head && !skip; ++k) {
        if (pair_tests) ++*pair_tests;
        skip = to_target > canon_dist(ix.vec(c), ix.vec(row[k].second), ix.D, ix.dist_type);
      }
    }
    if (new_comer >= 0 && c == (uint32_t)new_comer && !skip) inserted = true;
    if (skip && tail >= head) row[tail--] = cand[j];
    else if (!skip) row[head++] = cand[j];
  }
  return save_remains ? max_head : head;
}

struct BuildCtx {
  std::vector<std::mutex> locks;
  std::mutex global;
  explicit BuildCtx(int n) : locks(n) {}
};

static uint32_t connect_new(Index& ix, BuildCtx& bc, uint32_t cur_c, MaxQueue& top, int level) {
  const size_t Mcurmax = level ? ix.max_m : ix.max_m0;
  select_neighbors(ix, top, (size_t)ix.M);
  std::vector<uint32_t> sel;
  while (!top.empty()) { sel.push_back(top.top().second); top.pop(); }
  uint32_t next_ep = sel.back();
  {
    std::lock_guard<std::mutex> g(bc.locks[cur_c]);
    uint32_t* l = ix.list(cur_c, level);
    l[0] = (uint32_t)sel.size();
    for (size_t i = 0; i < sel.size(); ++i) l[1 + i] = sel[i];
  }
  for (uint32_t nb : sel) {
    std::lock_guard<std::mutex> g(bc.locks[nb]);
    uint32_t* l = ix.list(nb, level);
    uint32_t cnt = l[0];
    if (cnt < Mcurmax) {
      l[1 + cnt] = cur_c;
      l[0] = cnt + 1;
    } else {
      MaxQueue cands;
      cands.emplace(canon_dist(ix.vec(cur_c), ix.vec(nb), ix.D, ix.dist_type), cur_c);
      for (uint32_t j = 0; j < cnt; ++j)
        cands.emplace(canon_dist(ix.vec(l[1 + j]), ix.vec(nb), ix.D, ix.dist_type), l[1 + j]);
      select_neighbors(ix, cands, Mcurmax);
      uint32_t k = 0;
      while (!cands.empty()) { l[1 + k++] = cands.top().second; cands.pop(); }
      l[0] = k;
    }
  }
  return next_ep;
}

// search during construction: reads neighbour lists under the node lock, as hnswlib searchBaseLayer
static MaxQueue search_layer_build(Index& ix, BuildCtx& bc, const float* q, uint32_t ep, int level, Visited& vis) {
  MaxQueue top, cand;
  const size_t ef = (size_t)ix.ef_construction;
  float dep = canon_dist(q, ix.vec(ep), ix.D, ix.dist_type);
  float lowerBound = dep;
  top.emplace(dep, ep);
  cand.emplace(-dep, ep);
  vis.test_and_set(ep);
  std::vector<uint32_t> nb;
  while (!cand.empty()) {
    DistId cur = cand.top();
    if ((-cur.first) > lowerBound && top.size() == ef) break;
    cand.pop();
    {
      std::lock_guard<std::mutex> g(bc.locks[cur.second]);
      const uint32_t* l = ix.list(cur.second, level);
      nb.assign(l + 1, l + 1 + l[0]);
    }
    for (uint32_t n : nb) {
      if (vis.test_and_set(n)) continue;
      float d = canon_dist(q, ix.vec(n), ix.D, ix.dist_type);
      if (top.size() < ef || lowerBound > d) {
        cand.emplace(-d, n);
        top.emplace(d, n);
        if (top.size() > ef) top.pop();
        if (!top.empty()) lowerBound = top.top().first;
      }
    }
  }
  return top;
}

static void add_point(Index& ix, BuildCtx& bc, uint32_t cur_c, Visited& vis, std::atomic<int>& maxlevel,
                      std::atomic<long long>& enterpoint) {
  const int curlevel = ix.levels[cur_c];
  std::unique_lock<std::mutex> tl(bc.global);
  int maxlevelcopy = maxlevel.load();
  if (curlevel <= maxlevelcopy) tl.unlock();
  long long ep = enterpoint.load();
  if (ep >= 0) {
    uint32_t cur = (uint32_t)ep;
    const float* q = ix.vec(cur_c);
    if (curlevel < maxlevelcopy) {
      float dcur = canon_dist(q, ix.vec(cur), ix.D, ix.dist_type);
      for (int level = maxlevelcopy; level > curlevel; --level) {
        bool changed = true;
        std::vector<uint32_t> nb;
        while (changed) {
          changed = false;
          {
            std::lock_guard<std::mutex> g(bc.locks[cur]);
            const uint32_t* l = ix.list(cur, level);
            nb.assign(l + 1, l + 1 + l[0]);
          }
          for (uint32_t cand : nb) {
            float d = canon_dist(q, ix.vec(cand), ix.D, ix.dist_type);
            if (d < dcur) { dcur = d; cur = cand; changed = true; }
          }
        }
      }
    }
    for (int level = std::min(curlevel, maxlevelcopy); level >= 0; --level) {
      vis.reset(ix.N);
      vis.test_and_set(cur_c);
      MaxQueue top = search_layer_build(ix, bc, q, cur, level, vis);
      cur = connect_new(ix, bc, cur_c, top, level);
    }
  } else {
    enterpoint.store(cur_c);
    maxlevel.store(curlevel);
  }
  if (curlevel > maxlevelcopy) { enterpoint.store(cur_c); maxlevel.store(curlevel); }
}

static void build_index(Index& ix, int threads) {
  ix.alloc_links();
  ix.labels.resize(ix.N);
  for (int i = 0; i < ix.N; ++i) ix.labels[i] = (uint64_t)i;
  BuildCtx bc(ix.N);
  std::atomic<int> maxlevel(-1);
  std::atomic<long long> enterpoint(-1);
  if (ix.N == 0) return;
  {
    Visited vis;
    add_point(ix, bc, 0, vis, maxlevel, enterpoint);  // hnswlib python: first element alone
  }
#pragma omp parallel num_threads(threads)
  {
    Visited vis;
#pragma omp for schedule(dynamic, 64)
    for (int i = 1; i < ix.N; ++i) add_point(ix, bc, (uint32_t)i, vis, maxlevel, enterpoint);
  }
  ix.maxlevel = maxlevel.load();
  ix.enterpoint = (uint32_t)enterpoint.load();
}

}  // namespace

// ---------------------------------------------------------------- C ABI (ctypes)
extern "C" {

void* orc_create() { return new Index(); }
void orc_free(void* h) { delete static_cast<Index*>(h); }
const char* orc_error(void* h) { return static_cast<Index*>(h)->error.c_str(); }

int orc_load(void* h, const char* path, int dist_type) {
  Index& ix = *static_cast<Index*>(h);
  ix.dist_type = dist_type;
  return load_index(ix, path) ? 1 : 0;
}
int orc_save(void* h, const char* path) { return save_index(*static_cast<Index*>(h), path) ? 1 : 0; }

// assemble an index from flat arrays (tests hand-build tiny graphs with it)
//   links0: N x (1+max_m0) uint32 (count, ids); linksU: concatenated per node, levels[i] x (1+max_m)
int orc_from_arrays(void* h, const float* vectors, int N, int D, const int* levels, const uint32_t* links0,
                    const uint32_t* linksU, const uint64_t* labels, int max_m, int max_m0, int maxlevel,
                    uint32_t enterpoint, int dist_type, double mult, int efc) {
  Index& ix = *static_cast<Index*>(h);
  ix.N = N; ix.D = D; ix.max_m = max_m; ix.max_m0 = max_m0; ix.M = max_m; ix.maxlevel = maxlevel;
  ix.enterpoint = enterpoint; ix.dist_type = dist_type; ix.mult = mult; ix.ef_construction = efc;
  ix.vectors.assign(vectors, vectors + (size_t)N * D);
  ix.levels.assign(levels, levels + N);
  ix.alloc_links();
  std::memcpy(ix.links0.data(), links0, ix.links0.size() * 4);
  if (!ix.linksU.empty()) std::memcpy(ix.linksU.data(), linksU, ix.linksU.size() * 4);
  ix.labels.resize(N);
  for (int i = 0; i < N; ++i) ix.labels[i] = labels ? labels[i] : (uint64_t)i;
  ix.deleted.clear(); ix.n_deleted = 0;
  return 1;
}

// hnswlib-semantics CPU build with externally supplied levels (so that the level
// assignment equals the one the Python wrapper draws, cuhnsw/pyhnsw.py:65-71)
int orc_build(void* h, const float* data, int N, int D, const int* levels, int dist_type, int max_m, int max_m0,
              int ef_construction, double mult, int threads) {
  Index& ix = *static_cast<Index*>(h);
  ix.N = N; ix.D = D; ix.max_m = max_m; ix.max_m0 = max_m0; ix.M = max_m; ix.dist_type = dist_type;
  ix.ef_construction = ef_construction; ix.mult = mult;
  ix.vectors.assign(data, data + (size_t)N * D);
  ix.levels.assign(levels, levels + N);
  ix.deleted.clear(); ix.n_deleted = 0;
  build_index(ix, threads > 0 ? threads : 1);
  return 1;
}

// hnswlib markDelete / unmarkDelete on internal ids; returns the number of marked elements, -1 on a bad id
int orc_mark_deleted(void* h, const unsigned* ids, int n, int mark) {
  Index& ix = *static_cast<Index*>(h);
  if ((int)ix.deleted.size() != ix.N) ix.deleted.assign(ix.N, 0);
  for (int i = 0; i < n; ++i) {
    if (ids[i] >= (unsigned)ix.N) return -1;
    ix.deleted[ids[i]] = mark ? 1 : 0;
  }
  ix.n_deleted = 0;
  for (int i = 0; i < ix.N; ++i) ix.n_deleted += ix.deleted[i] ? 1 : 0;
  return ix.n_deleted;
}
int orc_num_deleted(void* h) { return static_cast<Index*>(h)->n_deleted; }
int orc_num_data(void* h) { return static_cast<Index*>(h)->N; }
int orc_num_dims(void* h) { return static_cast<Index*>(h)->D; }
int orc_maxlevel(void* h) { return static_cast<Index*>(h)->maxlevel; }
unsigned orc_enterpoint(void* h) { return static_cast<Index*>(h)->enterpoint; }
int orc_max_m(void* h) { return static_cast<Index*>(h)->max_m; }
int orc_max_m0(void* h) { return static_cast<Index*>(h)->max_m0; }
void orc_get_levels(void* h, int* out) { Index& ix = *static_cast<Index*>(h); std::memcpy(out, ix.levels.data(), (size_t)ix.N * 4); }
void orc_get_vectors(void* h, float* out) { Index& ix = *static_cast<Index*>(h); std::memcpy(out, ix.vectors.data(), ix.vectors.size() * 4); }
void orc_get_labels(void* h, uint64_t* out) { Index& ix = *static_cast<Index*>(h); std::memcpy(out, ix.labels.data(), (size_t)ix.N * 8); }
// copies the link list of `node` at `level` into out (capacity max_m0); returns the count, -1 if the node has no such level
int orc_get_links(void* h, int node, int level, unsigned* out) {
  Index& ix = *static_cast<Index*>(h);
  if (node < 0 || node >= ix.N || level < 0 || level > ix.levels[node]) return -1;
  const uint32_t* l = ix.list((uint32_t)node, level);
  std::memcpy(out, l + 1, 4 * (size_t)l[0]);
  return (int)l[0];
}
// whole level-0 table: N x (1+max_m0)
void orc_get_links0(void* h, unsigned* out) { Index& ix = *static_cast<Index*>(h); std::memcpy(out, ix.links0.data(), ix.links0.size() * 4); }

float orc_distance(const float* a, const float* b, int D, int dist_type) { return canon_dist(a, b, D, dist_type); }
float orc_api_distance(const float* a, const float* b, int D, int dist_type) { return api_dist(a, b, D, dist_type); }

// batch search. counters (may be null): per query n_dist, n_hops (level 0), n_dist_upper, n_sweeps_upper, max candidate-queue size
// convention: 0 = hnswlib distances (1-dot), 1 = cuhnsw API distances (-dot)
void orc_search(void* h, const float* q, int nq, int k, int ef, int* ids, float* dists, int* found, long long* counters,
                int threads, int convention) {
  const Index& ix = *static_cast<Index*>(h);
#pragma omp parallel num_threads(threads > 0 ? threads : 1)
  {
    Visited vis;
#pragma omp for schedule(dynamic, 16)
    for (int i = 0; i < nq; ++i) {
      Counters c;
      found[i] = search_one(ix, q + (size_t)i * ix.D, k, ef, vis, &c, ids + (size_t)i * k, dists + (size_t)i * k, convention);
      if (counters) {
        long long* o = counters + (size_t)i * 5;
        o[0] = c.n_dist; o[1] = c.n_hops; o[2] = c.n_dist_upper; o[3] = c.n_sweeps_upper; o[4] = c.max_cand;
      }
    }
  }
}

// per query: 1 if the hnswlib search meets equal distances in its result set, else 0
void orc_search_meets_ties(void* h, const float* q, int nq, int ef, unsigned char* out, int threads) {
  const Index& ix = *static_cast<Index*>(h);
#pragma omp parallel num_threads(threads > 0 ? threads : 1)
  {
    Visited vis;
#pragma omp for schedule(dynamic, 16)
    for (int i = 0; i < nq; ++i) {
      const float* qi = q + (size_t)i * ix.D;
      out[i] = 0;
      if (ix.N == 0) continue;
      uint32_t cur = ix.enterpoint;
      float dcur = canon_dist(qi, ix.vec(cur), ix.D, ix.dist_type);
      for (int level = ix.maxlevel; level > 0; --level) descend_level(ix, qi, level, cur, dcur, nullptr);
      vis.reset(ix.N);
      out[i] = search_meets_ties(ix, qi, cur, dcur, (size_t)ef, vis) ? 1 : 0;
    }
  }
}

// the same for the reverse_cand search (farthest waiting entry first)
void orc_search_far(void* h, const float* q, int nq, int k, int ef, int* ids, float* dists, int* found, long long* counters,
                    int threads, int convention) {
  const Index& ix = *static_cast<Index*>(h);
#pragma omp parallel num_threads(threads > 0 ? threads : 1)
  {
    Visited vis;
#pragma omp for schedule(dynamic, 16)
    for (int i = 0; i < nq; ++i) {
      Counters c;
      found[i] = search_one_far(ix, q + (size_t)i * ix.D, k, ef, vis, &c, ids + (size_t)i * k, dists + (size_t)i * k, convention);
      if (counters) {
        long long* o = counters + (size_t)i * 5;
        o[0] = c.n_dist; o[1] = c.n_hops; o[2] = c.n_dist_upper; o[3] = c.n_sweeps_upper; o[4] = 0;
      }
    }
  }
}

// greedy descent only: entry node at level 0 for each query (tests of the descent)
void orc_descend(void* h, const float* q, int nq, int* entries) {
  const Index& ix = *static_cast<Index*>(h);
  for (int i = 0; i < nq; ++i) {
    uint32_t cur = ix.enterpoint;
    float dcur = canon_dist(q + (size_t)i * ix.D, ix.vec(cur), ix.D, ix.dist_type);
    for (int level = ix.maxlevel; level > 0; --level) descend_level(ix, q + (size_t)i * ix.D, level, cur, dcur, nullptr);
    entries[i] = (int)cur;
  }
}

// neighbour-selection heuristic on explicit candidates: cand ids / distances to the target -> selected ids (nearest first)
int orc_select(void* h, const unsigned* cand_ids, const float* cand_d, int n, int M, unsigned* out_ids) {
  const Index& ix = *static_cast<Index*>(h);
  MaxQueue top;
  for (int i = 0; i < n; ++i) top.emplace(cand_d[i], cand_ids[i]);
  select_neighbors(ix, top, (size_t)M);
  std::vector<DistId> v;
  while (!top.empty()) { v.push_back(top.top()); top.pop(); }
  std::reverse(v.begin(), v.end());
  for (size_t i = 0; i < v.size(); ++i) out_ids[i] = v[i].second;
  return (int)v.size();
}

// the reference's SearchHeuristic on explicit candidates (ascending keys to the target): fills out_ids /
// out_keys[0..degree) and returns the degree; pair_tests (may be null) receives the number of candidate-pick
// distance evaluations
int orc_select_ref(void* h, const unsigned* cand_ids, const float* cand_d, int n, int max_m, int nn_num, int save_remains,
                   int new_comer, unsigned* out_ids, float* out_keys, long long* pair_tests) {
  const Index& ix = *static_cast<Index*>(h);
  std::vector<DistId> cand(n), row;
  for (int i = 0; i < n; ++i) cand[i] = DistId(cand_d[i], cand_ids[i]);
  long long tests = 0;
  const int deg = select_reference(ix, cand, max_m, nn_num, save_remains != 0, new_comer, row, &tests);
  for (int i = 0; i < deg; ++i) { out_ids[i] = row[i].second; out_keys[i] = row[i].first; }
  if (pair_tests) *pair_tests = tests;
  return deg;
}

// vectors only (no graph): enough for the selection heuristic and for distances by id
int orc_set_vectors(void* h, const float* vectors, int N, int D, int dist_type) {
  Index& ix = *static_cast<Index*>(h);
  ix.N = N; ix.D = D; ix.dist_type = dist_type;
  ix.vectors.assign(vectors, vectors + (size_t)N * D);
  ix.levels.assign(N, 0);
  ix.labels.resize(N);
  for (int i = 0; i < N; ++i) ix.labels[i] = (uint64_t)i;
  ix.alloc_links();
  return 1;
}

// exact top-k by brute force under the canonical distance; ascending by (distance, id)
void orc_bruteforce(const float* data, int N, int D, const float* q, int nq, int k, int dist_type, int* ids, float* dists,
                    int threads) {
#pragma omp parallel for schedule(dynamic, 4) num_threads(threads > 0 ? threads : 1)
  for (int i = 0; i < nq; ++i) {
    std::priority_queue<std::pair<float, int>> heap;
    const float* qq = q + (size_t)i * D;
    for (int j = 0; j < N; ++j) {
      float d = canon_dist(qq, data + (size_t)j * D, D, dist_type);
      if ((int)heap.size() < k) heap.emplace(d, j);
      else if (std::make_pair(d, j) < heap.top()) { heap.pop(); heap.emplace(d, j); }
    }
    int n = (int)heap.size();
    for (int r = n - 1; r >= 0; --r) { ids[(size_t)i * k + r] = heap.top().second; dists[(size_t)i * k + r] = heap.top().first; heap.pop(); }
    for (int r = n; r < k; ++r) { ids[(size_t)i * k + r] = -1; dists[(size_t)i * k + r] = INFINITY; }
  }
}

// graph validator: returns 0 if every invariant holds, else a bit mask of violations
//  1 id out of range, 2 self loop, 4 duplicate link, 8 degree above cap, 16 link to a node absent from that level
int orc_validate(void* h) {
  const Index& ix = *static_cast<Index*>(h);
  int bad = 0;
  for (int i = 0; i < ix.N; ++i)
    for (int l = 0; l <= ix.levels[i]; ++l) {
      const uint32_t* ll = ix.list(i, l);
      uint32_t cap = l ? ix.max_m : ix.max_m0;
      if (ll[0] > cap) { bad |= 8; continue; }
      for (uint32_t a = 0; a < ll[0]; ++a) {
        uint32_t x = ll[1 + a];
        if (x >= (uint32_t)ix.N) { bad |= 1; continue; }
        if (x == (uint32_t)i) bad |= 2;
        if (ix.levels[x] < l) bad |= 16;
        for (uint32_t b = 0; b < a; ++b) if (ll[1 + b] == x) bad |= 4;
      }
    }
  return bad;
}

// level-0 link keys as a builder stored them (N x max_m0, row i = keys of node i's links in list order) against
// the canonical distance between the two end points: returns the number of links whose stored key differs
// bitwise (the validator's "stored distance == recomputed distance")
long long orc_check_link_keys0(void* h, const float* keys0, int threads) {
  const Index& ix = *static_cast<Index*>(h);
  long long bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad) num_threads(threads > 0 ? threads : 1)
  for (int i = 0; i < ix.N; ++i) {
    const uint32_t* l = ix.list((uint32_t)i, 0);
    for (uint32_t j = 0; j < l[0]; ++j) {
      const float d = canon_dist(ix.vec((uint32_t)i), ix.vec(l[1 + j]), ix.D, ix.dist_type);
      const float got = keys0[(size_t)i * ix.max_m0 + j];
      if (std::memcmp(&d, &got, 4) != 0) ++bad;
    }
  }
  return bad;
}

int orc_max_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // extern "C"
