// The launched kernels: batch search, and the three phases of a build batch.
//
// search_kernel        replaces GetEntryPointsKernel + SearchGraphKernel
//                      (cpp/include/cuda_search_kernels.cuh:11-165 in the reference):
//                      one launch does the descent through every upper level and the
//                      level-0 ef-search for a whole query batch.
// build_search_kernel, apply_kernel, reverse_kernel
//                      replace BuildLevelGraphKernel + SearchHeuristic
//                      (cpp/include/cuda_build_kernels.cuh:68-338) and the per-level host
//                      orchestration (cpp/src/cuhnsw_build.cu:96-208).  The reference builds
//                      level by level, top down, every node of a level concurrently under
//                      per-node spin locks.  Here nodes are inserted in id order, each on all
//                      of its levels at once (hnswlib's order: early nodes leave long-range
//                      links on level 0, which is what keeps strongly clustered sets
//                      navigable), in batches of three lock-free phases separated by kernel
//                      boundaries:
//                        1. every node of the batch descends from the current entry point,
//                           searches each of its levels on the frozen graph and selects its
//                           neighbours there (read-only on the graph),
//                        2. the selections are written and each chosen neighbour y receives
//                           the newcomer in y's inbox of that level,
//                        3. one wavefront per touched (y, level) merges inbox and row (append
//                           while there is room, else the selection heuristic).
//                      The result is deterministic for a given batch schedule.
#pragma once
#include "device_core.h"

namespace cuhnsw_amd {

struct SlotPool {
  uint32_t* bitmaps;
  int bitmap_words;
  uint32_t* undo;
  int undo_cap;
  HeapEnt* cand_glob;
  int cand_glob_cap;
  HeapEnt* log;  // accepted entries of the running search
  int log_cap;
};

struct SearchArgs {
  const float* q;  // nq x D
  int nq, k, ef;
  int* nns;
  float* dists;
  int* found;
  int* stats;    // nq x 4 or null
  int* counter;  // work queue head
  int* status;   // set to 1 when a candidate queue ran out of room
  int* repeats;  // counts the queries that met equal keys in the sorted-set pass
  int* redo;     // their indices, for the literal pass; as input of the literal pass: the queries to answer (null = all)
  int* done;     // queries the sorted-set pass has finished with (answered or given up); done[1] is set to 1
                 // by the first wavefront of that pass to start
  int live;      // literal pass only: 1 = the sorted-set pass is running at the same time and a.redo is
                 // still being filled (entries start at -1); a.nq_total queries will pass through it
  int nq_total;
  int spin_limit;  // >= 0: polls of a live literal wavefront before it leaves with status 2 (tests force the
                   // fall-back with 0); < 0: no bound in polls, the two bounds in time below apply
  long long start_ticks;  // ticks of the device's wall clock a live literal wavefront waits for the first
                          // pass to START (done[1] != 0) before it takes the streams to be serialised
  long long stall_ticks;  // and for which it accepts no progress of the first pass once that has started
  const int* nq_dev;      // literal pass: when set, the number of list entries is read from here on the
                          // device (the count the first pass left) instead of taken from nq
  int slot_base;   // first slot of the pool this launch may use (two literal launches can be in flight)
  SlotPool pool;
  int cand_lds, lcap, hnswlib_dist;
  int vc_bits;  // log2 entries of the LDS visited cache of the literal search, 0 = none
  int fc_bits;  // log2 sets (two tags each) of the LDS visited filter of the sorted-set search, 0 = that search is off
  int fast_path;  // 0 = literal queues only (exact evaluation counters)
  int reverse;    // expand the farthest waiting candidate (reverse_cand); sorted-set pass only
  const uint32_t* deleted;  // one bit per element (hnswlib's delete marks) or null; literal queues in LDS only (NS == 0)
  int lean;       // literal pass: result set = sorted set with ids, visited = LDS filter of 2^lean sets
                  // (no bitmap, evaluation counters include repeats); 0 = exact bitmap
  // Sorted-set pass with its queries taken longest first (entry_kernel and the two order kernels below); all
  // null = queries in the caller's order, each descending from the top level itself.
  uint4* entry;     // per query: level-0 entry point, its key (bits), evaluations and sweeps of the descent
  int* order_hist;  // kOrderBuckets counters, then cursors
  int* order;       // nq query indices, largest entry key first
  // Trails of the sorted-set pass (device_core.h, struct Trail), all null / 0 = none are kept.  Buffer b holds
  // trail_cap records from trail + b * trail_cap on; wavefront w of the sorted-set pass starts on buffer w and,
  // each time it hands over a query whose trail the literal pass is to read, goes on with the next unused one
  // of the trail_spares buffers behind those (trail_next counts them; none left: it keeps no more trails).
  uint4* trail;
  int trail_cap, trail_first_spare, trail_spares;
  int* trail_next;
  int4* redo_trail;  // per entry of a.redo: (buffer or -1, records, expansions covered, evaluations up to there)
};

struct BuildArgs {
  int begin, count;        // batch = nodes begin .. begin+count-1
  const int* order;        // N entries or null: the i-th node a batch hands out is begin + order[begin + i] (the
                           // nodes with upper levels first: they take several searches, and a launch ends when
                           // its last node does)
  int cur_ep, cur_max;     // entry point and top level of the graph before this batch (cur_max < 0: empty)
  int efc, nn_num0, nn_numU, save_remains;
  int reverse;   // expand the farthest waiting candidate (reverse_cand)
  int own_cap0;  // how many links a new node may choose for itself on level 0 (<= max_m0)
  uint32_t* sel0_ids;  // count x max_m0: level-0 selections of the batch
  float* sel0_keys;
  int* sel0_cnt;
  uint32_t* selU_ids;  // upper rows x max_m: upper-level selections, indexed like linksU rows
  float* selU_keys;
  int* selU_cnt;
  int* counter;
  int* status;
  SlotPool pool;
  int cand_lds, lcap;
  int vc_bits, fc_bits;
  HeapEnt* inbox0;  // N x cap_in
  int* inbox0_cnt;  // N
  HeapEnt* inboxU;  // upper rows x cap_in
  int* inboxU_cnt;  // upper rows
  int cap_in;
  unsigned long long* dirty;  // node | level << 32
  int* dirty_cnt;
  int* dropped;  // reverse links that found no room in an inbox (kept: the cap_in closest newcomers)
  // Per link row (N level-0 rows, then the upper rows): 1 = the row as it stands is an output of the selection
  // rule (written by a selection, not appended to since), so that a later re-selection may take the shortcut
  // for newcomers.  The reference keeps the same fact per node and level as went_through_heuristic
  // (cpp/include/cuda_build_kernels.cuh:277,322).  Null = no shortcut.
  unsigned char* selected0;
  unsigned char* selectedU;
  // optional work counters of a build (null = off), level 0 in [0..4], upper levels in [5..9]:
  //   +0 distance evaluations of the searches and descents (one vector row each)
  //   +1 link rows read (expanded candidates, descent sweeps, rows merged with their inbox)
  //   +2 pair tests of the selection heuristic (one vector row each)
  //   +3 candidates the heuristic loaded to test them (one vector row each)
  //   +4 link rows written
  unsigned long long* counters;
};


__host__ __device__ inline size_t align16(size_t x) { return (x + 15) & ~(size_t)15; }

// elements per stored row: D rounded up so that every fp32 row starts on a 128-byte line (32 elements), or —
// `tight` — only to whole 16-byte chunks (4 elements), which shrinks the footprint and gives up the alignment
inline int padded_dims(int D, bool tight = false) { return tight ? (D + 3) / 4 * 4 : (D + 31) / 32 * 32; }
// float4 registers per lane that hold a query of Dp elements spread over 16 lanes (template parameter QR
// of the kernels); 0 = the query does not fit registers and is staged in LDS
inline int query_regs(int Dp) {
  const int chunks16 = ((Dp >> 2) + 15) / 16;
  return chunks16 <= 1 ? 1 : (chunks16 <= 2 ? 2 : (chunks16 <= 4 ? 4 : 0));
}

// LDS layout of one wavefront (shared by host sizing and device carving).  In the build's
// search kernel the visited filter of the sorted-set search (fcache) takes the place of the
// candidate queue and the literal search's visited cache.
struct LdsPlan {
  size_t qlds, top, cand, sorted_id, sorted_key, out_id, out_key, nbuf, dbuf, vcache, fcache, lfilter, total;
};
// fc_bits: filter lying over the queue (build); lf_bits: filter of its own beside the queue (the
// literal search on the sorted set)
__host__ __device__ inline LdsPlan plan_lds(int qr, int Dp, int ef, int cand_lds, int lcap, int n_sorted, int n_out,
                                            int vc_bits = 0, int fc_bits = 0, int lf_bits = 0) {
  LdsPlan p;
  size_t o = 0;
  p.qlds = o;
  if (qr == 0) o += (size_t)query_lds_chunks(Dp) * 16;
  p.top = o; o = align16(o + (size_t)(ef + 1) * 8);
  p.cand = o; o = align16(o + (size_t)cand_lds * 8);
  p.vcache = o; o = align16(o + (vc_bits > 0 ? ((size_t)2 << vc_bits) : 0));
  p.fcache = p.cand;
  const size_t fend = p.fcache + (fc_bits > 0 ? ((size_t)4 << fc_bits) : 0);
  if (fend > o) o = align16(fend);
  p.sorted_id = o; o = align16(o + (size_t)n_sorted * 4);
  p.sorted_key = o; o = align16(o + (size_t)n_sorted * 4);
  p.out_id = o; o = align16(o + (size_t)n_out * 4);
  p.out_key = o; o = align16(o + (size_t)n_out * 4);
  p.nbuf = o; o = align16(o + (size_t)lcap * 4);
  p.dbuf = o; o = align16(o + (size_t)lcap * 4);
  p.lfilter = o; o = align16(o + (lf_bits > 0 ? ((size_t)4 << lf_bits) : 0));
  p.total = o;
  return p;
}

__device__ __forceinline__ void bind_slot(Scratch& s, const SlotPool& pool, int slot) {
  s.bitmap = pool.bitmaps + (size_t)slot * pool.bitmap_words;
  s.bitmap_words = pool.bitmap_words;
  s.undo = pool.undo + (size_t)slot * pool.undo_cap;
  s.undo_cap = pool.undo_cap;
  s.cand_glob = pool.cand_glob + (size_t)slot * pool.cand_glob_cap;
  s.cand_glob_cap = pool.cand_glob_cap;
  s.log = pool.log + (size_t)slot * pool.log_cap;
  s.log_cap = pool.log_cap;
}

// LDS of the sorted-set search: query copy (long rows only), visited filter, row buffers
struct FastLdsPlan {
  size_t qlds, fcache, nbuf, dbuf, total;
};
__host__ __device__ inline FastLdsPlan plan_fast_lds(int qr, int Dp, int lcap, int fc_bits) {
  FastLdsPlan p;
  size_t o = 0;
  p.qlds = o;
  if (qr == 0) o += (size_t)query_lds_chunks(Dp) * 16;
  p.fcache = o; o = align16(o + ((size_t)4 << fc_bits));
  p.nbuf = o; o = align16(o + (size_t)lcap * 4);
  p.dbuf = o; o = align16(o + (size_t)lcap * 4);
  p.total = o;
  return p;
}

// ---- longest queries first -------------------------------------------------------------------------------
// A batch of a few rounds of wavefronts ends when its last query does, and the work of a query has a long
// tail (1.18 M x 50, ef 300: median 300 expansions and 1 190 evaluations, one query in a hundred 440 and
// 2 350, the largest 690 and 4 370).  How far the level-0 entry point is from the query predicts most of it
// (correlation 0.67 with the work; the twenty heaviest of 10 000 queries are all within the fifth with the
// largest entry keys): the level-0 search has to walk that distance, accepting and evicting on its way.  So
// the greedy descent through the upper levels is done for the whole batch first (entry_kernel: what every
// query would do anyway), the queries are put in descending order of their entry key (a counting sort on the
// key's leading bits: order_prefix_kernel, order_scatter_kernel) and the first pass takes them in that order.
// The answers do not depend on the order in which queries are taken.
constexpr int kOrderBits = 14;
constexpr int kOrderBuckets = 1 << kOrderBits;
// bucket 0 holds the largest keys (the float's bits made monotone, leading bits, reversed)
__device__ __forceinline__ int order_bucket(uint32_t key_bits) {
  const uint32_t u = key_bits ^ ((key_bits >> 31) ? 0xFFFFFFFFu : 0x80000000u);
  return (kOrderBuckets - 1) - (int)(u >> (32 - kOrderBits));
}
template <int DT, int QR>
__global__ void __launch_bounds__(64) entry_kernel(DevIndex ix, SearchArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  const FastLdsPlan lp = plan_fast_lds(QR, ix.Dp, a.lcap, 0);
  Scratch s;
  s.vcache = nullptr;
  s.vc_bits = 0;
  s.qlds = reinterpret_cast<float4*>(smem + lp.qlds);
  s.nbuf = reinterpret_cast<uint32_t*>(smem + lp.nbuf);
  s.dbuf = reinterpret_cast<float*>(smem + lp.dbuf);
  for (int qi = blockIdx.x; qi < a.nq; qi += gridDim.x) {
    QVec<QR> qv;
    load_query<QR>(qv, s.qlds, a.q + (size_t)qi * ix.D, ix.D, ix.Dp, lane);
    SearchState st;
    st.n_dist_upper = 0; st.n_sweeps = 0;
    uint32_t cur = ix.enterpoint;
    float dcur = dist_single<DT, QR>(ix, qv, cur, s, lane);
    descend<DT, QR>(ix, qv, ix.maxlevel, 0, cur, dcur, s, st, lane);
    if (lane == 0) {
      const uint32_t bits = __float_as_uint(dcur);
      a.entry[qi] = make_uint4(cur, bits, (uint32_t)st.n_dist_upper, (uint32_t)st.n_sweeps);
      atomicAdd(a.order_hist + order_bucket(bits), 1);
    }
    wave_sync();
  }
}
// The same descents, FOUR queries per wavefront, one per group of 16 lanes (rows of up to 128 elements: the
// query in one or two float4 registers per lane).  A descent is a chain of dependent fetches with a dozen
// evaluations each; on its own in a kernel it is bound by their latency, and a group of 16 lanes is what one
// evaluation occupies anyway: the four groups walk their own queries' levels side by side, each evaluating
// the ids of its current link row one after the other (eight or sixteen rows in flight per lane), with the same
// arithmetic, the same strict first minimum and the same counters as `descend`.
template <int DT, int QR, bool HALF>
__device__ __forceinline__ float entry4_key(const void* rows, uint32_t rowlen, uint32_t used, const QVec<QR>& qv,
                                            uint32_t id, int sub) {
  constexpr int R = QR > 0 ? QR : 1;
  const uint64_t first = (uint64_t)id * rowlen;
  float ax = 0.f, ay = 0.f, az = 0.f, aw = 0.f;
#pragma unroll
  for (int k = 0; k < R; ++k) {
    const uint32_t c = sub + 16 * k;
    const uint64_t at = first + (c < used ? c : 0);  // (as in dist_pass: one unconditional load, padding replaced)
    const float4 t = HALF ? load_chunk_f16(rows, at) : load_chunk_f32(rows, at);
    const float4 v = (DT == DIST_DOT || k < R / 2 || c < used) ? t : qv.q[k];
    acc4<DT>(qv.q[k], v, ax, ay, az, aw);
  }
  return finish16<DT, false>(ax, ay, az, aw);
}
template <int DT, int QR, bool HALF>
__device__ __forceinline__ void entry4_body(const DevIndex& ix, const SearchArgs& a) {
  const int lane = threadIdx.x, g = lane >> 4, sub = lane & 15;
  const uint32_t rowlen = (uint32_t)ix.Dp >> 2, used = (uint32_t)(ix.D + 3) >> 2;
  const void* rows = ix.vectors;
  for (int q0 = blockIdx.x * 4; q0 < a.nq; q0 += gridDim.x * 4) {
    const int qi = q0 + g;
    const bool have = qi < a.nq;
    QVec<QR> qv;
    load_query<QR>(qv, nullptr, a.q + (size_t)(have ? qi : 0) * ix.D, ix.D, ix.Dp, lane);
    uint32_t cur = ix.enterpoint;
    float dcur = entry4_key<DT, QR, HALF>(rows, rowlen, used, qv, cur, sub);
    int level = ix.maxlevel;
    bool active = have && level > 0;
    int sweeps = 0, evals = 0;
    while (__ballot(active) != 0ull) {
      const uint32_t* row = ix.linksU + (size_t)(ix.upper_off[active ? cur : ix.enterpoint] + (active ? level : 1) - 1) * ix.SU;
      float best = INFINITY;
      uint32_t best_id = cur;
      int n = 0;
      for (int base = 0; base < ix.SU; base += 16) {
        const uint32_t got = row[base + sub < ix.SU ? base + sub : 0];
        const uint32_t id = (active && base + sub < ix.SU) ? got : kEmpty;
        const unsigned long long valid = __ballot(id != kEmpty);
        n += __popc((uint32_t)(valid >> (16 * g)) & 0xFFFFu);
        constexpr int B = QR == 1 ? 16 : 8;  // rows in flight per lane: 16 float4 registers' worth
#pragma unroll
        for (int p0 = 0; p0 < 16; p0 += B) {
          if (((valid >> p0) & (0x0001000100010001ull * ((1u << B) - 1u))) == 0ull) continue;  // no id in these slots
          uint32_t ids[B];
          float keys[B];
#pragma unroll
          for (int j = 0; j < B; ++j) ids[j] = (uint32_t)__shfl((int)id, 16 * g + p0 + j, 64);
#pragma unroll
          for (int j = 0; j < B; ++j)
            keys[j] = entry4_key<DT, QR, HALF>(rows, rowlen, used, qv, ids[j] != kEmpty ? ids[j] : cur, sub);
#pragma unroll
          for (int j = 0; j < B; ++j)
            if (ids[j] != kEmpty && keys[j] < best) {  // strictly closer: the first occurrence of the minimum wins
              best = keys[j];
              best_id = ids[j];
            }
        }
      }
      if (active) {
        sweeps += 1;
        evals += n;
        if (n > 0 && best < dcur) {
          dcur = best;
          cur = best_id;  // and sweep again on this level
        } else {
          level -= 1;
          active = level > 0;
        }
      }
    }
    if (have && sub == 0) {
      const uint32_t bits = __float_as_uint(dcur);
      a.entry[qi] = make_uint4(cur, bits, (uint32_t)evals, (uint32_t)sweeps);
      atomicAdd(a.order_hist + order_bucket(bits), 1);
    }
  }
}
template <int DT, int QR>
__global__ void __launch_bounds__(64) entry4_kernel(DevIndex ix, SearchArgs a) {
  if (uni(ix.half) != 0) entry4_body<DT, QR, true>(ix, a);
  else entry4_body<DT, QR, false>(ix, a);
}
// counters -> first position of every bucket (exclusive prefix sum; one workgroup of 1024)
__global__ void __launch_bounds__(1024) order_prefix_kernel(int* hist) {
  __shared__ int part[1024];
  constexpr int per = kOrderBuckets / 1024;
  const int t = threadIdx.x;
  int local[per];
  int sum = 0;
#pragma unroll
  for (int i = 0; i < per; ++i) {
    local[i] = hist[t * per + i];
    sum += local[i];
  }
  part[t] = sum;
  __syncthreads();
  for (int step = 1; step < 1024; step <<= 1) {
    const int add = t >= step ? part[t - step] : 0;
    __syncthreads();
    part[t] += add;
    __syncthreads();
  }
  int run = part[t] - sum;
#pragma unroll
  for (int i = 0; i < per; ++i) {
    hist[t * per + i] = run;
    run += local[i];
  }
}
__global__ void __launch_bounds__(1024) order_scatter_kernel(const uint4* entry, int nq, int* cursor, int* order) {
  // The keys of a batch fall into a few dozen buckets: a workgroup ranks its 1024 queries in LDS and takes one
  // range per bucket it met from the global cursors (the order inside a bucket is free).
  __shared__ int cnt[kOrderBuckets];
  const int t = threadIdx.x;
  for (int i = t; i < kOrderBuckets; i += 1024) cnt[i] = 0;
  __syncthreads();
  const int qi = blockIdx.x * 1024 + t;
  int bucket = 0, rank = 0;
  if (qi < nq) {
    bucket = order_bucket(entry[qi].y);
    rank = atomicAdd(&cnt[bucket], 1);
  }
  __syncthreads();
  for (int i = t; i < kOrderBuckets; i += 1024) {
    const int c = cnt[i];
    if (c > 0) cnt[i] = atomicAdd(cursor + i, c);
  }
  __syncthreads();
  if (qi < nq) order[cnt[bucket] + rank] = qi;
}

// First pass of a search batch: every query on the sorted set in registers (ef < 64*NS).
// A query in which two equal keys meet is not answered here: its index is appended to
// a.redo (a.repeats counts them) and the literal search_kernel answers it afterwards.
// (with at most five keys per lane and the query in at most two float4 registers the kernel is
// held to 72 registers, seven wavefronts per SIMD, at the price of up to five spilled registers;
// eight wavefronts are no faster; with eight keys per lane it fits 96 registers, five wavefronts
// per SIMD, without spilling; the other shapes would spill heavily)
// TRAILS: the pass leaves trails for the literal pass (a.trail set; 2 to 3 % more instructions: the host launches
// this instance for batches of a round or two of wavefronts, where a query handed over late is a good part of the
// batch's time, and the instance without the trail code otherwise).
template <int DT, int QR, int NS, bool TRAILS>
__global__ void __launch_bounds__(64, (QR >= 1 && QR <= 2) ? (NS <= 5 ? 7 : (NS == 8 ? 5 : 1)) : 1) search_fast_kernel(DevIndex ix, SearchArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  const FastLdsPlan lp = plan_fast_lds(QR, ix.Dp, a.lcap, a.fc_bits);
  Scratch s;
  s.vcache = reinterpret_cast<uint16_t*>(smem + lp.fcache);
  s.vc_bits = a.fc_bits;
  s.qlds = reinterpret_cast<float4*>(smem + lp.qlds);
  s.nbuf = reinterpret_cast<uint32_t*>(smem + lp.nbuf);
  s.dbuf = reinterpret_cast<float*>(smem + lp.dbuf);
  // tells a literal pass waiting beside this one that the two kernels do run at the same time
  if (blockIdx.x == 0 && lane == 0) __hip_atomic_store(a.done + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  int trail_buf = (TRAILS && a.trail) ? (int)blockIdx.x : -1;  // the buffer this wavefront's trails go to

  for (;;) {
    int qi = 0;
    if (lane == 0) {
      qi = atomicAdd(a.counter, 1);
      if (qi < a.nq && a.order) qi = a.order[qi];
    }
    qi = __builtin_amdgcn_readfirstlane(qi);
    if (qi >= a.nq) break;
    Trail tr;
    if (TRAILS && trail_buf >= 0) {
      tr.rec = a.trail + (size_t)trail_buf * a.trail_cap;
      tr.cap = a.trail_cap;
      tr.on = true;
    }
    QVec<QR> qv;
    load_query<QR>(qv, s.qlds, a.q + (size_t)qi * ix.D, ix.D, ix.Dp, lane);
    SearchState st;
    st.top_size = 0; st.cand_size = 0; st.n_acc = 0; st.lower = 0.f; st.maxkey = -INFINITY; st.undo_cnt = 0;
    st.n_dist = 0; st.n_hops = 0; st.n_dist_upper = 0; st.n_sweeps = 0; st.fail = 0;

    uint32_t cur = ix.enterpoint;
    if (a.entry) {  // the descent through the upper levels has been done for the whole batch
      const uint4 en = a.entry[qi];
      cur = (uint32_t)__builtin_amdgcn_readfirstlane((int)en.x);
      st.n_dist_upper = __builtin_amdgcn_readfirstlane((int)en.z);
      st.n_sweeps = __builtin_amdgcn_readfirstlane((int)en.w);
    } else {
      float dcur = dist_single<DT, QR>(ix, qv, cur, s, lane);
      descend<DT, QR>(ix, qv, ix.maxlevel, 0, cur, dcur, s, st, lane);
    }

    Frontier<NS> fr;
    frontier_init<NS>(fr, a.ef, lane);
    filter_reset(s, lane);
    visit_lossy_single(s, cur, lane);
    if (lane == 0) s.nbuf[0] = cur;
    wave_sync();
    // (the flag is made wavefront-uniform explicitly and both outcomes are plain branches)
    const int how =
        __builtin_amdgcn_readfirstlane(search_level_fast<DT, QR, NS, false, TRAILS>(ix, qv, 0, a.ef, s, st, fr, 1, lane, a.reverse != 0, a.k >= a.ef, TRAILS ? &tr : nullptr));
    const int T0 = st.top_size < a.k ? st.top_size : a.k;
    // Equal keys across the cut at k: which of them stays is up to the result heap, which the
    // literal search reproduces.  Equal keys among the k best: the answer lists them by label.
    const bool cut_tie = how == 2 && !a.reverse && frontier_tie_within<NS>(fr, a.ef, T0, st.top_size, lane, T0 - 1);
    const int inner_tie = __builtin_amdgcn_readfirstlane(
        (how == 2 && !a.reverse && frontier_tie_within<NS>(fr, a.ef, T0 - 1, st.top_size, lane)) ? 1 : 0);
    const bool gave_up = how == 1 || cut_tie || (inner_tie && T0 > (1 << a.fc_bits));  // (the filter's LDS is the sort's buffer)
    if (gave_up) {
      // (the trail's records are written by many lanes: all of them out before lane 0 publishes the entry)
      const bool with_trail = TRAILS && a.redo_trail && trail_buf >= 0 && tr.n > 0 && tr.hops > 0;
      // a search that went all the way (only the cut at k is open) and whose trail covers every hop: the literal
      // pass needs no search at all, only the result heap replayed from the trail (hops stored negative)
      const bool whole = how != 1 && tr.hops == st.n_hops;
      if (with_trail) __threadfence();
      int spare = 0;
      if (lane == 0) {
        const int slot = atomicAdd(a.repeats, 1);
        if (a.redo_trail) a.redo_trail[slot] = make_int4(with_trail ? trail_buf : -1, tr.n, whole ? -tr.hops : tr.hops, tr.n_dist);
        __hip_atomic_store(&a.redo[slot], qi, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        if (with_trail) spare = atomicAdd(a.trail_next, 1);
      }
      // (the lanes meet again HERE: threaded through to the loop's end, lane 0's way out of the branch above
      // would make everything the next lines set look lane-dependent to the compiler)
      __builtin_amdgcn_wave_barrier();
      if (with_trail) {
        // that buffer belongs to the literal pass now
        spare = __builtin_amdgcn_readfirstlane(spare);
        trail_buf = spare < a.trail_spares ? a.trail_first_spare + spare : -1;
      }
    } else {
      const int T = __builtin_amdgcn_readfirstlane(st.top_size < a.k ? st.top_size : a.k);
      wave_sync();
      frontier_dump<NS>(fr, a.ef, T, s.nbuf, s.dbuf, lane);
      wave_sync();
      if (inner_tie) order_equal_keys(ix, s.nbuf, s.dbuf, T, reinterpret_cast<uint32_t*>(s.vcache), lane);
      if (!a.hnswlib_dist && T > 0) {
        dist_list<DT, QR, true>(ix, qv, s.qlds, s.nbuf, T, s.dbuf, lane);
        wave_sync();
      }
      for (int r = lane; r < a.k; r += 64) {
        int out_id = -1;
        float out_d = INFINITY;
        if (r < T) {
          const uint32_t id = s.nbuf[r];
          out_id = ix.labels ? (int)ix.labels[id] : (int)id;
          out_d = s.dbuf[r];
        }
        a.nns[(size_t)qi * a.k + r] = out_id;
        a.dists[(size_t)qi * a.k + r] = out_d;
      }
      if (lane == 0) {
        a.found[qi] = T;
        if (a.stats) {
          a.stats[(size_t)qi * 4 + 0] = st.n_dist;
          a.stats[(size_t)qi * 4 + 1] = st.n_hops;
          a.stats[(size_t)qi * 4 + 2] = st.n_dist_upper;
          a.stats[(size_t)qi * 4 + 3] = st.n_sweeps;
        }
      }
    }
    // The count the literal pass watches.  Only a query that was handed over has published something that pass
    // reads (its list entry, its trail): there the count is raised with release order, after them; an answered
    // query's results are the host's to read, after the kernel.
    if (lane == 0) {
      if (gave_up) __hip_atomic_fetch_add(a.done, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_fetch_add(a.done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    wave_sync();
  }
}

// Search with literal hnswlib priority queues: the only pass for ef beyond the sorted set's
// capacity, the second pass (over a.redo) otherwise.
// NS > 0: result keys in registers (ef < 64*NS); NS == 0: literal result heap in LDS.
// (held to 96 registers, five wavefronts per SIMD, where the query fits two float4 registers: a
// batch answered by the literal queues alone runs 7-10 % faster for a dozen spilled registers)
template <int DT, int QR, int NS>
__global__ void __launch_bounds__(64, (QR >= 1 && QR <= 2 && NS > 0 && NS <= 5) ? 5 : 1) search_kernel(DevIndex ix, SearchArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  const bool lean = NS > 0 && a.lean > 0;
  const LdsPlan lp = plan_lds(QR, ix.Dp, NS > 0 ? -1 : a.ef, a.cand_lds, a.lcap, 0, 0, lean ? 0 : a.vc_bits, 0, a.lean);
  Scratch s;
  if (lean) {
    s.vcache = reinterpret_cast<uint16_t*>(smem + lp.lfilter);
    s.vc_bits = a.lean;
  } else {
    s.vcache = a.vc_bits > 0 ? reinterpret_cast<uint16_t*>(smem + lp.vcache) : nullptr;
    s.vc_bits = a.vc_bits;
  }
  s.qlds = reinterpret_cast<float4*>(smem + lp.qlds);
  s.top = reinterpret_cast<HeapEnt*>(smem + lp.top);
  s.cand = reinterpret_cast<HeapEnt*>(smem + lp.cand);
  s.cand_lds = a.cand_lds;
  s.nbuf = reinterpret_cast<uint32_t*>(smem + lp.nbuf);
  s.dbuf = reinterpret_cast<float*>(smem + lp.dbuf);
  s.tree = make_stage_tree(lane);
  bind_slot(s, a.pool, a.slot_base + blockIdx.x);
  // after the search the candidate queue is dead: its LDS share (>= ef + 1 entries) then
  // holds the collected results, or the literal heap when a tie has to be replayed
  if (NS > 0) s.top = s.cand;

  for (;;) {
    int qi = 0;
    int entry = 0;  // which entry of the list this is
    if (lane == 0) {
      qi = atomicAdd(a.counter, 1);
      if (a.live) {
        entry = qi;
        // entry qi of the list appears once the sorted-set pass has given up that many
        // queries; it never will if that pass has finished them all and the entry is still
        // empty.  The wait is bounded in wall-clock time: if the first pass has not even started
        // after start_ticks (the two streams are being serialised, as under a counter-collecting
        // profiler), or has made no progress for stall_ticks, the wavefront leaves with status 2
        // and the host answers the rest after the first pass.
        int got = -1;
        if (qi < a.nq_total) {
          const long long t_begin = wall_clock64();
          long long t_progress = t_begin;
          int seen_done = -1;
          // (relaxed agent-scope loads: they read the L2 and, unlike acquire loads, do not
          // invalidate this CU's vector cache on every poll; the list entry is the only thing
          // read from the other pass, and it is read after the count that vouches for it)
          // every waiter polls its own list entry; the shared count is looked at only now and
          // then, and the pauses grow, so that the waiting does not crowd the memory channel
          // of the counters the other pass is working with
          for (int spins = 0;; ++spins) {
            got = __hip_atomic_load(&a.redo[qi], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (got >= 0) break;
            if (a.spin_limit >= 0 && spins >= a.spin_limit) {
              atomicOr(a.status, 2);
              break;
            }
            if ((spins & 3) == 3) {
              const int done_now = __hip_atomic_load(a.done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              if (done_now >= a.nq_total) {
                got = __hip_atomic_load(&a.redo[qi], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
              }
              const long long now = wall_clock64();
              if (done_now != seen_done) {
                seen_done = done_now;
                t_progress = now;
              }
              const bool started = __hip_atomic_load(a.done + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
              if (started ? (now - t_progress > a.stall_ticks) : (now - t_begin > a.start_ticks)) {
                atomicOr(a.status, 2);
                break;
              }
            }
            if (spins < 16) {
              __builtin_amdgcn_s_sleep(32);
            } else {
              __builtin_amdgcn_s_sleep(127);
              __builtin_amdgcn_s_sleep(127);
              __builtin_amdgcn_s_sleep(127);
            }
          }
        }
        qi = got;
      } else if (qi >= (a.nq_dev ? *a.nq_dev : a.nq)) {
        qi = -1;
      } else if (a.redo) {
        entry = qi;
        qi = a.redo[qi];  // second pass: only the queries the sorted-set pass gave up
      }
    }
    qi = __builtin_amdgcn_readfirstlane(qi);
    if (qi < 0) break;
    // the trail the sorted-set pass left for this query, if any (its records were written by another
    // wavefront before the list entry was: read them from memory, not from this CU's cache)
    int4 tmeta = make_int4(-1, 0, 0, 0);
    if (lean && a.redo_trail) {
      entry = __builtin_amdgcn_readfirstlane(entry);
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      const int4 m = a.redo_trail[entry];
      tmeta = make_int4(__builtin_amdgcn_readfirstlane(m.x), __builtin_amdgcn_readfirstlane(m.y),
                        __builtin_amdgcn_readfirstlane(m.z), __builtin_amdgcn_readfirstlane(m.w));
    }
    // beside the first pass a literal wavefront is one among a few dozen on its CU and its query
    // is on the batch's critical path: it goes first whenever it has an instruction ready
    if (a.live) __builtin_amdgcn_s_setprio(3);
    QVec<QR> qv;
    load_query<QR>(qv, s.qlds, a.q + (size_t)qi * ix.D, ix.D, ix.Dp, lane);
    SearchState st;
    st.top_size = 0; st.cand_size = 0; st.n_acc = 0; st.lower = 0.f; st.maxkey = -INFINITY; st.undo_cnt = 0;
    st.n_dist = 0; st.n_hops = 0; st.n_dist_upper = 0; st.n_sweeps = 0; st.fail = 0;
    TopKeys<NS> tk;
    topkeys_init<NS>(tk, a.ef, lane);

    uint32_t cur = ix.enterpoint;
    float dcur;
    if (a.entry) {  // the descent through the upper levels has been done for the whole batch
      const uint4 en = a.entry[qi];
      cur = (uint32_t)__builtin_amdgcn_readfirstlane((int)en.x);
      dcur = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane((int)en.y));
      st.n_dist_upper = __builtin_amdgcn_readfirstlane((int)en.z);
      st.n_sweeps = __builtin_amdgcn_readfirstlane((int)en.w);
    } else {
      dcur = dist_single<DT, QR>(ix, qv, cur, s, lane);
      descend<DT, QR>(ix, qv, ix.maxlevel, 0, cur, dcur, s, st, lane);
    }

    int T;
    bool literal = NS == 0;
    bool have_result = false;  // s.nbuf / s.dbuf already hold the T answers in order
    if (lean) {
      Frontier<NS> fr;
      frontier_init<NS>(fr, a.ef, lane);
      filter_reset(s, lane);
      visit_lossy_single(s, cur, lane);
      if (lane == 0) s.nbuf[0] = cur;
      wave_sync();
      bool ambiguous = false;
      // A trail that covers a whole search (the first pass went all the way: only the cut at k is open) IS
      // hnswlib's sequence of accepted entries wherever it sets no stretch apart.  From its last marker on
      // nothing but the result heap needs replaying: the search below stops there (with no marker at all it
      // is not even started), and the heap is fed from the log of what the search accepted so far and then
      // from the rest of the trail — no queue, no set, no rows.
      const uint4* trail = tmeta.x >= 0 ? a.trail + (size_t)tmeta.x * a.trail_cap : nullptr;
      const bool whole = trail != nullptr && tmeta.z < 0;
      const int trail_hops = tmeta.z < 0 ? -tmeta.z : tmeta.z;
      int last_marker = -1;
      if (whole) {
        for (int base = 0; base < tmeta.y; base += 64) {
          const int i = base + lane;
          const unsigned long long m = __ballot(i < tmeta.y && trail[i < tmeta.y ? i : 0].x >= kTrailBack);
          if (m != 0ull) last_marker = base + 63 - __builtin_clzll(m);
        }
      }
      int rest_from = (whole && last_marker < 0) ? 0 : -1;  // >= 0: the trail's records from here on are the rest of the accepted sequence
      if (rest_from < 0)
        search_level_lean<DT, QR, NS>(ix, qv, a.ef, s, st, fr, 1, lane, &ambiguous, trail, tmeta.y,
                                      trail != nullptr ? trail_hops : 0, tmeta.w, whole ? last_marker : -1, &rest_from);
      if (rest_from >= 0 && !st.fail) {
        __threadfence_block();
        LdsHeap top{s.top};
        int size = 0;
        if (st.n_acc == 0) {  // (no search was made: the entry point is the first accepted entry)
          HeapEnt seed;
          seed.key = dcur;
          seed.id = cur;
          coop_push<false>(top, size, seed, lane);
        }
        for (int i = 0; i < st.n_acc; ++i) {
          const HeapEnt e = uniform_ent(s.log[i]);
          coop_push<false>(top, size, e, lane);
          if (size > a.ef) coop_pop<false>(top, size, s.tree, lane);
        }
        for (int base = rest_from; base < tmeta.y; base += 64) {
          const int cnt = tmeta.y - base < 64 ? tmeta.y - base : 64;
          const uint4 r = trail[base + (lane < cnt ? lane : 0)];   // 64 records per fetch, handed out lane by lane
          for (int j = 0; j < cnt; ++j) {
            HeapEnt e;
            e.key = __builtin_bit_cast(float, __builtin_amdgcn_readlane((int)r.z, j));
            e.id = (uint32_t)__builtin_amdgcn_readlane((int)r.y, j);
            coop_push<false>(top, size, e, lane);
            if (size > a.ef) coop_pop<false>(top, size, s.tree, lane);
          }
        }
        st.top_size = size;
        st.n_hops = trail_hops;
        if (st.n_acc == 0) st.n_dist = tmeta.w;
        literal = true;
        T = 0;  // (set below, once the heap is down to k entries)
      } else {
      T = st.top_size < a.k ? st.top_size : a.k;
      // The first T entries of the set (equal keys among them in label order) are hnswlib's
      // answer unless equal keys sit across the cut, or the whole set is returned after an
      // eviction had twins to choose from; then the result heap is replayed from the log, as below.
      const bool inner_tie = !st.fail && frontier_tie_within<NS>(fr, a.ef, T - 1, st.top_size, lane);
      const bool replay = !st.fail && (frontier_tie_within<NS>(fr, a.ef, T, st.top_size, lane, T - 1) ||
                                       (ambiguous && T == st.top_size) || (inner_tie && T > (1 << a.lean)));
      if (!st.fail && !replay) {
        wave_sync();
        frontier_dump<NS>(fr, a.ef, T, s.nbuf, s.dbuf, lane);
        wave_sync();
        if (inner_tie) order_equal_keys(ix, s.nbuf, s.dbuf, T, reinterpret_cast<uint32_t*>(s.vcache), lane);
        have_result = true;
      } else if (replay) {
        __threadfence_block();
        literal = true;
        LdsHeap top{s.top};
        int size = 0;
        for (int i = 0; i < st.n_acc; ++i) {
          const HeapEnt e = uniform_ent(s.log[i]);
          coop_push<false>(top, size, e, lane);
          if (size > a.ef) coop_pop<false>(top, size, s.tree, lane);
        }
        st.top_size = size;
      }
      }
    } else if (NS == 0 && a.reverse) {
      // reverse_cand beyond the register set's capacity: a sorted list in LDS; the answer is its first k entries
      vcache_reset(s, lane);
      visit_single(s, st, cur, lane);
      if (lane == 0) s.nbuf[0] = cur;
      wave_sync();
      search_level_far_lds<DT, QR>(ix, qv, 0, a.ef, s, st, 1, lane);
      literal = false;
      T = st.top_size < a.k ? st.top_size : a.k;
      wave_sync();
      for (int e = lane; e < T; e += 64) {  // (the list has its own LDS: NS == 0)
        s.nbuf[e] = s.top[e].id & ~kExpanded;
        s.dbuf[e] = s.top[e].key;
      }
      have_result = true;
    } else {
    vcache_reset(s, lane);
    visit_single(s, st, cur, lane);
    if (lane == 0) s.nbuf[0] = cur;
    wave_sync();
    search_level<DT, QR, NS, false>(ix, qv, 0, a.ef, s, st, tk, 1, lane, NS == 0 ? a.deleted : nullptr);

    // the k best.  With the keys in registers: the entries of the log at or below the k-th
    // key are the answer unless equal keys straddle the cut; then (and for NS == 0) the
    // literal heap decides: replay every accepted entry through it, pop down to k.
    T = st.top_size < a.k ? st.top_size : a.k;
    if (NS > 0 && !st.fail) {
      __threadfence_block();
      const float bound = topkeys_at<NS>(tk, T - 1, a.ef, reinterpret_cast<float*>(s.cand), lane);
      const int cnt = collect_le(s.log, st.n_acc, bound, s.top, a.lcap, lane);
      if (cnt != T) {
        literal = true;
        LdsHeap top{s.top};
        int size = 0;
        for (int i = 0; i < st.n_acc; ++i) {
          const HeapEnt e = uniform_ent(s.log[i]);
          coop_push<false>(top, size, e, lane);
          if (size > a.ef) coop_pop<false>(top, size, s.tree, lane);
        }
        st.top_size = size;
      }
    }
    }
    if (literal) {
      LdsHeap top{s.top};
      while (st.top_size > a.k) coop_pop<false>(top, st.top_size, s.tree, lane);
      T = st.top_size;
    }
    wave_sync();
    if (!have_result) {
      uint64_t* tie = nullptr;
      if (ix.labels) {
        // labels of the T survivors; with the keys in registers s.top aliases the queue's share,
        // whose first lcap entries hold the survivors themselves
        tie = reinterpret_cast<uint64_t*>(s.cand + (NS > 0 ? a.lcap : 0));
        for (int e = lane; e < T; e += 64) tie[e] = ix.labels[s.top[e].id];
        wave_sync();
      }
      rank_sort(s.top, tie, T, s.nbuf, s.dbuf, lane);
      wave_sync();
    }
    if (!a.hnswlib_dist && T > 0) {
      dist_list<DT, QR, true>(ix, qv, s.qlds, s.nbuf, T, s.dbuf, lane);
      wave_sync();
    }
    for (int r = lane; r < a.k; r += 64) {
      int out_id = -1;
      float out_d = INFINITY;
      if (r < T) {
        uint32_t id = s.nbuf[r];
        out_id = ix.labels ? (int)ix.labels[id] : (int)id;
        out_d = s.dbuf[r];
      }
      a.nns[(size_t)qi * a.k + r] = out_id;
      a.dists[(size_t)qi * a.k + r] = out_d;
    }
    if (lane == 0) {
      a.found[qi] = st.fail ? -1 : T;
      if (st.fail) atomicOr(a.status, 1);
      if (a.stats) {
        a.stats[(size_t)qi * 4 + 0] = st.n_dist;
        a.stats[(size_t)qi * 4 + 1] = st.n_hops;
        a.stats[(size_t)qi * 4 + 2] = st.n_dist_upper;
        a.stats[(size_t)qi * 4 + 3] = st.n_sweeps;
      }
    }
    if (!lean) undo_visited(s, st, lane);
    wave_sync();
    if (a.live) __builtin_amdgcn_s_setprio(0);  // waiting for the next query is nobody's critical path
  }
}

// loads the (zero padded, 128-byte aligned) vector of a stored node as the "query"
template <int QR, bool HALF>
__device__ __forceinline__ void load_node_query_t(QVec<QR>& qv, float4* qlds, const DevIndex& ix, uint32_t node, int lane) {
  const int rowlen = ix.Dp >> 2;
  const int used = (ix.D + 3) >> 2;  // chunks that hold data (the last one zero padded)
  const uint64_t first = (uint64_t)node * (uint32_t)rowlen;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  if (QR > 0) {
    const int sub = lane & 15;
#pragma unroll
    for (int k = 0; k < (QR > 0 ? QR : 1); ++k) {
      const int c = sub + 16 * k;
      const uint64_t at = first + (c < used ? c : 0);  // unconditional load
      const float4 t = HALF ? load_chunk_f16(ix.vectors, at) : load_chunk_f32(ix.vectors, at);
      qv.q[k] = c < used ? t : zero;
    }
  } else {
    const int chunks = query_lds_chunks(ix.Dp);
    wave_sync();
    for (int c = lane; c < chunks; c += 64) {
      const uint64_t at = first + (c < used ? c : 0);
      const float4 t = HALF ? load_chunk_f16(ix.vectors, at) : load_chunk_f32(ix.vectors, at);
      qlds[c] = c < used ? t : zero;
    }
    wave_sync();
  }
}
template <int QR>
__device__ __forceinline__ void load_node_query(QVec<QR>& qv, float4* qlds, const DevIndex& ix, uint32_t node, int lane) {
  if (uni(ix.half) != 0) load_node_query_t<QR, true>(qv, qlds, ix, node, lane);
  else load_node_query_t<QR, false>(qv, qlds, ix, node, lane);
}

// Neighbour selection (HNSW Alg. 4 / hnswlib getNeighborsByHeuristic2) with the two
// extras of the reference's SearchHeuristic (cpp/include/cuda_build_kernels.cuh:68-162):
// the first nn_num candidates pass unconditionally, and with save_remains pruned
// candidates fill the row from the tail.  Candidates sid/skey[0..T) are ascending.
// Returns the degree; oid/okey[0..degree) is the new row.
//
// new_from > 0 is the reference's new_comer shortcut (cuda_build_kernels.cuh:109-110,122-125,137-138) in the
// form that is exact for any number of newcomers: the candidates with an id below new_from are a row that
// this very rule produced before (each of them was tested against every pick before it and passed), the
// others are newcomers.  A newcomer is tested against every pick before it, as always; an old candidate only
// against the NEWCOMERS picked before it — the old picks before it are a subset of those it has passed
// already.  Same row as the full rule, at a fraction of its pair tests.  (Only with nn_num = 0 and without
// save_remains: free picks and tail fill make a row that the rule's own tests do not vouch for.)
template <int DT, int QR>
__device__ __forceinline__ int select_neighbors(const DevIndex& ix, const uint32_t* sid, const float* skey, int T, int m,
                                                int nn_num, int save_remains, uint32_t* oid, float* okey, Scratch& s,
                                                int lane, unsigned int* work = nullptr, uint32_t new_from = 0u) {
  int head = 0;
  int tail = (m < T ? m : T) - 1;
  const int max_head = tail + 1;
  uint32_t* picked_new = s.nbuf;  // ids of the newcomers picked so far (new_from > 0 only)
  int n_new = 0;
  // candidates are examined in list order whatever the outcome, so the next candidate's
  // vector can be fetched while the current one is being tested (register copy; for long
  // rows the LDS copy is filled when the candidate comes up)
  QVec<QR> cv_next;
  if (QR > 0 && T > 0) load_node_query<QR>(cv_next, s.qlds, ix, sid[0], lane);
  for (int j = 0; j < T; ++j) {
    if (head >= m) break;
    const uint32_t c = sid[j];
    const float dq = skey[j];
    bool skip = false;
    QVec<QR> cv = cv_next;
    if (QR > 0 && j + 1 < T) load_node_query<QR>(cv_next, s.qlds, ix, sid[j + 1], lane);
    const bool newcomer = c >= new_from;  // (new_from = 0: every candidate gets the full test)
    const uint32_t* against = newcomer ? oid : picked_new;
    const int n_against = newcomer ? head : n_new;
    if (head >= nn_num && n_against > 0) {
      if (QR == 0) load_node_query<QR>(cv, s.qlds, ix, c, lane);
      if (work && lane == 0) {  // (LDS: +2 pair tests, +3 candidate rows of this level's counters)
        work[2] += (unsigned int)n_against;
        work[3] += 1u;
      }
      dist_list<DT, QR, false>(ix, cv, s.qlds, against, n_against, s.dbuf, lane);
      wave_sync();
      bool mine = false;
      for (int t = lane; t < n_against; t += 64) mine = mine || (dq > s.dbuf[t]);
      skip = __ballot(mine) != 0ull;
      wave_sync();
    }
    if (!skip) {
      if (lane == 0) {
        oid[head] = c;
        okey[head] = dq;
        if (new_from > 0u && newcomer) picked_new[n_new] = c;
      }
      head++;
      if (new_from > 0u && newcomer) n_new++;
    } else if (tail >= head) {
      if (lane == 0) { oid[tail] = c; okey[tail] = dq; }
      tail--;
    }
    wave_sync();
  }
  return save_remains ? max_head : head;
}

// Phase 1 of a build batch: search + select, read-only on the graph.
// (held to six / five wavefronts per SIMD where the query fits one / two float4 registers: a few
// spilled registers, 3-4 % off the build time of the 1.18 M x 50 and 10 M x 96 sets)
template <int DT, int QR, int NS>
__global__ void __launch_bounds__(64, (NS <= 5 && QR == 1) ? 6 : ((NS <= 5 && QR == 2) ? 5 : 1)) build_search_kernel(DevIndex ix, BuildArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  const int m_max = ix.max_m0 > ix.max_m ? ix.max_m0 : ix.max_m;
  const bool sorted_set = NS > 0 && a.fc_bits > 0;
  const LdsPlan lp = plan_lds(QR, ix.Dp, sorted_set ? -1 : a.efc, a.cand_lds, a.lcap, a.efc, m_max, a.vc_bits, a.fc_bits);
  Scratch s;
  s.vcache = sorted_set ? reinterpret_cast<uint16_t*>(smem + lp.fcache)
                        : (a.vc_bits > 0 ? reinterpret_cast<uint16_t*>(smem + lp.vcache) : nullptr);
  s.vc_bits = sorted_set ? a.fc_bits : a.vc_bits;
  s.qlds = reinterpret_cast<float4*>(smem + lp.qlds);
  s.top = reinterpret_cast<HeapEnt*>(smem + lp.top);
  s.cand = reinterpret_cast<HeapEnt*>(smem + lp.cand);
  s.cand_lds = a.cand_lds;
  s.nbuf = reinterpret_cast<uint32_t*>(smem + lp.nbuf);
  s.dbuf = reinterpret_cast<float*>(smem + lp.dbuf);
  uint32_t* sid = reinterpret_cast<uint32_t*>(smem + lp.sorted_id);
  float* skey = reinterpret_cast<float*>(smem + lp.sorted_key);
  uint32_t* oid = reinterpret_cast<uint32_t*>(smem + lp.out_id);
  float* okey = reinterpret_cast<float*>(smem + lp.out_key);
  s.tree = make_stage_tree(lane);
  bind_slot(s, a.pool, blockIdx.x);
  // this wavefront's share of a.counters (LDS, so that counting costs the kernel no registers when it is off)
  __shared__ unsigned int work[16];
  if (lane < 16) work[lane] = 0u;
  wave_sync();

  for (;;) {
    int b = 0;
    if (lane == 0) {
      b = atomicAdd(a.counter, 1);
      if (b < a.count && a.order) b = a.order[a.begin + b];
    }
    b = __builtin_amdgcn_readfirstlane(b);
    if (b >= a.count) break;
    const uint32_t x = (uint32_t)(a.begin + b);
    const int lx = ix.levels[x];
    const int top_level = lx < a.cur_max ? lx : a.cur_max;  // levels x shares with the graph so far
    if (lane == 0) a.sel0_cnt[b] = 0;
    // (the very first node has nothing to link to; a plain branch, not a `continue` after the
    // one-lane store above, keeps the control flow simple for the compiler)
    if (top_level >= 0) {
      QVec<QR> qv;
      load_node_query<QR>(qv, s.qlds, ix, x, lane);
      SearchState st;
      st.undo_cnt = 0; st.n_dist = 0; st.n_hops = 0; st.n_dist_upper = 0; st.n_sweeps = 0; st.fail = 0;

      // hnswlib addPoint: greedy descent from the entry point down to the node's top level,
      // then search + select on every level it has, entering each level at the closest
      // neighbour chosen one level up
      uint32_t cur = (uint32_t)a.cur_ep;
      if (a.cur_max > lx) {
        float dcur = dist_single<DT, QR>(ix, qv, cur, s, lane);
        descend<DT, QR>(ix, qv, a.cur_max, lx, cur, dcur, s, st, lane);
      }
      for (int level = top_level; level >= 0; --level) {
        const int m_cap = level == 0 ? ix.max_m0 : ix.max_m;
        st.top_size = 0; st.cand_size = 0; st.n_acc = 0; st.lower = 0.f; st.maxkey = -INFINITY;
        const int evals_before = st.n_dist, hops_before = st.n_hops;
        int T;
        if (sorted_set) {
          filter_reset(s, lane);
          // sorted set in registers: the efc best come out in order (equal keys in the order
          // the set placed them, which is deterministic).  The new node itself cannot turn up:
          // nothing links to it before the batch's later phases.
          visit_lossy_single(s, cur, lane);
          if (lane == 0) s.nbuf[0] = cur;
          wave_sync();
          Frontier<NS> fr;
          frontier_init<NS>(fr, a.efc, lane);
          search_level_fast<DT, QR, NS, true>(ix, qv, level, a.efc, s, st, fr, 1, lane, a.reverse != 0);
          T = st.top_size;
          wave_sync();
          frontier_dump<NS>(fr, a.efc, T, sid, skey, lane);
          wave_sync();
        } else if (NS == 0 && a.reverse) {
          // reverse_cand beyond the register set's capacity: a sorted list in LDS, already in order
          vcache_reset(s, lane);
          visit_single(s, st, x, lane);  // a node never links to itself
          visit_single(s, st, cur, lane);
          if (lane == 0) s.nbuf[0] = cur;
          wave_sync();
          search_level_far_lds<DT, QR>(ix, qv, level, a.efc, s, st, 1, lane);
          T = st.top_size;
          wave_sync();
          for (int e = lane; e < T; e += 64) {
            sid[e] = s.top[e].id & ~kExpanded;
            skey[e] = s.top[e].key;
          }
          wave_sync();
        } else {
          vcache_reset(s, lane);
          visit_single(s, st, x, lane);  // a node never links to itself
          visit_single(s, st, cur, lane);
          if (lane == 0) s.nbuf[0] = cur;
          wave_sync();
          TopKeys<NS> tk;
          topkeys_init<NS>(tk, a.efc, lane);
          search_level<DT, QR, NS, true>(ix, qv, level, a.efc, s, st, tk, 1, lane);
          T = st.top_size;
          if (NS > 0 && T > 0) {
            __threadfence_block();
            const float bound = topkeys_at<NS>(tk, T - 1, a.efc, reinterpret_cast<float*>(s.cand), lane);
            T = collect_best(s.log, st.n_acc, bound, T, s.top, lane);
          }
          wave_sync();
          rank_sort(s.top, nullptr, T, sid, skey, lane);
          wave_sync();
        }
        unsigned int* level_work = a.counters ? work + (level == 0 ? 0 : 5) : nullptr;
        const int deg = select_neighbors<DT, QR>(ix, sid, skey, T, level == 0 ? a.own_cap0 : m_cap,
                                                 level == 0 ? a.nn_num0 : a.nn_numU, a.save_remains, oid, okey, s, lane,
                                                 level_work);
        if (level_work && lane == 0) {
          level_work[0] += (unsigned int)(st.n_dist - evals_before);
          level_work[1] += (unsigned int)(st.n_hops - hops_before);
          level_work[4] += 1u;
        }
        if (QR == 0) load_node_query<QR>(qv, s.qlds, ix, x, lane);  // the LDS query copy was reused by the selection
        uint32_t* out_ids;
        float* out_keys;
        if (level == 0) {
          out_ids = a.sel0_ids + (size_t)b * ix.max_m0;
          out_keys = a.sel0_keys + (size_t)b * ix.max_m0;
          if (lane == 0) a.sel0_cnt[b] = deg;
        } else {
          const size_t r = (size_t)(ix.upper_off[x] + level - 1);
          out_ids = a.selU_ids + r * ix.max_m;
          out_keys = a.selU_keys + r * ix.max_m;
          if (lane == 0) a.selU_cnt[r] = deg;
        }
        for (int j = lane; j < m_cap; j += 64) {
          out_ids[j] = j < deg ? oid[j] : kEmpty;
          out_keys[j] = j < deg ? okey[j] : 0.f;
        }
        if (deg > 0) cur = oid[0];  // closest selected neighbour: entry for the level below
        wave_sync();
        if (!sorted_set) {
          undo_visited(s, st, lane);
          wave_sync();
        }
      }
      if (lane == 0 && st.fail) *a.status = 1;
      if (a.counters && lane == 0) {
        work[5] += (unsigned int)st.n_dist_upper + (a.cur_max > lx ? 1u : 0u);  // the descent and its entry point
        work[6] += (unsigned int)st.n_sweeps;
      }
    }
  }
  wave_sync();
  if (a.counters && lane < 10 && work[lane] != 0u) atomicAdd(a.counters + lane, (unsigned long long)work[lane]);
}

__device__ __forceinline__ uint32_t* link_row_mut(const DevIndex& ix, uint32_t node, int level) {
  return level == 0 ? ix.links0 + (size_t)node * ix.S0 : ix.linksU + (size_t)(ix.upper_off[node] + level - 1) * ix.SU;
}
__device__ __forceinline__ float* dist_row_mut(const DevIndex& ix, uint32_t node, int level) {
  return level == 0 ? ix.dists0 + (size_t)node * ix.S0 : ix.distsU + (size_t)(ix.upper_off[node] + level - 1) * ix.SU;
}

// Phase 2: write the selected rows and post the reverse links.  Thread (b, j) handles slot j
// of node b on each of its levels.
__global__ void __launch_bounds__(256) apply_kernel(DevIndex ix, BuildArgs a) {
  const int m_max = ix.max_m0 > ix.max_m ? ix.max_m0 : ix.max_m;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long long)a.count * m_max) return;
  const int b = (int)(i / m_max), j = (int)(i % m_max);
  const uint32_t x = (uint32_t)(a.begin + b);
  const int lx = ix.levels[x];
  const int top_level = lx < a.cur_max ? lx : a.cur_max;
  for (int level = 0; level <= top_level; ++level) {
    const int m_cap = level == 0 ? ix.max_m0 : ix.max_m;
    if (j >= m_cap) continue;
    const uint32_t* sel_ids;
    const float* sel_keys;
    int deg;
    if (level == 0) {
      sel_ids = a.sel0_ids + (size_t)b * ix.max_m0;
      sel_keys = a.sel0_keys + (size_t)b * ix.max_m0;
      deg = a.sel0_cnt[b];
    } else {
      const size_t r = (size_t)(ix.upper_off[x] + level - 1);
      sel_ids = a.selU_ids + r * ix.max_m;
      sel_keys = a.selU_keys + r * ix.max_m;
      deg = a.selU_cnt[r];
    }
    const uint32_t y = j < deg ? sel_ids[j] : kEmpty;
    const float key = sel_keys[j];
    link_row_mut(ix, x, level)[j] = y;
    dist_row_mut(ix, x, level)[j] = key;
    if (j == 0 && a.selected0) {
      // (with free picks or the tail fill the row holds entries the rule's tests do not vouch for)
      const unsigned char pure = (level == 0 ? a.nn_num0 : a.nn_numU) == 0 && !a.save_remains;
      if (level == 0) a.selected0[x] = pure;
      else a.selectedU[(size_t)(ix.upper_off[x] + level - 1)] = pure;
    }
    if (j < deg) {
      int* cnt;
      HeapEnt* box;
      if (level == 0) {
        cnt = a.inbox0_cnt + y;
        box = a.inbox0 + (size_t)y * a.cap_in;
      } else {
        const size_t ry = (size_t)(ix.upper_off[y] + level - 1);
        cnt = a.inboxU_cnt + ry;
        box = a.inboxU + ry * a.cap_in;
      }
      const int slot = atomicAdd(cnt, 1);
      if (slot < a.cap_in) {
        HeapEnt e;
        e.key = key;
        e.id = x;
        box[slot] = e;
      }
      if (slot == 0) a.dirty[atomicAdd(a.dirty_cnt, 1)] = (unsigned long long)y | ((unsigned long long)level << 32);
    }
  }
}

// More newcomers chose node y on this level than its inbox holds (a hub of a clustered set, late in a
// large batch).  Which of them reached the inbox depends on the order of the atomics, so the inbox is
// not used: the batch's selections are scanned for y and the cap closest newcomers by (key, id) are
// collected into obox (LDS, cap entries) — the same set in every run.  Returns how many newcomers chose
// y in all.  Rare; one wavefront reads the whole batch's selection rows.
__device__ __forceinline__ int gather_overflowed_inbox(const DevIndex& ix, const BuildArgs& a, uint32_t y, int level,
                                                       HeapEnt* obox, int cap, int lane) {
  int size = 0, total = 0;
  for (int base = 0; base < a.count; base += 64) {
    const int b = base + lane;
    bool hit = false;
    float my_key = 0.f;
    uint32_t my_id = kEmpty;
    if (b < a.count) {
      const uint32_t x = (uint32_t)(a.begin + b);
      const int lx = ix.levels[x];
      const int top_level = lx < a.cur_max ? lx : a.cur_max;
      if (level <= top_level) {
        const uint32_t* ids;
        const float* keys;
        int deg;
        if (level == 0) {
          ids = a.sel0_ids + (size_t)b * ix.max_m0;
          keys = a.sel0_keys + (size_t)b * ix.max_m0;
          deg = a.sel0_cnt[b];
        } else {
          const size_t r = (size_t)(ix.upper_off[x] + level - 1);
          ids = a.selU_ids + r * ix.max_m;
          keys = a.selU_keys + r * ix.max_m;
          deg = a.selU_cnt[r];
        }
        for (int j = 0; j < deg; ++j) {
          if (ids[j] == y) {
            hit = true;
            my_key = keys[j];
            my_id = x;
          }
        }
      }
    }
    unsigned long long todo = __ballot(hit);
    total += __popcll(todo);
    while (todo != 0ull) {
      const int j = __builtin_ctzll(todo);
      todo &= todo - 1ull;
      const float key = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_key), j));
      const uint32_t id = (uint32_t)__builtin_amdgcn_readlane((int)my_id, j);
      if (size < cap) {
        if (lane == 0) {
          obox[size].key = key;
          obox[size].id = id;
        }
        size += 1;
      } else {
        // the farthest entry of the list by (key, id) gives way if the newcomer is closer
        const HeapEnt m = obox[lane < cap ? lane : 0];
        const bool in = lane < cap;
        const float far_key = -wave_min(in ? -m.key : INFINITY);
        const bool at_far = in && m.key == far_key;
        uint32_t far_id = at_far ? m.id : 0u;
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1) {
          const uint32_t o = (uint32_t)__shfl_xor((int)far_id, sh, 64);
          far_id = o > far_id ? o : far_id;
        }
        const bool closer = key < far_key || (key == far_key && id < far_id);
        if (closer && at_far && m.id == far_id) {
          obox[lane].key = key;
          obox[lane].id = id;
        }
      }
      wave_sync();
    }
  }
  return total;
}

// Phase 3: one wavefront per (node, level) that received reverse links.
template <int DT, int QR>
__global__ void __launch_bounds__(64) reverse_kernel(DevIndex ix, BuildArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  const int s_max = ix.S0 > ix.SU ? ix.S0 : ix.SU;
  const int m_max = ix.max_m0 > ix.max_m ? ix.max_m0 : ix.max_m;
  const int ncand = s_max + a.cap_in;
  // plan: "top" region holds the merged candidates, sorted_* their ranking
  const LdsPlan lp = plan_lds(QR, ix.Dp, ncand, 0, a.lcap, ncand, m_max > a.cap_in ? m_max : a.cap_in);
  Scratch s;
  s.qlds = reinterpret_cast<float4*>(smem + lp.qlds);
  HeapEnt* cbuf = reinterpret_cast<HeapEnt*>(smem + lp.top);
  s.nbuf = reinterpret_cast<uint32_t*>(smem + lp.nbuf);
  s.dbuf = reinterpret_cast<float*>(smem + lp.dbuf);
  uint32_t* sid = reinterpret_cast<uint32_t*>(smem + lp.sorted_id);
  float* skey = reinterpret_cast<float*>(smem + lp.sorted_key);
  uint32_t* oid = reinterpret_cast<uint32_t*>(smem + lp.out_id);
  float* okey = reinterpret_cast<float*>(smem + lp.out_key);
  const int n_dirty = *a.dirty_cnt;
  __shared__ unsigned int work[16];
  if (lane < 16) work[lane] = 0u;
  wave_sync();

  for (int di = blockIdx.x; di < n_dirty; di += gridDim.x) {
    const unsigned long long entry = a.dirty[di];
    const uint32_t y = (uint32_t)(entry & 0xffffffffull);
    const int level = (int)(entry >> 32);
    const int S = row_stride(ix, level);
    const int m_cap = level == 0 ? ix.max_m0 : ix.max_m;
    int* cnt;
    const HeapEnt* box;
    if (level == 0) {
      cnt = a.inbox0_cnt + y;
      box = a.inbox0 + (size_t)y * a.cap_in;
    } else {
      const size_t ry = (size_t)(ix.upper_off[y] + level - 1);
      cnt = a.inboxU_cnt + ry;
      box = a.inboxU + ry * a.cap_in;
    }
    const int posted = *cnt;
    int nin = posted < a.cap_in ? posted : a.cap_in;
    if (posted > a.cap_in) {
      // (the overflow list takes the LDS of the selection's output rows, which are not in use yet; the
      // host sizes them for cap_in entries)
      HeapEnt* obox = reinterpret_cast<HeapEnt*>(smem + lp.out_id);
      const int total = gather_overflowed_inbox(ix, a, y, level, obox, a.cap_in, lane);
      if (lane == 0) atomicAdd(a.dropped, total - a.cap_in);
      box = obox;
      wave_sync();
    }
    uint32_t* row = link_row_mut(ix, y, level);
    float* drow = dist_row_mut(ix, y, level);
    // existing links
    int n0 = 0;
    for (int base = 0; base < S; base += 64) {
      uint32_t id = (base + lane < S) ? row[base + lane] : kEmpty;
      float key = (base + lane < S) ? drow[base + lane] : 0.f;
      bool valid = id != kEmpty;
      unsigned long long mask = __ballot(valid);
      int pos = n0 + lanes_below(mask);
      if (valid) { cbuf[pos].key = key; cbuf[pos].id = id; }
      n0 += __popcll(mask);
    }
    wave_sync();
    // newcomers that are not linked yet
    int T = n0;
    for (int base = 0; base < nin; base += 64) {
      HeapEnt e;
      e.key = 0.f; e.id = kEmpty;
      bool keep = false;
      if (base + lane < nin) {
        e = box[base + lane];
        keep = true;
        for (int t = 0; t < n0; ++t) keep = keep && (cbuf[t].id != e.id);
      }
      unsigned long long mask = __ballot(keep);
      int pos = T + lanes_below(mask);
      if (keep) cbuf[pos] = e;
      T += __popcll(mask);
    }
    wave_sync();
    const int n_new = T - n0;
    if (n_new > 0) {
      unsigned char* selected = !a.selected0 ? nullptr
                                : (level == 0 ? a.selected0 + y : a.selectedU + (size_t)(ix.upper_off[y] + level - 1));
      if (T <= m_cap) {
        // room for all: append the newcomers, ordered by (key, id)
        rank_sort(cbuf + n0, nullptr, n_new, sid, skey, lane);
        wave_sync();
        for (int t = lane; t < n_new; t += 64) {
          row[n0 + t] = sid[t];
          drow[n0 + t] = skey[t];
        }
        if (selected && lane == 0) *selected = 0;  // no longer what the selection rule alone would leave
      } else {
        rank_sort(cbuf, nullptr, T, sid, skey, lane);
        wave_sync();
        // A row that is an output of the rule is re-selected with the shortcut for newcomers: the nodes of this
        // batch (ids from a.begin on; everything the row held before has a smaller id).
        const int nn_num = level == 0 ? a.nn_num0 : a.nn_numU;
        const bool pure = nn_num == 0 && !a.save_remains;
        const bool shortcut = pure && selected && uni((int)*selected) != 0;
        const int deg = select_neighbors<DT, QR>(ix, sid, skey, T, m_cap, nn_num, a.save_remains, oid, okey, s, lane,
                                                 a.counters ? work + (level == 0 ? 0 : 5) : nullptr,
                                                 shortcut ? (uint32_t)a.begin : 0u);
        for (int j = lane; j < m_cap; j += 64) {
          row[j] = j < deg ? oid[j] : kEmpty;
          drow[j] = j < deg ? okey[j] : 0.f;
        }
        if (selected && lane == 0) *selected = pure ? 1 : 0;
      }
    }
    if (lane == 0) *cnt = 0;
    if (a.counters && lane == 0) {
      unsigned int* level_work = work + (level == 0 ? 0 : 5);
      level_work[1] += 1u;
      level_work[4] += n_new > 0 ? 1u : 0u;
    }
    wave_sync();
  }
  wave_sync();
  if (a.counters && lane < 10 && work[lane] != 0u) atomicAdd(a.counters + lane, (unsigned long long)work[lane]);
}

// Measurement aid: nothing but the search's memory access pattern.  Every 16-lane group fetches pseudo-random
// vector rows of the resident index, U rows per group in flight, each lane one 16-byte chunk per 64 elements,
// exactly as the distance passes do; `dependent` makes each batch of loads wait for the one before, as a hop
// waits for its rows.  Gives the rate at which this GPU's memory system delivers random rows of THIS index.
template <int U>
__global__ void __launch_bounds__(64) gather_probe_kernel(DevIndex ix, int batches, int dependent, float* sink) {
  const int lane = threadIdx.x, g = lane >> 4, sub = lane & 15;
  const uint32_t rowlen = (uint32_t)ix.Dp >> 2, used = ((uint32_t)ix.D + 3u) >> 2;
  const int nk = (int)((used + 15u) >> 4);
  uint32_t x = (uint32_t)(blockIdx.x * 4 + g) * 2654435761u + 12345u;
  float acc = 0.f;
  uint32_t chain = 0u;
  for (int b = 0; b < batches; ++b) {
    for (int k = 0; k < nk; ++k) {
      float4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        uint32_t y = x + (uint32_t)u * 0x9E3779B9u;
        y ^= y >> 15; y *= 0x2C1B3C6Du; y ^= y >> 12; y *= 0x297A2D39u; y ^= y >> 15;
        const uint32_t id = (uint32_t)(((unsigned long long)y * (unsigned long long)ix.N) >> 32) + chain;
        const uint32_t c = sub + 16u * (uint32_t)k;
        const unsigned long long at = (unsigned long long)id * rowlen + (c < used ? c : 0u);
        v[u] = ix.half ? load_chunk_f16(ix.vectors, at) : load_chunk_f32(ix.vectors, at);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) acc += (v[u].x + v[u].y) + (v[u].z + v[u].w);
    }
    x = x * 1664525u + 1013904223u;
    if (dependent) chain = acc == 1234567.0f ? 1u : 0u;  // (never true: the next addresses just have to wait for this sum)
  }
  if (acc == 7654321.0f) sink[blockIdx.x] = acc;
}

// Upload helper for fp16 storage: N x D floats into rows of Dp halves (the padding was zeroed before).
__global__ void __launch_bounds__(256) pad_rows_half_kernel(const float* src, _Float16* dst, long long n, int D, int Dp) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * D) return;
  const long long row = i / D;
  const int col = (int)(i - row * D);
  dst[row * Dp + col] = (_Float16)src[i];  // round to nearest even; the host rounds its copy the same way
}

// Upload helper: copies N x D floats into rows of Dp floats (the padding was zeroed before).
__global__ void __launch_bounds__(256) pad_rows_kernel(const float* src, float* dst, long long n, int D, int Dp) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * D) return;
  const long long row = i / D;
  const int col = (int)(i - row * D);
  dst[row * Dp + col] = src[i];
}

}  // namespace cuhnsw_amd
