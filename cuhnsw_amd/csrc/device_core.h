// Wavefront-level building blocks shared by the search and build kernels (gfx950,
// 64-lane wavefronts, one wavefront per query / inserted node).
//
//   * distances: a 64-lane wavefront works on FOUR rows at a time, 16 lanes per row,
//     each lane loading float4 (dwordx4) chunks of the row, so one load instruction
//     of the wavefront fetches 4 x 256 contiguous bytes.  The 16 lanes are reduced
//     with DPP (quad_perm, row_half_mirror, row_mirror); no LDS, no barrier.
//     Replaces dot / squaresum / GetDistanceByVec of the reference
//     (cpp/include/cuda_dist_kernels.cuh:13-124), which reduce over a 32-thread
//     block through shared memory.
//   * the search runs on ONE sorted set of (key, id, expanded) kept in registers
//     (Frontier, search_level_fast): result set and candidate set of hnswlib at once, which
//     is exact unless the layout of hnswlib's heaps would decide between equal keys; its
//     visited filter is a four-way tag cache in LDS only (visit_lossy).  Replaces the
//     global-memory, thread-0 heap of the reference (cpp/include/cuda_heap_kernels.cuh:13-49),
//     its GetCand / CheckAlreadyExists scans (cpp/include/cuda_utils_kernels.cuh:50-151) and
//     its lossy visited table (cpp/include/cuda_utils_kernels.cuh:185-210).
//   * where equal keys do decide, the search is repeated with hnswlib's two priority queues
//     reproduced move for move: candidate queue in LDS as a libstdc++ heap, each push / pop
//     executed cooperatively by the wavefront (heap_coop.h), result set as sorted keys in
//     registers plus a log (search_level), or as the sorted set with ids (search_level_lean);
//     visited set either an exact bitmap per wavefront in global memory, cleared through an
//     undo list, or the LDS filter.
//
// Canonical fp32 distance arithmetic: element i is accumulated with one fused
// multiply-add into partial sum (i mod 64) in increasing i; the 64 partials are
// combined by a pairwise adjacent tree (s = 1,2 inside a lane, s = 4..32 across the
// 16 lanes).  The key used for ordering is 1 - dot (hnswlib) or the squared L2.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "heap_coop.h"
#include "index_file.h"
#include "options.h"

namespace cuhnsw_amd {

struct DevIndex {
  const void* vectors;       // N x Dp, rows zero padded to Dp (multiple of 32 elements); fp32, or fp16 when half != 0
  const uint64_t* labels;    // N, or null when labels are the internal ids
  uint32_t* links0;          // N x S0
  uint32_t* linksU;          // upper rows x SU
  const int64_t* upper_off;  // N
  const int* levels;         // N
  float* dists0;             // build only: key of every level-0 link
  float* distsU;             // build only
  int N, D, Dp, S0, SU, max_m, max_m0, maxlevel;
  uint32_t enterpoint;
  int half;                  // vectors are stored as fp16 (all arithmetic stays fp32 on the stored values)
};

// per resident wavefront scratch: LDS pointers + this wavefront's global slot
struct Scratch {
  HeapEnt* top;        // LDS, ef + 1 entries
  HeapEnt* cand;       // LDS, cand_lds entries
  HeapEnt* cand_glob;  // global overflow of the candidate queue
  int cand_lds, cand_glob_cap;
  uint32_t* nbuf;      // LDS, lcap ids
  float* dbuf;         // LDS, lcap keys
  float4* qlds;        // LDS copy of the query (only when the query is not kept in registers)
  uint16_t* vcache;    // LDS, direct-mapped cache of ids known to be visited (null = none)
  int vc_bits;         // log2 of its size: slot = id & (size-1), tag = id >> vc_bits
  uint32_t* bitmap;    // global, one bit per node
  uint32_t* undo;      // global, ids whose bit is set
  int undo_cap;
  int bitmap_words;
  HeapEnt* log;        // global, every accepted (key, id) in acceptance order
  int log_cap;
  StageTree tree;      // per-lane constants of the cooperative heap pop
};

struct SearchState {
  int top_size, cand_size;  // top_size: entries of the result set = min(accepted, ef)
  int n_acc;                // accepted so far (= log entries)
  float maxkey;             // largest accepted key
  float lower;
  int undo_cnt;
  int n_dist, n_hops, n_dist_upper, n_sweeps;
  int fail;
};

struct LdsHeap {
  HeapEnt* a;
  __device__ __forceinline__ HeapEnt get(int i) const { return a[i]; }
  __device__ __forceinline__ void set(int i, HeapEnt e) { a[i] = e; }
};
struct SplitHeap {
  HeapEnt* lds;
  HeapEnt* glob;
  int nlds;
  // The global branch waits for its own load at once (s_waitcnt vmcnt(0)).  It is the rare
  // path; without the explicit wait the compiler merges both branches into one flat load
  // and then has to drain ALL outstanding vector-memory traffic (the fire-and-forget log and
  // undo stores too) before unrelated instructions of the hot loop.
  __device__ __forceinline__ HeapEnt get(int i) const {
    if (i < nlds) return lds[i];
    HeapEnt r = glob[i - nlds];
    __builtin_amdgcn_s_waitcnt(0x0F70);
    return r;
  }
  __device__ __forceinline__ void set(int i, HeapEnt e) {
    if (i < nlds) {
      lds[i] = e;
    } else {
      glob[i - nlds] = e;
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
  }
};

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
// sum over each group of 16 consecutive lanes; every lane of the group gets the same bits.
// Must be executed with all 64 lanes active.
__device__ __forceinline__ float reduce16(float x) {
  x = x + dpp_move<0xB1>(x);   // quad_perm [1,0,3,2]
  x = x + dpp_move<0x4E>(x);   // quad_perm [2,3,0,1]
  x = x + dpp_move<0x141>(x);  // row_half_mirror
  x = x + dpp_move<0x140>(x);  // row_mirror
  return x;
}
// Tells the compiler that a value is the same in all lanes (it is then kept in a scalar register
// and branches on it are scalar branches instead of exec-mask juggling).
__device__ __forceinline__ float uni(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}
__device__ __forceinline__ int uni(int x) { return __builtin_amdgcn_readfirstlane(x); }
// how many lanes below this one have their bit set in a wavefront-uniform mask (v_mbcnt: no lane masks in registers)
__device__ __forceinline__ int lanes_below(unsigned long long mask) {
  return (int)__builtin_amdgcn_mbcnt_hi((unsigned int)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned int)mask, 0u));
}
__device__ __forceinline__ float wave_min(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = fminf(x, __shfl_xor(x, m, 64));
  return uni(x);  // (the same in every lane: said so, or all that depends on it counts as lane-dependent)
}

template <int DT>
__device__ __forceinline__ void acc4(const float4 q, const float4 v, float& ax, float& ay, float& az, float& aw) {
  if (DT == DIST_DOT) {
    ax = __builtin_fmaf(q.x, v.x, ax);
    ay = __builtin_fmaf(q.y, v.y, ay);
    az = __builtin_fmaf(q.z, v.z, az);
    aw = __builtin_fmaf(q.w, v.w, aw);
  } else {
    float tx = q.x - v.x, ty = q.y - v.y, tz = q.z - v.z, tw = q.w - v.w;
    ax = __builtin_fmaf(tx, tx, ax);
    ay = __builtin_fmaf(ty, ty, ay);
    az = __builtin_fmaf(tz, tz, az);
    aw = __builtin_fmaf(tw, tw, aw);
  }
}
// One chunk (four consecutive elements) of stored vectors: 16 bytes of fp32, or 8 bytes of fp16
// widened to fp32 (exact).  `chunk` counts chunks from the start of the array.
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load_chunk_f32(const void* base, uint64_t chunk) {
  return reinterpret_cast<const float4*>(base)[chunk];
}
__device__ __forceinline__ float4 load_chunk_f16(const void* base, uint64_t chunk) {
  const half4_t h = reinterpret_cast<const half4_t*>(base)[chunk];
  const floatx4_t f = __builtin_convertvector(h, floatx4_t);
  return make_float4(f.x, f.y, f.z, f.w);
}

// RAW = false: ordering key (1 - dot | squared L2); RAW = true: API value (-dot | squared L2)
template <int DT, bool RAW>
__device__ __forceinline__ float finish16(float ax, float ay, float az, float aw) {
  float s = (ax + ay) + (az + aw);
  s = reduce16(s);
  if (DT == DIST_DOT) return RAW ? -s : 1.0f - s;
  return s;
}

// Query kept in registers: lane `sub` of each 16-lane group holds float4 chunks
// sub, sub+16, ... (QR of them).  QR == 0 selects the LDS copy instead.
template <int QR>
struct QVec {
  float4 q[QR > 0 ? QR : 1];
};

// Long rows (the query is read from LDS): 16 lanes own a row, so a lane fetches every 16th chunk of it,
// kLongB of them per round.  The LDS copy of the query is zero-padded to whole rounds (kLongB * 16 chunks),
// so that a round reads it without guards.
constexpr int kLongB = 8;
__host__ __device__ inline int query_lds_chunks(int Dp) {
  const int chunk_rows = ((Dp >> 2) + 15) / 16;
  return (chunk_rows + kLongB - 1) / kLongB * kLongB * 16;
}

// fills the query holder from a row of D floats (any alignment)
template <int QR>
__device__ __forceinline__ void load_query(QVec<QR>& qv, float4* qlds, const float* src, int D, int Dp, int lane) {
  if (QR > 0) {
    const int sub = lane & 15;
#pragma unroll
    for (int k = 0; k < (QR > 0 ? QR : 1); ++k) {
      int i = 4 * (sub + 16 * k);
      float4 t;
      t.x = i + 0 < D ? src[i + 0] : 0.0f;
      t.y = i + 1 < D ? src[i + 1] : 0.0f;
      t.z = i + 2 < D ? src[i + 2] : 0.0f;
      t.w = i + 3 < D ? src[i + 3] : 0.0f;
      qv.q[k] = t;
    }
  } else {
    const int chunks = query_lds_chunks(Dp);
    for (int c = lane; c < chunks; c += 64) {
      int i = 4 * c;
      float4 t;
      t.x = i + 0 < D ? src[i + 0] : 0.0f;
      t.y = i + 1 < D ? src[i + 1] : 0.0f;
      t.z = i + 2 < D ? src[i + 2] : 0.0f;
      t.w = i + 3 < D ? src[i + 3] : 0.0f;
      qlds[c] = t;
    }
    wave_sync();
  }
}

// one pass over 4*U rows starting at ids[r]: loads first, arithmetic after
template <int DT, int R, int U, bool RAW, bool HALF>
__device__ __forceinline__ void dist_pass(const void* rows, uint32_t rowlen, uint32_t used, const float4* q,
                                          const uint32_t* ids, int r, int n, float* out, int g, int sub) {
  float4 v[U][R];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int idx = r + 4 * u + g;
    const uint32_t id = ids[idx < n ? idx : n - 1];
    const uint64_t first = (uint64_t)id * rowlen;  // one 32x32->64 multiply-add
#pragma unroll
    for (int k = 0; k < R; ++k) {
      // always one unconditional load (a guarded one is split into dword loads); a chunk past
      // the row's data (`used` chunks; the row's stride may be longer) re-reads chunk 0, which costs no
      // further memory line.  The query holds zeros there, which is all a dot product needs (finite
      // data); for L2 the chunk is replaced by the query's own zeros.  The data is longer than
      // 16 * (R / 2) chunks, so only the upper half of k can be past its end.
      const uint32_t c = sub + 16 * k;
      const uint64_t at = first + (c < used ? c : 0);
      const float4 t = HALF ? load_chunk_f16(rows, at) : load_chunk_f32(rows, at);
      v[u][k] = (DT == DIST_DOT || k < R / 2 || c < used) ? t : q[k];
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float ax = 0.f, ay = 0.f, az = 0.f, aw = 0.f;
#pragma unroll
    for (int k = 0; k < R; ++k) acc4<DT>(q[k], v[u][k], ax, ay, az, aw);
    const float key = finish16<DT, RAW>(ax, ay, az, aw);
    const int idx = r + 4 * u + g;
    if (sub == 0 && idx < n) out[idx] = key;
  }
  // (the lanes meet again here, not at the caller's loop end: see trail_mark)
  __builtin_amdgcn_wave_barrier();
}

// long rows: 16 lanes still own one row (the summation order is tied to 16 lanes), so a lane
// has rowlen/16 chunks to fetch; they are issued B at a time for each of U groups of four rows, to keep
// U * B loads per lane in flight; the query chunks come from LDS, one read for all U groups.  Rounds that
// lie wholly inside the rows' data carry no guards; the last one re-reads chunk 0 for chunks past the end
// and multiplies zeros there (the LDS copy of the query is zero-padded to whole rounds).
template <int DT, bool RAW, bool HALF, int U, int B>
__device__ __forceinline__ void dist_long_pass(const void* rows, int rowlen, int used, const float4* qlds, const uint32_t* ids,
                                               int r, int n, float* out, int g, int sub) {
  static_assert(B == kLongB, "the LDS copy of the query is padded to rounds of kLongB chunk rows");
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  const int nk = (used + 15) >> 4;  // chunk rows that hold data
  const int nfull = used >> 4;      // chunk rows that hold nothing else
  uint64_t first[U];
  float ax[U], ay[U], az[U], aw[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int idx = r + 4 * u + g;
    const uint32_t id = ids[idx < n ? idx : n - 1];
    first[u] = (uint64_t)id * (uint32_t)rowlen;
    ax[u] = ay[u] = az[u] = aw[u] = 0.f;
  }
  int k0 = 0;
  for (; k0 + B <= nfull; k0 += B) {
    float4 v[U][B];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const uint64_t at = first[u] + (uint32_t)(sub + 16 * (k0 + b));
        v[u][b] = HALF ? load_chunk_f16(rows, at) : load_chunk_f32(rows, at);
      }
    }
    // (the round's query chunks are read in one go, ahead of the arithmetic: read one by one each would be
    // waited for in turn, which is what a lone wavefront's time goes to)
    float4 qq[B];
#pragma unroll
    for (int b = 0; b < B; ++b) qq[b] = qlds[sub + 16 * (k0 + b)];
#pragma unroll
    for (int b = 0; b < B; ++b) {
#pragma unroll
      for (int u = 0; u < U; ++u) acc4<DT>(qq[b], v[u][b], ax[u], ay[u], az[u], aw[u]);
    }
  }
  if (k0 < nk) {  // (k0 + B > nfull >= nk - 1: one more round reaches the end)
    float4 v[U][B];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int b = 0; b < B; ++b) {
        const int c = sub + 16 * (k0 + b);
        const uint64_t at = first[u] + (uint32_t)(c < used ? c : 0);  // unconditional load (chunk 0 past the end)
        const float4 t = HALF ? load_chunk_f16(rows, at) : load_chunk_f32(rows, at);
        v[u][b] = c < used ? t : zero;
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const float4 qq = qlds[sub + 16 * (k0 + b)];  // zeros past the end
#pragma unroll
      for (int u = 0; u < U; ++u) acc4<DT>(qq, v[u][b], ax[u], ay[u], az[u], aw[u]);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const float key = finish16<DT, RAW>(ax[u], ay[u], az[u], aw[u]);
    const int idx = r + 4 * u + g;
    if (sub == 0 && idx < n) out[idx] = key;
  }
  __builtin_amdgcn_wave_barrier();  // (the lanes meet again here, not at the loop's end: see trail_mark)
}
// U = 2: eight rows at a time while more than four are left (twice the loads in flight, 64 more registers:
// for the search of few queries at a time, where a wavefront waits for its own loads and arithmetic in turn)
template <int DT, bool RAW, bool HALF, int U>
__device__ __forceinline__ void dist_long(const void* rows, int rowlen, int used, const float4* qlds, const uint32_t* ids,
                                          int n, float* out, int g, int sub) {
  int r = 0;
  while (r < n) {
    if (U >= 2 && n - r > 4) {
      dist_long_pass<DT, RAW, HALF, (U >= 2 ? 2 : 1), kLongB>(rows, rowlen, used, qlds, ids, r, n, out, g, sub);
      r += 8;
    } else {
      dist_long_pass<DT, RAW, HALF, 1, kLongB>(rows, rowlen, used, qlds, ids, r, n, out, g, sub);
      r += 4;
    }
  }
}

// keys of ids[0..n) (LDS) against the query -> out[0..n) (LDS).  n is wavefront-uniform.
template <int DT, int QR, bool RAW, bool HALF, int WIDE = 1>
__device__ __forceinline__ void dist_list_t(const DevIndex& ix, const QVec<QR>& qv, const float4* qlds, const uint32_t* ids,
                                            int n, float* out, int lane) {
  const int g = lane >> 4, sub = lane & 15;
  const int rowlen = ix.Dp >> 2;
  const int used = (ix.D + 3) >> 2;  // chunks of a row that hold data
  const void* rows = ix.vectors;
  if (QR > 0) {
    constexpr int R = QR > 0 ? QR : 1;
    constexpr int UMAX = R == 1 ? 4 : (R == 2 ? 2 : 1);  // groups of 4 rows in flight
    int r = 0;
    while (r < n) {
      const int rem = n - r;
      if (UMAX >= 4 && rem > 8) {
        dist_pass<DT, R, (UMAX >= 4 ? 4 : 1), RAW, HALF>(rows, rowlen, used, qv.q, ids, r, n, out, g, sub);
        r += 16;
      } else if (UMAX >= 2 && rem > 4) {
        dist_pass<DT, R, (UMAX >= 2 ? 2 : 1), RAW, HALF>(rows, rowlen, used, qv.q, ids, r, n, out, g, sub);
        r += 8;
      } else {
        dist_pass<DT, R, 1, RAW, HALF>(rows, rowlen, used, qv.q, ids, r, n, out, g, sub);
        r += 4;
      }
    }
  } else {
    dist_long<DT, RAW, HALF, WIDE>(rows, rowlen, used, qlds, ids, n, out, g, sub);
  }
}
// (the element type of the stored vectors is a property of the index: one scalar branch per list)
// WIDE (long rows only): groups of four rows in flight, see dist_long
template <int DT, int QR, bool RAW, int WIDE = 1>
__device__ __forceinline__ void dist_list(const DevIndex& ix, const QVec<QR>& qv, const float4* qlds,
                                          const uint32_t* ids, int n, float* out, int lane) {
  if (uni(ix.half) != 0) dist_list_t<DT, QR, RAW, true, WIDE>(ix, qv, qlds, ids, n, out, lane);
  else dist_list_t<DT, QR, RAW, false, WIDE>(ix, qv, qlds, ids, n, out, lane);
}

__device__ __forceinline__ const uint32_t* link_row(const DevIndex& ix, uint32_t node, int level) {
  return level == 0 ? ix.links0 + (size_t)node * ix.S0 : ix.linksU + (size_t)(ix.upper_off[node] + level - 1) * ix.SU;
}
__device__ __forceinline__ int row_stride(const DevIndex& ix, int level) { return level == 0 ? ix.S0 : ix.SU; }

// The visited bitmap of a slot is touched by one wavefront only; the atomic is there because
// two lanes of that wavefront may hit the same word.  Workgroup scope is therefore enough
// and lets the read-modify-write complete in the XCD's own L2 instead of being pushed out
// to device-coherent memory as an agent-scope atomic (atomicOr) is.
__device__ __forceinline__ uint32_t visited_fetch_or(uint32_t* word, uint32_t bit) {
  return __hip_atomic_fetch_or(word, bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// In front of the bitmap sits a small direct-mapped cache in LDS of ids already known to be
// visited (16-bit tags, slot = low id bits).  Most neighbours of an expanded node were seen
// a few hops earlier; a cache hit answers "visited" exactly (tags are only written for ids
// whose bit is set) and saves the global atomic — on the 1.18M-point benchmark the atomics
// were more than half of all L2 requests and nearly all of the DRAM write traffic.
__device__ __forceinline__ void vcache_reset(Scratch& s, int lane) {
  if (s.vcache == nullptr) return;
  uint4* c4 = reinterpret_cast<uint4*>(s.vcache);
  const int n4 = (1 << s.vc_bits) >> 3;  // 8 tags per 16 bytes
  for (int i = lane; i < n4; i += 64) c4[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
  wave_sync();
}

// marks one id visited (lane 0 does it); returns nothing, logs it for the undo
__device__ __forceinline__ void visit_single(Scratch& s, SearchState& st, uint32_t id, int lane) {
  if (lane == 0) {
    visited_fetch_or(&s.bitmap[id >> 5], 1u << (id & 31));
    if (st.undo_cnt < s.undo_cap) s.undo[st.undo_cnt] = id;
    if (s.vcache != nullptr) s.vcache[id & ((1u << s.vc_bits) - 1u)] = (uint16_t)(id >> s.vc_bits);
  }
  st.undo_cnt += 1;
}

// Reads a link row, marks its ids visited and compacts the ones seen for the first
// time into s.nbuf (stored order kept).  Returns how many.
__device__ __forceinline__ int visit_row(const uint32_t* row, int S, Scratch& s, SearchState& st, int lane) {
  int n = 0;
  for (int base = 0; base < S; base += 64) {
    uint32_t id = (base + lane < S) ? row[base + lane] : kEmpty;
    bool ask = id != kEmpty;
    uint32_t slot = 0;
    uint16_t tag = 0;
    if (s.vcache != nullptr && ask) {
      slot = id & ((1u << s.vc_bits) - 1u);
      tag = (uint16_t)(id >> s.vc_bits);
      ask = s.vcache[slot] != tag;  // hit: visited for sure
    }
    bool newly = false;
    if (ask) {
      uint32_t bit = 1u << (id & 31);
      uint32_t old = visited_fetch_or(&s.bitmap[id >> 5], bit);
      newly = (old & bit) == 0;
      if (s.vcache != nullptr) s.vcache[slot] = tag;
    }
    unsigned long long mask = __ballot(newly);
    int pos = n + lanes_below(mask);
    if (newly) {
      s.nbuf[pos] = id;
      int u = st.undo_cnt + pos;
      if (u < s.undo_cap) s.undo[u] = id;
    }
    n += __popcll(mask);
    wave_sync();
  }
  st.undo_cnt += n;
  return n;
}

// The same for rows of at most 64 slots, split in two so that the vector rows of the
// neighbours can be fetched WHILE the visited atomics are in flight instead of after them:
// visit_issue() starts the atomics for every neighbour the cache does not vouch for and
// compacts those ids into s.nbuf; the caller computes their distances; visit_commit() then
// reads the atomics' answers, blanks the entries that turn out to have been visited before
// (kEmpty in s.nbuf; their distances are discarded) and logs the new ones for the undo.
// The speculative rows are few: after the cache most remaining neighbours are new.
struct VisitPending {
  uint32_t id, bit, old;
  int pos, n_ask;
  bool ask;
};
__device__ __forceinline__ VisitPending visit_issue(const uint32_t* row, int S, Scratch& s, int lane) {
  VisitPending v;
  v.id = lane < S ? row[lane] : kEmpty;
  v.ask = v.id != kEmpty;
  uint32_t slot = 0;
  uint16_t tag = 0;
  if (s.vcache != nullptr && v.ask) {
    slot = v.id & ((1u << s.vc_bits) - 1u);
    tag = (uint16_t)(v.id >> s.vc_bits);
    v.ask = s.vcache[slot] != tag;
  }
  const unsigned long long mask = __ballot(v.ask);
  v.pos = lanes_below(mask);
  v.n_ask = __popcll(mask);
  v.bit = 1u << (v.id & 31);
  v.old = 0u;
  if (v.ask) {
    v.old = visited_fetch_or(&s.bitmap[v.id >> 5], v.bit);
    s.nbuf[v.pos] = v.id;
    if (s.vcache != nullptr) s.vcache[slot] = tag;
  }
  return v;
}
__device__ __forceinline__ int visit_commit(const VisitPending& v, Scratch& s, SearchState& st, int lane) {
  const bool newly = v.ask && (v.old & v.bit) == 0u;
  const unsigned long long mask = __ballot(newly);
  if (v.ask && !newly) s.nbuf[v.pos] = kEmpty;
  if (newly) {
    const int u = st.undo_cnt + lanes_below(mask);
    if (u < s.undo_cap) s.undo[u] = v.id;
  }
  const int n_new = __popcll(mask);
  st.undo_cnt += n_new;
  return n_new;
}

// Reads a link row and compacts its valid ids into s.nbuf without touching the visited set.
__device__ __forceinline__ int load_row(const uint32_t* row, int S, Scratch& s, int lane) {
  int n = 0;
  for (int base = 0; base < S; base += 64) {
    uint32_t id = (base + lane < S) ? row[base + lane] : kEmpty;
    bool valid = id != kEmpty;
    unsigned long long mask = __ballot(valid);
    int pos = n + lanes_below(mask);
    if (valid) s.nbuf[pos] = id;
    n += __popcll(mask);
  }
  return n;
}

// clears the bits this wavefront set; leaves the slot's bitmap all zero
__device__ __forceinline__ void undo_visited(Scratch& s, SearchState& st, int lane) {
  if (st.undo_cnt <= s.undo_cap) {
    for (int i = lane; i < st.undo_cnt; i += 64) s.bitmap[s.undo[i] >> 5] = 0u;
  } else {
    for (int w = lane; w < s.bitmap_words; w += 64) s.bitmap[w] = 0u;
  }
  // (the bitmap belongs to this wavefront alone: its clearing stores only have to be done before its next
  // atomics are issued.  An agent-scope fence here would write the L2 back and invalidate the L1 once per query.)
  __threadfence_block();
  st.undo_cnt = 0;
}

// The result set's KEYS, kept sorted in registers: lane L holds sorted positions
// [L*NS, L*NS + NS).  hnswlib's search uses top_candidates only through its size and its
// largest key (lowerBound), and both depend on the multiset of accepted keys alone, not on
// the heap's layout — so during the search the ids are not needed and the eviction
// "push, then pop the maximum" becomes one sorted insert (about 35 vector instructions, no
// LDS).  Which ids survive is decided at the end from the log of accepted entries; only a
// tie exactly at the k-th key needs the literal heap, which is then replayed from the log.
// Unused positions hold +inf; when the set is full the evicted key falls off the end.
template <int NS>
struct TopKeys {
  float k[NS > 0 ? NS : 1];
};
// The keys are kept right-aligned: sorted position p lives in physical slot p + 64*NS - ef,
// the slots below hold -inf and never move.  The largest key of a FULL set then always sits
// in the last slot of lane 63 — a fixed register, which matters: indexing the register
// array with a run-time position would push it through scratch memory.
template <int NS>
__device__ __forceinline__ void topkeys_init(TopKeys<NS>& t, int ef, int lane) {
  constexpr int N = NS > 0 ? NS : 1;
#pragma unroll
  for (int j = 0; j < N; ++j) t.k[j] = (lane * N + j < 64 * N - ef) ? -INFINITY : INFINITY;
}
template <int NS>
__device__ __forceinline__ void topkeys_insert(TopKeys<NS>& t, float v, int lane) {
  constexpr int N = NS > 0 ? NS : 1;
  int c = 0;  // keys of this lane below v
#pragma unroll
  for (int j = 0; j < N; ++j) c += t.k[j] < v ? 1 : 0;
  // previous lane's count and last key (lane 0: "all below", nothing to take over)
  const int prev_c = __builtin_amdgcn_update_dpp(N, c, 0x138, 0xF, 0xF, false);  // wave_shr:1
  const float prev_last = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, t.k[N - 1]), 0x138, 0xF, 0xF, false));
  const bool shifted = prev_c < N;         // the insertion happened in an earlier lane
  const int pos = shifted ? 0 : c;         // c == N: this lane is untouched
  const float incoming = shifted ? prev_last : v;
#pragma unroll
  for (int j = N - 1; j >= 0; --j) {
    const float below = j > 0 ? t.k[j - 1] : incoming;
    t.k[j] = j > pos ? below : (j == pos ? incoming : t.k[j]);
  }
}
// largest key of a full set
template <int NS>
__device__ __forceinline__ float topkeys_max(const TopKeys<NS>& t) {
  constexpr int N = NS > 0 ? NS : 1;
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, t.k[N - 1]), 63));
}
// key at sorted position pos (wavefront-uniform, once per search): through an LDS copy
template <int NS>
__device__ __forceinline__ float topkeys_at(const TopKeys<NS>& t, int pos, int ef, float* lds_tmp, int lane) {
  constexpr int N = NS > 0 ? NS : 1;
  wave_sync();
#pragma unroll
  for (int j = 0; j < N; ++j) lds_tmp[lane * N + j] = t.k[j];
  wave_sync();
  const float x = lds_tmp[pos + 64 * N - ef];
  wave_sync();
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, x)));
}

// Offers nbuf/dbuf[0..n) in stored order (hnswlib's accept rule, identical to the
// reference's, cpp/include/cuda_utils_kernels.cuh:220-225).  Wavefront-uniform: every lane
// runs it, the heap moves are cooperative.  NS > 0: result keys in registers (TopKeys);
// NS == 0: literal result heap in LDS (s.top), for ef beyond the register capacity.
// deleted (NS == 0 only): one bit per element, hnswlib's delete marks (hnswlib searchBaseLayerST, has_deletions):
// a marked element is queued as a candidate like any other and never enters the result heap; the bound moves
// only while that heap holds something.
template <int NS>
__device__ __forceinline__ void accept_list(Scratch& s, SearchState& st, TopKeys<NS>& tk, int n, int ef, int lane,
                                            const uint32_t* deleted = nullptr) {
  SplitHeap cand{s.cand, s.cand_glob, s.cand_lds};
  const int cand_cap = s.cand_lds + s.cand_glob_cap;
  for (int base = 0; base < n; base += 64) {
    // every lane takes one offer; blanked entries (speculatively fetched neighbours that had
    // been visited before) and offers that already fail against the current bound are
    // dropped at once (the bound never rises once the set is full), the others are taken in
    // stored order and re-checked against the bound as it moves
    const int mine = base + lane;
    const float my_key = mine < n ? s.dbuf[mine] : INFINITY;
    const uint32_t my_id = mine < n ? s.nbuf[mine] : 0u;
    unsigned long long todo = __ballot(mine < n && my_id != kEmpty && (st.top_size < ef || st.lower > my_key));
    unsigned long long marked = 0ull;
    if (NS == 0 && deleted != nullptr)
      marked = __ballot(mine < n && my_id != kEmpty && ((deleted[my_id >> 5] >> (my_id & 31u)) & 1u) != 0u);
    while (todo != 0ull) {
      const int j = __builtin_ctzll(todo);
      todo &= todo - 1ull;
      HeapEnt e;
      e.key = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_key), j));
      e.id = (uint32_t)__builtin_amdgcn_readlane((int)my_id, j);
      // (if/else nesting with one way out of the loops, as in search_level_fast)
      if (st.top_size < ef || st.lower > e.key) {
        if (st.cand_size >= cand_cap || (NS > 0 && st.n_acc >= s.log_cap)) {
          st.fail = 1;
          todo = 0ull;
        } else {
          if (NS > 0 && lane == 0) s.log[st.n_acc] = e;
          st.n_acc += 1;
          // the candidate queue normally fits its LDS share: keep that case on pure LDS
          // instructions (the split accessor compiles to flat loads)
          if (st.cand_size < s.cand_lds) {
            LdsHeap cand_fast{s.cand};
            coop_push<true>(cand_fast, st.cand_size, e, lane);
          } else {
            coop_push<true>(cand, st.cand_size, e, lane);
          }
          if (NS > 0) {
            topkeys_insert<NS>(tk, e.key, lane);
            st.top_size = st.n_acc < ef ? st.n_acc : ef;
            st.maxkey = fmaxf(st.maxkey, e.key);
            st.lower = st.n_acc >= ef ? topkeys_max<NS>(tk) : st.maxkey;  // hnswlib's lowerBound
          } else {
            LdsHeap top{s.top};
            if (((marked >> j) & 1ull) == 0ull) {
              coop_push<false>(top, st.top_size, e, lane);
              if (st.top_size > ef) coop_pop<false>(top, st.top_size, s.tree, lane);
            }
            wave_sync();
            if (st.top_size > 0)
              st.lower = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, s.top[0].key)));
          }
        }
      }
    }
    if (st.fail) base = n;
  }
}

// Best-first search of one level (hnswlib searchBaseLayerST / searchBaseLayer).
// On entry s.nbuf[0..n_seed) holds seed ids that are already marked visited.  On exit
// the accepted entries are in s.log[0..st.n_acc) and tk holds the result keys (NS > 0), or
// s.top[0..st.top_size) is the literal result max-heap (NS == 0).  BUILD selects hnswlib's
// construction-time stop rule; so do delete marks (see accept_list): a result heap short of ef never stops
// the search, marked candidates beyond the bound are walked through.
template <int DT, int QR, int NS, bool BUILD>
__device__ __forceinline__ void search_level(const DevIndex& ix, const QVec<QR>& qv, int level, int ef, Scratch& s,
                                             SearchState& st, TopKeys<NS>& tk, int n_seed, int lane,
                                             const uint32_t* deleted = nullptr) {
  SplitHeap cand{s.cand, s.cand_glob, s.cand_lds};
  const int S = row_stride(ix, level);
  constexpr int kWide = (QR == 0 && !BUILD && NS <= 8) ? 2 : 1;  // (the search on long rows: dist_long)
  int n = n_seed;
  if (n > 0) {
    dist_list<DT, QR, false>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
    st.n_dist += n;
  }
  while (true) {
    wave_sync();
    int cid = -1;
    accept_list<NS>(s, st, tk, n, ef, lane, deleted);
    if (!st.fail && st.cand_size > 0) {
      wave_sync();
      const HeapEnt c = uniform_ent(s.cand[0]);
      const bool stop = (BUILD || (NS == 0 && deleted != nullptr)) ? (c.key > st.lower && st.top_size == ef) : (c.key > st.lower);
      if (!stop) {
        cid = (int)c.id;
        if (st.cand_size <= s.cand_lds) {
          LdsHeap cand_fast{s.cand};
          coop_pop<true>(cand_fast, st.cand_size, s.tree, lane);
        } else {
          coop_pop<true>(cand, st.cand_size, s.tree, lane);
        }
      }
    }
    wave_sync();
    if (cid < 0) break;
    st.n_hops += 1;
    const uint32_t* row = link_row(ix, (uint32_t)cid, level);
    if (S <= 64) {
      const VisitPending vp = visit_issue(row, S, s, lane);
      wave_sync();
      n = vp.n_ask;
      if (n > 0) dist_list<DT, QR, false, kWide>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
      wave_sync();
      st.n_dist += visit_commit(vp, s, st, lane);
    } else {
      n = visit_row(row, S, s, st, lane);
      wave_sync();
      if (n > 0) dist_list<DT, QR, false, kWide>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
      st.n_dist += n;
    }
  }
}

// ---- the tie-free fast path -------------------------------------------------------------
// hnswlib expands a candidate only while its key is <= lowerBound, the largest key of the
// result set, and once an entry has been evicted from the result set its key stays >= every
// later lowerBound.  So the candidates that are ever expanded are exactly the not yet
// expanded members of the result set, and ONE sorted set of (key, id, expanded) does the work
// of both priority queues (the reference's kernel uses the same view of the algorithm,
// cpp/include/cuda_search_kernels.cuh:99-164).  The equivalence is exact as long as no two
// keys that are in the set at the same time are equal: then the order of expansion, the
// evicted entry and the final order do not depend on how a heap lays equal keys out.  The set
// lives in registers, sorted, lane L holding positions [L*NS, L*NS + NS) (right-aligned like
// TopKeys); an insert is a shift through one DPP exchange, the next candidate is the first
// entry without the expanded mark.  An insert that meets an equal key reports it; the search
// kernel then repeats the query with the literal queues, the build (where any deterministic
// choice among equal keys is as good) carries on.
template <int NS>
struct Frontier {
  float k[NS > 0 ? NS : 1];
  uint32_t v[NS > 0 ? NS : 1];  // id; bit 31 = expanded (also set on the padding)
};
constexpr uint32_t kExpanded = 0x80000000u;
template <int NS>
__device__ __forceinline__ void frontier_init(Frontier<NS>& f, int ef, int lane) {
  constexpr int N = NS > 0 ? NS : 1;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    f.k[j] = (lane * N + j < 64 * N - ef) ? -INFINITY : INFINITY;
    f.v[j] = kEmpty;
  }
}
// Inserts (v, id) unless the id is already in the set (a neighbour met again after the lossy
// visited filter forgot it).  Returns 0 = inserted, 1 = inserted next to an equal key of
// another id, 2 = already present, nothing done.  Wavefront-uniform.
// With a[-1] the last key of the lane below, the new key at sorted position j is the median
// of (a[j-1], v, a[j]): a[j] where v is not below it, a[j-1] where v is below that too, else
// v itself; the ids follow the same two comparisons.  Equal keys keep their order of arrival.
template <int NS>
__device__ __forceinline__ int frontier_insert(Frontier<NS>& f, float v, uint32_t id, int lane) {
  constexpr int N = NS > 0 ? NS : 1;
  bool eq = false;
#pragma unroll
  for (int j = 0; j < N; ++j) eq = eq || f.k[j] == v;
  const bool any_eq = __ballot(eq) != 0ull;
  bool dup = false;
  if (any_eq) {
    bool same = false;
#pragma unroll
    for (int j = 0; j < N; ++j) same = same || (f.k[j] == v && (f.v[j] & ~kExpanded) == id);
    dup = __ballot(same) != 0ull;
  }
  // (one exit: early returns out of an inlined function inside the caller's loops cost the
  // caller a good deal of scalar control flow)
  if (!dup) {
    // last entry of the lane below (lane 0: "-inf", never taken over)
    const float prev_k = __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, f.k[N - 1]), 0x138, 0xF, 0xF, false));
    const uint32_t prev_v = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)f.v[N - 1], 0x138, 0xF, 0xF, false);
    bool below[N + 1];  // below[j + 1]: v sorts before a[j]; below[0]: before the lane below's last
    below[0] = v < prev_k;
#pragma unroll
    for (int j = 0; j < N; ++j) below[j + 1] = v < f.k[j];
#pragma unroll
    for (int j = N - 1; j >= 0; --j) {
      const float lo_k = j > 0 ? f.k[j - 1] : prev_k;
      const uint32_t lo_v = j > 0 ? f.v[j - 1] : prev_v;
      f.k[j] = __builtin_amdgcn_fmed3f(lo_k, v, f.k[j]);
      f.v[j] = below[j + 1] ? (below[j] ? lo_v : id) : f.v[j];
    }
  }
  return dup ? 2 : (any_eq ? 1 : 0);
}
// The same shift for a key that is known to differ from every key of the set (the caller has looked).
template <int NS>
__device__ __forceinline__ void frontier_insert_distinct(Frontier<NS>& f, float v, uint32_t id) {
  constexpr int N = NS > 0 ? NS : 1;
  const float prev_k = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, f.k[N - 1]), 0x138, 0xF, 0xF, false));
  const uint32_t prev_v = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)f.v[N - 1], 0x138, 0xF, 0xF, false);
#pragma unroll
  for (int j = N - 1; j >= 0; --j) {
    const float lo_k = j > 0 ? f.k[j - 1] : prev_k;
    const uint32_t lo_v = j > 0 ? f.v[j - 1] : prev_v;
    const bool before_this = v < f.k[j], before_lower = v < lo_k;
    f.k[j] = __builtin_amdgcn_fmed3f(lo_k, v, f.k[j]);
    f.v[j] = before_this ? (before_lower ? lo_v : id) : f.v[j];
  }
}
template <int NS>
__device__ __forceinline__ float frontier_max(const Frontier<NS>& f) {
  constexpr int N = NS > 0 ? NS : 1;
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f.k[N - 1]), 63));
}
// closest (far: farthest) entry not yet expanded: marks it and returns its id, or -1 when none
// is left.  The farthest one is what the reference expands with its reverse_cand option
// (GetCand, cpp/include/cuda_utils_kernels.cuh:104-151).
template <int NS>
__device__ __forceinline__ int frontier_take(Frontier<NS>& f, int lane, bool far = false) {
  constexpr int N = NS > 0 ? NS : 1;
  uint32_t vf = kEmpty;
  int L;
  if (!far) {
#pragma unroll
    for (int j = N - 1; j >= 0; --j) vf = (f.v[j] & kExpanded) == 0u ? f.v[j] : vf;
    const unsigned long long mask = __ballot((vf & kExpanded) == 0u);
    if (mask == 0ull) return -1;
    L = __builtin_ctzll(mask);
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) vf = (f.v[j] & kExpanded) == 0u ? f.v[j] : vf;
    const unsigned long long mask = __ballot((vf & kExpanded) == 0u);
    if (mask == 0ull) return -1;
    L = 63 - __builtin_clzll(mask);
  }
  const uint32_t id = (uint32_t)__builtin_amdgcn_readlane((int)vf, L);
  // (an id is in the set once: the entry that holds it is the one taken, whichever lane that is)
#pragma unroll
  for (int j = 0; j < N; ++j) f.v[j] = f.v[j] == id ? (id | kExpanded) : f.v[j];
  return (int)id;
}
// key of the entry with this id (which is in the set)
template <int NS>
__device__ __forceinline__ float frontier_key_of(const Frontier<NS>& f, uint32_t id) {
  constexpr int N = NS > 0 ? NS : 1;
  float kf = 0.f;
  bool hit = false;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const bool h = (f.v[j] & ~kExpanded) == id;
    kf = h ? f.k[j] : kf;
    hit = hit || h;
  }
  const unsigned long long mask = __ballot(hit);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kf), __builtin_ctzll(mask | (1ull << 63))));
}
// is there an entry not yet expanded with exactly this key?
template <int NS>
__device__ __forceinline__ bool frontier_open_key(const Frontier<NS>& f, float key) {
  constexpr int N = NS > 0 ? NS : 1;
  bool hit = false;
#pragma unroll
  for (int j = 0; j < N; ++j) hit = hit || ((f.v[j] & kExpanded) == 0u && f.k[j] == key);
  return __ballot(hit) != 0ull;
}
// do the two largest keys of a full set coincide?
template <int NS>
__device__ __forceinline__ bool frontier_max_twice(const Frontier<NS>& f) {
  constexpr int N = NS > 0 ? NS : 1;
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f.k[N - 1]), 63));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f.k[N > 1 ? N - 2 : 0]), 63));
  return a == b;
}
// do two neighbouring keys coincide among sorted positions p, p+1 with from <= p < upto and p+1 < count?
template <int NS>
__device__ __forceinline__ bool frontier_tie_within(const Frontier<NS>& f, int ef, int upto, int count, int lane,
                                                    int from = 0) {
  constexpr int N = NS > 0 ? NS : 1;
  const float next_first = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, f.k[0]), 0x130, 0xF, 0xF, false));  // wave_shl:1
  bool hit = false;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int pos = lane * N + j - (64 * N - ef);
    const float nxt = j + 1 < N ? f.k[j + 1 < N ? j + 1 : 0] : next_first;
    hit = hit || (pos >= from && pos < upto && pos + 1 < count && f.k[j] == nxt);
  }
  return __ballot(hit) != 0ull;
}
// The waiting (not yet expanded) entries whose key coincides with a neighbour's: while the tie-free loop runs on a
// set that holds equal keys, these are the entries it must not expand or push out by itself.
struct TieWatch {
  int id0 = -1, id1 = -1, id2 = -1, id3 = -1;  // (-1: unused; no taken candidate compares equal)
  float hi = -INFINITY;                        // their largest key
};
// Fills w; false when there are more than four such entries.
template <int NS>
__device__ __forceinline__ bool frontier_watch_list(const Frontier<NS>& f, TieWatch& w) {
  constexpr int N = NS > 0 ? NS : 1;
  const float prev_last = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, f.k[N - 1]), 0x138, 0xF, 0xF, false));  // wave_shr:1
  const float next_first = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, f.k[0]), 0x130, 0xF, 0xF, false));  // wave_shl:1
  unsigned long long m[N];
  int total = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float below = j > 0 ? f.k[j > 0 ? j - 1 : 0] : prev_last;
    const float above = j + 1 < N ? f.k[j + 1 < N ? j + 1 : 0] : next_first;
    m[j] = __ballot((f.v[j] & kExpanded) == 0u && (f.k[j] == below || f.k[j] == above));
    total += __popcll(m[j]);
  }
  w = TieWatch();
  if (total > 4) return false;
  int cnt = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    while (m[j] != 0ull) {
      const int L = __builtin_ctzll(m[j]);
      m[j] &= m[j] - 1ull;
      const int id = __builtin_amdgcn_readlane((int)f.v[j], L);
      const float key = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f.k[j]), L));
      if (cnt == 0) w.id0 = id;
      else if (cnt == 1) w.id1 = id;
      else if (cnt == 2) w.id2 = id;
      else w.id3 = id;
      w.hi = uni(fmaxf(w.hi, key));
      cnt += 1;
    }
  }
  return true;
}
// takes the expanded mark off an entry again
template <int NS>
__device__ __forceinline__ void frontier_untake(Frontier<NS>& f, uint32_t id) {
  constexpr int N = NS > 0 ? NS : 1;
#pragma unroll
  for (int j = 0; j < N; ++j) f.v[j] = f.v[j] == (id | kExpanded) ? id : f.v[j];
}
// writes the sorted entries [0, count) to out_id / out_key (LDS)
template <int NS>
__device__ __forceinline__ void frontier_dump(const Frontier<NS>& f, int ef, int count, uint32_t* out_id, float* out_key,
                                              int lane) {
  constexpr int N = NS > 0 ? NS : 1;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int pos = lane * N + j - (64 * N - ef);
    if (pos >= 0 && pos < count) {
      out_id[pos] = f.v[j] & ~kExpanded;
      out_key[pos] = f.k[j];
    }
  }
}

// The reference's reverse_cand search (expand the farthest waiting candidate, GetCand(..., reverse),
// cpp/include/cuda_utils_kernels.cuh:104-151) for result sets beyond the register set's capacity: one sorted list in
// LDS (s.top, ef entries, ascending; bit 31 of the id = expanded), equal keys in order of arrival, the last entry
// leaves a full list.  An insert counts the keys not above the new one (the list is sorted: whole chunks of 64
// until the first that is not) and moves the tail up one place, 64 entries at a time from the top; the next
// candidate is the last entry without the mark.  Exact visited bitmap.  A list of a thousand entries makes an
// insert a few dozen LDS round trips: the option is there for completeness, not for speed.  On entry
// s.nbuf[0..n_seed) holds the seeds (marked visited); on exit s.top[0..st.top_size) is the result in order.
template <int DT, int QR>
__device__ __forceinline__ void search_level_far_lds(const DevIndex& ix, const QVec<QR>& qv, int level, int ef, Scratch& s,
                                                     SearchState& st, int n_seed, int lane) {
  HeapEnt* set = s.top;
  const int S = row_stride(ix, level);
  int size = 0;
  int n = n_seed;
  while (true) {
    if (n > 0) dist_list<DT, QR, false>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
    st.n_dist += n;
    wave_sync();
    for (int j = 0; j < n; ++j) {
      const float key = s.dbuf[j];   // (the same address in every lane)
      const uint32_t id = s.nbuf[j];
      const float last_key = size > 0 ? set[size - 1].key : INFINITY;
      if (size < ef || last_key > key) {
        // where it goes: after every entry whose key is not above it
        int p = 0;
        for (int base = 0; base < size; base += 64) {
          const int i = base + lane;
          const unsigned long long le = __ballot(i < size && set[i < size ? i : 0].key <= key);
          p += __popcll(le);
          if (__popcll(le) < (size - base < 64 ? size - base : 64)) break;
        }
        const int new_size = size < ef ? size + 1 : ef;
        // entries [p, new_size - 1) move up one place, the topmost chunk first (each chunk is read whole
        // before it is written)
        for (int hi = new_size - 1; hi > p; hi -= 64) {
          const int dst = hi - lane;
          HeapEnt e = set[dst > p ? dst - 1 : p];
          wave_sync();
          if (dst > p) set[dst] = e;
          wave_sync();
        }
        if (lane == 0) {
          HeapEnt e;
          e.key = key;
          e.id = id;
          set[p] = e;
        }
        wave_sync();
        size = new_size;
      }
    }
    // the farthest entry still waiting
    int pick = -1;
    for (int hi = size - 1; hi >= 0 && pick < 0; hi -= 64) {
      const int i = hi - lane;
      const unsigned long long open = __ballot(i >= 0 && (set[i >= 0 ? i : 0].id & kExpanded) == 0u);
      if (open != 0ull) pick = hi - __builtin_ctzll(open);
    }
    if (pick < 0) break;
    const uint32_t cid = set[pick].id;
    wave_sync();
    if (lane == 0) set[pick].id = cid | kExpanded;
    st.n_hops += 1;
    n = visit_row(link_row(ix, cid, level), S, s, st, lane);
    wave_sync();
  }
  st.top_size = size;
}

// The sorted-set search's visited filter: a four-way set-associative tag cache in LDS alone, no
// bitmap.  A set is one 64-bit word holding four 16-bit tags (set = low id bits, tag = the
// rest; 0xFFFF = empty); a new tag pushes the oldest of the four out.  A hit is exact ("seen
// before"), a miss may be a node whose tag has been pushed out since: it is then evaluated
// again, which changes nothing — if it is still in the set the insert finds it, and if it was
// rejected or evicted its key is still not below the bound.  No atomics, no global memory,
// nothing to undo.  s.vcache / s.vc_bits hold the table and log2 of its size in 32-bit words.
// (Four ways rather than two at the same size: on the 1.18 M-point set the neighbourhoods
// overlap so much that most forgotten nodes were victims of set conflicts, not of capacity —
// repeated evaluations fell from 31 % to 12 % of the distinct ones.)
__device__ __forceinline__ void filter_reset(Scratch& s, int lane) {
  uint4* c4 = reinterpret_cast<uint4*>(s.vcache);
  const int n4 = (1 << s.vc_bits) >> 2;  // 2 sets per 16 bytes
  for (int i = lane; i < n4; i += 64) c4[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
  wave_sync();
}
__device__ __forceinline__ uint2 filter_push(uint2 w, uint32_t tag) {
  return make_uint2((w.x << 16) | tag, (w.y << 16) | (w.x >> 16));
}
// Compacts the ids of a link row that the filter does not know into s.nbuf; returns how many.
__device__ __forceinline__ int visit_lossy(const uint32_t* row, int S, Scratch& s, int lane) {
  int n = 0;
  uint2* sets = reinterpret_cast<uint2*>(s.vcache);
  const int set_bits = s.vc_bits - 1;
  const uint32_t mask_bits = (1u << set_bits) - 1u;
  for (int base = 0; base < S; base += 64) {
    const uint32_t got = row[base + lane < S ? base + lane : 0];  // unconditional load, then a select
    const uint32_t id = (base + lane < S) ? got : kEmpty;
    // (every lane looks its set up — an empty slot's id maps to some set and to a tag no set can hold — so that
    // the only predicated part is the two LDS writes at the end)
    const uint32_t slot = id & mask_bits;
    const uint32_t tag = id >> set_bits;
    const uint2 w = sets[slot];
    const bool ask = (id != kEmpty) & ((w.x & 0xFFFFu) != tag) & ((w.x >> 16) != tag) & ((w.y & 0xFFFFu) != tag) &
                     ((w.y >> 16) != tag);
    const unsigned long long mask = __ballot(ask);
    if (ask) {
      sets[slot] = filter_push(w, tag);
      s.nbuf[n + lanes_below(mask)] = id;
    }
    n += __popcll(mask);
  }
  return n;
}
__device__ __forceinline__ void visit_lossy_single(Scratch& s, uint32_t id, int lane) {
  if (lane == 0) {
    uint2* sets = reinterpret_cast<uint2*>(s.vcache);
    const int set_bits = s.vc_bits - 1;
    const uint32_t slot = id & ((1u << set_bits) - 1u);
    sets[slot] = filter_push(sets[slot], id >> set_bits);
  }
}

// The trail of a sorted-set search: the entries it accepted, hop by hop, wherever its course is certainly
// hnswlib's own.  A query that is given up afterwards is not searched again from its entry point: the
// literal pass takes the accepted entries of those hops from the trail — no link rows, no vectors, no
// arithmetic, only its queue and set operations in hnswlib's order — and searches on from where the trail
// ends.  One 16-byte record per accepted entry: (expanded node, accepted node, key bits, number of the hop);
// hops without an accepted entry leave none.  While equal keys wait side by side (a group that is followed
// through) the order of expansion may differ from hnswlib's and with it what each hop accepts: those hops are
// not recorded, two markers (kTrailOwn from hop h on, kTrailBack from hop h on) tell the literal pass to make
// them itself, in its own order; after such a group the set, the bound and the nodes met are the same again
// under either order, and so is what every later hop accepts.  The trail ends for good when the twins of an
// eviction come up (a node outside the set is expanded there).
constexpr uint32_t kTrailOwn = 0xFFFFFFFFu;
constexpr uint32_t kTrailBack = 0xFFFFFFFEu;
struct Trail {
  uint4* rec = nullptr;  // this search's records, or null: no trail is kept
  int cap = 0;
  int n = 0;         // records written; -1: the trail outgrew its buffer and is void
  int hops = 0;      // expansions the trail covers (all of them completed)
  int n_dist = 0;    // evaluations up to there
  bool on = false;   // still recording
  bool own = false;  // inside a stretch the literal pass makes itself
};
// (The wave barriers after the one-lane and some-lanes stores below emit nothing; they keep the end of such a
// branch a block of its own.  Merged into the join of the surrounding wavefront-uniform branches, it makes the
// compiler take every value that differs between those for lane-dependent -- the trail's state then sits in
// vector registers, of which the pass has none to spare.)
__device__ __forceinline__ void trail_mark(Trail& tr, uint32_t kind, int hop, int lane) {
  if (tr.on) {
    if (tr.n + 1 > tr.cap) {
      tr.on = false;
      tr.n = -1;
    } else {
      if (lane == 0) tr.rec[tr.n] = make_uint4(kind, 0u, 0u, (uint32_t)hop);
      __builtin_amdgcn_wave_barrier();
      tr.n += 1;
      tr.own = kind == kTrailOwn;
    }
  }
}
__device__ __forceinline__ void trail_hop(Trail& tr, unsigned long long accepted, int cid, int hop, uint32_t my_id,
                                          float my_key, int lane) {
  if (tr.on && !tr.own && accepted != 0ull && cid >= 0) {
    const int cnt = __popcll(accepted);
    if (tr.n + cnt > tr.cap) {
      tr.on = false;
      tr.n = -1;
    } else {
      if (__builtin_amdgcn_inverse_ballot_w64(accepted)) {  // (the lanes whose bit is set)
        tr.rec[tr.n + lanes_below(accepted)] = make_uint4((uint32_t)cid, my_id, __float_as_uint(my_key), (uint32_t)hop);
      }
      __builtin_amdgcn_wave_barrier();
      tr.n += cnt;
    }
  }
}
// the trail ends here: `hops` expansions are complete
__device__ __forceinline__ void trail_stop(Trail& tr, int hops, int n_dist) {
  if (tr.on) {
    tr.on = false;
    tr.hops = hops;
    tr.n_dist = n_dist;
  }
}

// One phase of the tie-free loop of search_level_fast (below).  Nine searches in ten never hold two equal keys in
// their set; until the first such pair turns up the search runs here, with none of the bookkeeping that equal keys
// need.  FULL = false: while the set fills (the bound is the largest key accepted so far, every offer is accepted);
// FULL = true: the set holds ef entries (the bound is its last key, an accepted offer pushes one out) — two
// instantiations, so that the hot one carries neither the fill test nor the running maximum.  TRAILS: the hop's
// accepted entries go on the search's trail (a kernel instance of its own: a pass that keeps no trails pays
// nothing for them).  WATCH: the set holds equal keys that do no harm as long as the waiting entries on the watch
// list (those with an equal in the set) are neither expanded nor pushed out here -- the loop hands back to the
// general one when that is about to happen.  BUILD: equal keys are taken in order of arrival and nothing is ever
// handed back.  Returns 0: no waiting entry is left, the search is over; 1: an offer met an equal key of another
// node, or its eviction would reach a watched entry (resume_at = which offer of the list in s.nbuf / s.dbuf);
// 2 (FULL = false only): the set is full now, the other phase goes on; 3 (WATCH only): the next candidate is a
// watched entry (its expanded mark has been taken off again, n = 0).  n = ids waiting in s.nbuf on entry.
template <int DT, int QR, int NS, bool FULL, bool TRAILS, bool WATCH, bool BUILD = false>
__device__ __forceinline__ int tie_free_phase(const DevIndex& ix, const QVec<QR>& qv, int level, int ef, int S, Scratch& s,
                                              SearchState& st, Frontier<NS>& fr, int& n, int& hop_cid, int& resume_at,
                                              unsigned long long& accepted, Trail& tr, const TieWatch& watch, int lane) {
  constexpr int N = NS > 0 ? NS : 1;
  constexpr int kWide = (QR == 0 && !BUILD && NS <= 8) ? 2 : 1;  // (the search on long rows: dist_long)
  // (said to be wavefront-uniform, so that they sit in scalar registers through the loop)
  const int w0 = WATCH ? uni(watch.id0) : -1, w1 = WATCH ? uni(watch.id1) : -1;
  const int w2 = WATCH ? uni(watch.id2) : -1, w3 = WATCH ? uni(watch.id3) : -1;
  const float w_hi = WATCH ? uni(watch.hi) : -INFINITY;
  while (true) {
    if (n > 0) dist_list<DT, QR, false, kWide>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
    st.n_dist += n;
    wave_sync();
    // (unconditional LDS reads at a clamped index, then a select: no exec-mask branches)
    const int last = n > 0 ? n - 1 : 0;
    const int at = lane < last ? lane : last;
    const float got_key = s.dbuf[at];
    const uint32_t my_id = s.nbuf[at];
    const float my_key = lane < n ? got_key : INFINITY;
    unsigned long long todo = FULL ? __ballot(st.lower > my_key) : __ballot(lane < n);
    while (todo != 0ull) {
      const int j = __builtin_ctzll(todo);
      todo &= todo - 1ull;
      const float key = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_key), j));
      const uint32_t id = (uint32_t)__builtin_amdgcn_readlane((int)my_id, j);
      if (FULL ? st.lower > key : (st.n_acc < ef || st.lower > key)) {
        bool eq = false;
#pragma unroll
        for (int t = 0; t < N; ++t) eq = eq || fr.k[t] == key;
        // (WATCH: an eviction that would reach a watched entry, or its equal, is the general loop's as well)
        // (while the set is not full its last key is the padding's +inf)
        if (WATCH) eq = eq || (lane == 63 && fr.k[N - 1] <= w_hi);
        if (__ballot(eq) == 0ull) {
          frontier_insert_distinct<NS>(fr, key, id);
          if (TRAILS) accepted |= 1ull << j;
          st.n_acc = st.n_acc + 1;
          if (!FULL && st.n_acc < ef) {
            st.maxkey = uni(fmaxf(st.maxkey, key));
            st.lower = st.maxkey;
          } else {
            st.lower = frontier_max<NS>(fr);  // hnswlib's lowerBound
          }
        } else {
          bool same = false;
#pragma unroll
          for (int t = 0; t < N; ++t) same = same || (fr.k[t] == key && (fr.v[t] & ~kExpanded) == id);
          if (__ballot(same) == 0ull) {
            if constexpr (BUILD) {
              // the build takes equal keys as they come (order of arrival): any deterministic choice is as good
              frontier_insert_distinct<NS>(fr, key, id);
              st.n_acc = st.n_acc + 1;
              if (!FULL && st.n_acc < ef) {
                st.maxkey = uni(fmaxf(st.maxkey, key));
                st.lower = st.maxkey;
              } else {
                st.lower = frontier_max<NS>(fr);
              }
            } else {
              resume_at = j;  // an equal key of another node (WATCH: or a watched eviction): the rules for equal keys apply from this offer on
              todo = 0ull;
            }
          }
          // (else: a node met again after the visited filter forgot it; it is in the set already)
        }
      }
    }
    if (resume_at >= 0) return 1;
    if (TRAILS) trail_hop(tr, accepted, hop_cid, st.n_hops, my_id, my_key, lane);
    accepted = 0ull;
    const int cid = frontier_take<NS>(fr, lane, false);
    if (cid < 0) return 0;
    if (WATCH && (cid == w0 || cid == w1 || cid == w2 || cid == w3)) {
      frontier_untake<NS>(fr, (uint32_t)cid);  // a watched entry's turn: the general loop takes it, with its bookkeeping
      n = 0;
      return 3;
    }
    hop_cid = cid;
    st.n_hops += 1;
    wave_sync();
    n = visit_lossy(link_row(ix, (uint32_t)cid, level), S, s, lane);
    wave_sync();
    if (!FULL && st.n_acc >= ef) return 2;
  }
}

// Best-first search of one level on the sorted set (needs the LDS tag filter).  On entry
// s.nbuf[0..n_seed) holds the seeds, already entered into the filter.  Returns 0: fr holds the
// result (st.top_size entries, ascending), all keys were distinct; 2: the same, but equal keys
// met on the way (the caller has to look at the cut at k); 1: given up — the outcome would
// depend on how hnswlib's heaps lay equal keys out.  st.n_dist counts the evaluations
// performed, repeated ones included.
//
// When do equal keys matter?  (a) Several waiting candidates share the smallest key d: hnswlib
// expands them in its heap's order.  If none of their expansions produces a key below d the
// order is immaterial — every node evaluated on the way is evaluated once whichever member
// meets it first, a key below d would be accepted under any order (d is within the bound), so
// none exists under any order, the whole group is expanded back to back and the set afterwards
// is the ef smallest of old set and offers either way — up to entries whose key equals the
// bound the set ends up with: whether such an offer is accepted or turned away, and which of
// several such entries is evicted, does depend on the order.  So a group during which an offer was turned
// away or an entry evicted whose key equals the bound at the group's end gives the query up.  A key below d
// turning up during the group does not by itself: such a candidate (and whatever closer ones it leads to) is
// expanded before the rest of the group under any order, and by the same argument the set after the last
// member is the same — provided every member does get expanded under any order, i.e. the bound is still at
// or above d when the group is through and no member was pushed out of the set before its turn; a second group
// of equal keys among those closer candidates is not followed (given up).  (b) An eviction finds equal largest keys: which one leaves is the heap's
// choice, and the one that leaves stays a live candidate of hnswlib as long as that key is
// within the bound.  The search goes on, but gives up if it comes to expand an entry with such
// a key, or ends while such a key is still within the bound — except in the one case that covers most of
// them: a single such eviction, out of exactly two equal largest keys, with fewer than the whole set asked
// for.  Then the two twins are known (the one the set kept, the one it pushed out: the "ghost", remembered
// with its expanded mark), hnswlib holds both in its candidate queue whichever of them its result heap kept,
// and when their key comes up — last of all, it is the bound — it expands each of them that is not expanded
// yet, in its heap's order.  If neither expansion has an offer accepted, the order is immaterial: nothing
// changes but the visited marks, and the search ends there.  So the twins are expanded one after the other
// (the ghost too, though it is not in the set), and only an accepted offer on the way gives the query up.
// (c) Equal keys across
// the cut at k (the result heap's choice) or among the k best (listed by label): the caller's business.
// far: expand the farthest waiting entry instead of the closest (the reference's
// reverse_cand); that is no hnswlib search any more, equal keys simply keep their order of
// arrival and nothing is ever given up.  BUILD likewise never gives up.
template <int DT, int QR, int NS, bool BUILD, bool TRAILS = false>
__device__ __forceinline__ int search_level_fast(const DevIndex& ix, const QVec<QR>& qv, int level, int ef, Scratch& s,
                                                  SearchState& st, Frontier<NS>& fr, int n_seed, int lane,
                                                  bool far = false, bool whole_set = false, Trail* trail = nullptr) {
  const int S = row_stride(ix, level);
  constexpr int kWide = (QR == 0 && !BUILD && NS <= 8) ? 2 : 1;  // (the search on long rows: dist_long)
  int n = n_seed;
  const bool exact = !BUILD && !far;  // the outcome has to be hnswlib's
  Trail no_trail;
  Trail& tr = trail ? *trail : no_trail;
  unsigned long long accepted = 0ull;  // offers of the current hop that entered the set
  int hop_cid = -1;                    // the node the current hop expanded (-1: the seeds)
  int ghosts = 0;                     // evictions that had equal largest keys to choose from
  uint32_t ghost = kEmpty;            // the entry the (single) such eviction pushed out, with its expanded mark
  bool twin_phase = false;            // the twins of that eviction are being expanded: no offer may be accepted
  bool have_tie = false;              // equal keys have met in the set
  bool in_group = false;              // the entries being expanded share one key with others still waiting
  float group_key = 0.f;
  float group_edge = INFINITY;        // closest key turned away or evicted while the group is expanded
  float ek_min = INFINITY;            // smallest key at which an eviction had equal largest keys to choose from
  bool gave_up = false;
  // Until two equal keys meet in the set the search runs in tie_free_phase — same decisions, half the
  // instructions per accepted candidate — and only then moves on to the general loop below, at the very offer
  // that met the equal key (resume_at).
  int resume_at = -1;
  bool calm = (exact || (BUILD && !far)) && S <= 64;  // no equal keys are at work (or none matter): the tie-free loop may run
  TieWatch watch;
  while (true) {
    if (calm) {
      int how = st.n_acc >= ef ? 2 : 0;
      if constexpr (BUILD) {
        if (how == 0) how = tie_free_phase<DT, QR, NS, false, false, false, true>(ix, qv, level, ef, S, s, st, fr, n, hop_cid, resume_at, accepted, tr, watch, lane);
        if (how == 2) how = tie_free_phase<DT, QR, NS, true, false, false, true>(ix, qv, level, ef, S, s, st, fr, n, hop_cid, resume_at, accepted, tr, watch, lane);
      } else if (!have_tie) {
        if (how == 0) how = tie_free_phase<DT, QR, NS, false, TRAILS, false>(ix, qv, level, ef, S, s, st, fr, n, hop_cid, resume_at, accepted, tr, watch, lane);
        if (how == 2) how = tie_free_phase<DT, QR, NS, true, TRAILS, false>(ix, qv, level, ef, S, s, st, fr, n, hop_cid, resume_at, accepted, tr, watch, lane);
      } else {
        // (after equal keys have met, the tie-free loop takes over again only once the set is full: how == 2)
        how = tie_free_phase<DT, QR, NS, true, TRAILS, true>(ix, qv, level, ef, S, s, st, fr, n, hop_cid, resume_at, accepted, tr, watch, lane);
      }
      st.top_size = st.n_acc < ef ? st.n_acc : ef;
      if (how == 0) {
        trail_stop(tr, st.n_hops, st.n_dist);
        return have_tie ? 2 : 0;
      }
      calm = false;
      // (what these were when the tie-free loop took over; said again so that none of them has to live through it)
      ghosts = 0;
      ghost = kEmpty;
      twin_phase = false;
      in_group = false;
      group_key = 0.f;
      group_edge = INFINITY;
      ek_min = INFINITY;
      gave_up = false;
    }
    while (true) {
      if (resume_at < 0) {
        if (n > 0) dist_list<DT, QR, false, kWide>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
        st.n_dist += n;
        wave_sync();
      }
      for (int base = 0; base < n; base += 64) {
        const int mine = base + lane;
        // unconditional LDS reads at a clamped index, then a select: no exec-mask branches
        const int at = mine < n ? mine : 0;
        const float my_key = mine < n ? s.dbuf[at] : INFINITY;
        const uint32_t my_id = s.nbuf[at];
        const bool pass = mine < n && (st.n_acc < ef || st.lower > my_key);
        unsigned long long todo = __ballot(pass);
        if (resume_at >= 0) {
          todo &= ~((1ull << resume_at) - 1ull);  // the offers before it have been dealt with (one list of at most 64)
          resume_at = -1;
        }
        // offers turned away while a group of equal keys is being expanded: remember the closest
        if (exact && in_group) group_edge = uni(fminf(group_edge, wave_min((mine < n && !pass) ? my_key : INFINITY)));
        // (plain if/else nesting, one way out of the loop: `continue` and `return` in here make the
        // compiler thread a state variable through a dozen scalar blocks per accepted candidate)
        while (todo != 0ull) {
          const int j = __builtin_ctzll(todo);
          todo &= todo - 1ull;
          const float key = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_key), j));
          const uint32_t id = (uint32_t)__builtin_amdgcn_readlane((int)my_id, j);
          if (st.n_acc < ef || st.lower > key) {
            // an eviction out of several equal largest keys: the heap's choice decides which of
            // them stays in the result set, and the other one stays a live candidate of hnswlib
            const bool twins = exact && have_tie && st.n_acc >= ef && frontier_max_twice<NS>(fr);
            // the entry a full set is about to push out, where somebody will ask for it
            const uint32_t evicted = (twins || (exact && in_group && st.n_acc >= ef && st.lower == group_key))
                                         ? (uint32_t)__builtin_amdgcn_readlane((int)fr.v[(NS > 0 ? NS : 1) - 1], 63)
                                         : kEmpty;
            const int r = frontier_insert<NS>(fr, key, id, lane);
            if (r != 2) {
              accepted |= 1ull << j;
              if (twins) {
                ek_min = uni(fminf(ek_min, st.lower));
                ghost = evicted;
                // (three or more equal largest keys, a second event, the whole set asked for: the plain rule)
                ghosts += (frontier_max_twice<NS>(fr) || whole_set) ? 2 : 1;
              }
              if (exact && twin_phase) {
                gave_up = true;  // which twin hnswlib expands first now decides whether the other one is expanded at all
                todo = 0ull;
              }
              have_tie = have_tie || r == 1;
              if (exact && in_group && st.n_acc >= ef) {
                group_edge = uni(fminf(group_edge, st.lower));  // the entry this insert evicted
                // a member of the group pushed out before its turn: with another order it would have been expanded
                if (st.lower == group_key && (evicted & kExpanded) == 0u) {
                  gave_up = true;
                  todo = 0ull;
                }
              }
              st.n_acc = uni(st.n_acc + 1);
              st.maxkey = uni(fmaxf(st.maxkey, key));
              st.lower = uni(st.n_acc >= ef ? frontier_max<NS>(fr) : st.maxkey);  // hnswlib's lowerBound
            }
          } else if (exact && in_group) {
            group_edge = uni(fminf(group_edge, key));
          }
        }
        if (gave_up) base = n;  // leave the outer loop as well
        else trail_hop(tr, accepted, hop_cid, st.n_hops, my_id, my_key, lane);  // (a trail is kept for rows of one pass only)
        accepted = 0ull;
      }
      if (gave_up) {
        trail_stop(tr, st.n_hops - 1, st.n_dist - n);  // (a trail still recording here: the hop under way, and its evaluations, are not on it)
        break;
      }
      st.top_size = st.n_acc < ef ? st.n_acc : ef;
      int cid = frontier_take<NS>(fr, lane, far);
      const bool was_in_group = in_group;
      if (exact && have_tie) {
        const float d = cid >= 0 ? frontier_key_of<NS>(fr, (uint32_t)cid) : INFINITY;
        if (in_group && cid >= 0 && d < group_key) {
          // a closer candidate turned up inside the group: it is expanded before the rest of the group under any
          // order.  A group within the group is not followed.
          gave_up = frontier_open_key<NS>(fr, d);
        } else if (in_group && d != group_key) {
          // the group is through.  With another order of its members an offer or an entry whose
          // key equals the bound reached now could have ended up on the other side of it; and with the bound
          // below the group's key a member popped late would not have been expanded at all.
          gave_up = st.n_acc >= ef && (group_edge == st.lower || st.lower < group_key);
          in_group = false;
        }
        if (cid >= 0) {
          if (d >= ek_min) {
            // the twin the set kept: it is the set's last entry and its key is the bound
            if (ghosts == 1 && !in_group && !frontier_open_key<NS>(fr, d)) twin_phase = true;
            else gave_up = true;
          }
          if (!in_group && !twin_phase) {
            in_group = frontier_open_key<NS>(fr, d);  // other waiting entries with this very key
            group_key = d;
            group_edge = INFINITY;
          }
        } else if (!gave_up && st.n_acc >= ef && st.lower >= ek_min) {
          // an entry evicted out of equal largest keys that are still within the bound is one
          // hnswlib would go on to expand
          if (ghosts == 1) {
            if ((ghost & kExpanded) == 0u) {
              cid = (int)ghost;  // the twin the set pushed out: expanded like any other, nothing of it may be accepted
              ghost |= kExpanded;
              twin_phase = true;
            }
          } else {
            gave_up = true;
          }
        }
      }
      // the trail: over for good, or the hops of a group of equal keys begin or end with the next one
      if (twin_phase || gave_up || cid < 0) trail_stop(tr, st.n_hops, st.n_dist);
      else if (in_group != was_in_group) trail_mark(tr, in_group ? kTrailOwn : kTrailBack, st.n_hops + 1, lane);
      if (gave_up || cid < 0) break;
      hop_cid = cid;
      st.n_hops += 1;
      wave_sync();
      n = visit_lossy(link_row(ix, (uint32_t)cid, level), S, s, lane);
      wave_sync();
      // Equal keys that sit in the set do no harm while none of them that still waits is expanded or pushed out
      // (unless the whole set is the answer): no group can form, and which of two expanded twins an eviction
      // pushes out changes neither the keys of the set nor hnswlib's candidates.  With no group under way and
      // no eviction out of equal largest keys on record whose key is still within the bound (once the bound is
      // below it, the entry such an eviction pushed out is as dead for hnswlib as any other), the tie-free loop
      // takes over again from this hop's offers, with the waiting entries that have an equal (at most four) on
      // its watch list; it comes back at the next offer that meets an equal key, when a watched entry's turn
      // comes, or when an eviction reaches one.
      if (exact && S <= 64 && !whole_set && st.n_acc >= ef && !in_group && !twin_phase && (ghosts == 0 || st.lower < ek_min) &&
          frontier_watch_list<NS>(fr, watch)) {
        calm = true;
        break;
      }
    }
    if (!calm) break;
  }
  return gave_up ? 1 : (have_tie ? 2 : 0);
}

// hnswlib's level-0 search with the literal candidate queue (which alone decides the order of
// expansion among equal keys) but with the sorted set with ids as result set and the LDS-only
// visited filter of the sorted-set search: a neighbour the filter has forgotten is evaluated
// again and then either found in the set by its id, or turned away by the accept rule as it
// was (or would be) the first time — the candidate queue sees exactly hnswlib's sequence of
// pushes and pops.  No bitmap, no atomics, nothing to undo.  Every accepted entry is also
// logged (s.log) for the caller's replay of the result heap.  *ambiguous is set when an
// eviction had equal largest keys to choose from: the set then holds the same keys as
// hnswlib's result heap but possibly another of the twins.  st.n_dist counts the evaluations
// performed, repeated ones included.  On entry s.nbuf[0..n_seed) holds the seeds, already
// entered into the filter.
template <int DT, int QR, int NS>
__device__ __forceinline__ void search_level_lean(const DevIndex& ix, const QVec<QR>& qv, int ef, Scratch& s, SearchState& st,
                                                  Frontier<NS>& fr, int n_seed, int lane, bool* ambiguous,
                                                  const uint4* trail = nullptr, int trail_n = 0, int trail_hops = 0,
                                                  int trail_n_dist = 0, int stop_marker = -1, int* rest_from = nullptr) {
  SplitHeap cand{s.cand, s.cand_glob, s.cand_lds};
  const int cand_cap = s.cand_lds + s.cand_glob_cap;
  const int S = row_stride(ix, 0);
  int n = n_seed;
  bool amb = false;
  // The first trail_hops expansions were made by the sorted-set pass too: outside the stretches its markers
  // set apart, their accepted entries come from its trail (records in hop order, none for a hop that accepted
  // nothing) instead of from link rows and vectors.  Every entry goes through the accept rule again: it
  // passes as it did there.
  int trail_at = 0;
  bool from_trail = false;
  bool own_stretch = false;  // between two markers: hops this pass makes itself
  if (trail_hops > 0) st.n_dist += trail_n_dist;  // the evaluations that pass made up to the trail's end count as performed
  while (true) {
    if (n > 0 && !from_trail) dist_list<DT, QR, false, (QR == 0 && NS <= 8) ? 2 : 1>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
    st.n_dist += from_trail ? 0 : n;
    wave_sync();
    for (int base = 0; base < n; base += 64) {
      const int mine = base + lane;
      const int at = mine < n ? mine : 0;
      const float my_key = mine < n ? s.dbuf[at] : INFINITY;
      const uint32_t my_id = s.nbuf[at];
      unsigned long long todo = __ballot(mine < n && (st.n_acc < ef || st.lower > my_key));
      while (todo != 0ull) {
        const int j = __builtin_ctzll(todo);
        todo &= todo - 1ull;
        HeapEnt e;
        e.key = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_key), j));
        e.id = (uint32_t)__builtin_amdgcn_readlane((int)my_id, j);
        if (st.n_acc < ef || st.lower > e.key) {
          const bool twins = st.n_acc >= ef && frontier_max_twice<NS>(fr);
          if (frontier_insert<NS>(fr, e.key, e.id, lane) != 2) {
            amb = amb || twins;
            if (st.cand_size >= cand_cap || st.n_acc >= s.log_cap) {
              st.fail = 1;  // (one way out of the loops: see search_level_fast)
              todo = 0ull;
            } else {
              if (lane == 0) s.log[st.n_acc] = e;
              st.n_acc = uni(st.n_acc + 1);
              if (st.cand_size < s.cand_lds) {
                LdsHeap cand_fast{s.cand};
                coop_push<true>(cand_fast, st.cand_size, e, lane);
              } else {
                coop_push<true>(cand, st.cand_size, e, lane);
              }
              st.maxkey = uni(fmaxf(st.maxkey, e.key));
              st.lower = uni(st.n_acc >= ef ? frontier_max<NS>(fr) : st.maxkey);  // hnswlib's lowerBound
            }
          }
        }
      }
      if (st.fail) base = n;
    }
    if (st.fail) break;
    st.top_size = st.n_acc < ef ? st.n_acc : ef;
    int cid = -1;
    if (st.cand_size > 0) {
      wave_sync();
      const HeapEnt c = uniform_ent(s.cand[0]);
      if (!(c.key > st.lower)) {
        cid = (int)c.id;
        if (st.cand_size <= s.cand_lds) {
          LdsHeap cand_fast{s.cand};
          coop_pop<true>(cand_fast, st.cand_size, s.tree, lane);
        } else {
          coop_pop<true>(cand, st.cand_size, s.tree, lane);
        }
      }
    }
    wave_sync();
    if (cid < 0) break;
    st.n_hops += 1;
    from_trail = false;
    if (st.n_hops <= trail_hops) {
      // markers that take effect with this hop (a group may end and the next begin at the same one)
      while (true) {
        const uint4 m = trail[trail_at < trail_n ? trail_at : 0];
        const uint32_t kind = (uint32_t)__builtin_amdgcn_readfirstlane((int)m.x);
        const uint32_t at_hop = (uint32_t)__builtin_amdgcn_readfirstlane((int)m.w);
        if (trail_at >= trail_n || kind < kTrailBack || at_hop != (uint32_t)st.n_hops) break;
        own_stretch = kind == kTrailOwn;
        trail_at += 1;
      }
      // (stop_marker >= 0: the trail covers the whole search and this is the index of its last marker.  Once past
      // it, every further accepted entry is on the trail: the caller needs no more of this search.)
      if (stop_marker >= 0 && !own_stretch && trail_at > stop_marker) {
        *rest_from = trail_at;
        break;
      }
      if (!own_stretch) {
        // this hop's records: a run from trail_at on (at most one link row's worth: under 64)
        const bool have = trail_at + lane < trail_n;
        const uint4 r = trail[have ? trail_at + lane : 0];
        const bool mine = have && r.x < kTrailBack && r.w == (uint32_t)st.n_hops;
        const unsigned long long run = __ballot(mine);
        const bool wrong = mine && r.x != (uint32_t)cid;
        if (__ballot(wrong) != 0ull) {
          trail_hops = 0;  // not the node that pass expanded here: nothing more is taken from the trail
        } else {
          n = __popcll(run);
          if (mine) {
            s.nbuf[lane] = r.y;
            s.dbuf[lane] = __uint_as_float(r.z);
          }
          // the filter learns the nodes (a later hop this pass makes itself need not evaluate them again), one
          // lane after the other: two records of a hop may fall into the same set of tags
          uint2* sets = reinterpret_cast<uint2*>(s.vcache);
          const int set_bits = s.vc_bits - 1;
          for (unsigned long long pend = run; pend != 0ull; pend &= pend - 1ull) {
            if (lane == __builtin_ctzll(pend)) {
              const uint32_t slot = r.y & ((1u << set_bits) - 1u);
              sets[slot] = filter_push(sets[slot], r.y >> set_bits);
            }
          }
          trail_at += n;
          from_trail = true;
        }
      }
    }
    if (!from_trail) n = visit_lossy(link_row(ix, (uint32_t)cid, 0), S, s, lane);
    wave_sync();
  }
  *ambiguous = amb;
}

// Greedy descent through levels from_level .. to_level+1 (hnswlib searchKnn upper
// loop; cpp/include/cuda_search_kernels.cuh:22-66 in the reference): each sweep
// scans the neighbour list captured at its start and moves to the strictly
// closest entry, which for a strict running minimum is the first occurrence of the
// list minimum.
template <int DT, int QR>
__device__ __forceinline__ void descend(const DevIndex& ix, const QVec<QR>& qv, int from_level, int to_level,
                                        uint32_t& cur, float& dcur, Scratch& s, SearchState& st, int lane) {
  for (int level = from_level; level > to_level; --level) {
    bool changed = true;
    while (changed) {
      changed = false;
      int n = load_row(link_row(ix, cur, level), ix.SU, s, lane);
      wave_sync();
      st.n_sweeps += 1;
      if (n == 0) break;
      dist_list<DT, QR, false>(ix, qv, s.qlds, s.nbuf, n, s.dbuf, lane);
      st.n_dist_upper += n;
      wave_sync();
      float best = INFINITY;
      int bidx = -1;
      for (int base = 0; base < n; base += 64) {
        int t = base + lane;
        float d = t < n ? s.dbuf[t] : INFINITY;
        float m = wave_min(d);
        if (m < best) {
          best = m;
          unsigned long long mask = __ballot(d == m);
          bidx = base + __ffsll((long long)mask) - 1;
        }
      }
      if (bidx >= 0 && best < dcur) {
        dcur = uni(best);
        cur = (uint32_t)uni((int)s.nbuf[bidx]);
        changed = true;
      }
      wave_sync();
    }
  }
}

// key of one node against the query (all lanes return it)
template <int DT, int QR>
__device__ __forceinline__ float dist_single(const DevIndex& ix, const QVec<QR>& qv, uint32_t id, Scratch& s, int lane) {
  if (lane == 0) s.nbuf[0] = id;
  wave_sync();
  dist_list<DT, QR, false>(ix, qv, s.qlds, s.nbuf, 1, s.dbuf, lane);
  wave_sync();
  float d = s.dbuf[0];
  wave_sync();
  return d;
}

// Ascending (key, tie) ranking of n LDS entries into out_id / out_key (rank sort,
// O(n^2 / 64) per lane).  tie[] may be null (then the id breaks ties).
__device__ __forceinline__ void rank_sort(const HeapEnt* in, const uint64_t* tie, int n, uint32_t* out_id, float* out_key,
                                          int lane) {
  for (int e = lane; e < n; e += 64) {
    HeapEnt me = in[e];
    uint64_t mt = tie ? tie[e] : (uint64_t)me.id;
    int rank = 0;
    for (int f = 0; f < n; ++f) {
      HeapEnt o = in[f];
      uint64_t ot = tie ? tie[f] : (uint64_t)o.id;
      rank += (o.key < me.key || (o.key == me.key && ot < mt)) ? 1 : 0;
    }
    out_id[rank] = me.id;
    out_key[rank] = me.key;
  }
}

// ids[0..n) with keys[0..n) ascending (LDS): puts the ids of every run of equal keys into the
// order of their labels, which is how hnswlib's answer orders equal distances (its result queue
// compares (distance, label) pairs).  tmp: n words of LDS.
__device__ __forceinline__ void order_equal_keys(const DevIndex& ix, uint32_t* ids, const float* keys, int n, uint32_t* tmp,
                                                 int lane) {
  for (int e = lane; e < n; e += 64) tmp[e] = ids[e];
  wave_sync();
  for (int e = lane; e < n; e += 64) {
    const float k = keys[e];
    const uint32_t me = tmp[e];
    const uint64_t ml = ix.labels ? ix.labels[me] : (uint64_t)me;
    int rank = e;
    for (int f = e - 1; f >= 0 && keys[f] == k; --f) {
      const uint32_t o = tmp[f];
      rank -= (ix.labels ? ix.labels[o] : (uint64_t)o) > ml ? 1 : 0;
    }
    for (int f = e + 1; f < n && keys[f] == k; ++f) {
      const uint32_t o = tmp[f];
      rank += (ix.labels ? ix.labels[o] : (uint64_t)o) < ml ? 1 : 0;
    }
    ids[rank] = me;
  }
  wave_sync();
}

// Collects from the log the entries that make up the k best: those with key <= bound.
// Returns how many there are (they are stored while they fit cap).  More than `want`
// means equal keys straddle the cut, which only the literal heap can resolve.
__device__ __forceinline__ int collect_le(const HeapEnt* log, int n, float bound, HeapEnt* out, int cap, int lane) {
  int cnt = 0;
  for (int base = 0; base < n; base += 64) {
    const int i = base + lane;
    HeapEnt e;
    e.key = INFINITY;
    e.id = 0;
    if (i < n) e = log[i];
    const bool keep = i < n && e.key <= bound;
    const unsigned long long mask = __ballot(keep);
    const int pos = cnt + lanes_below(mask);
    if (keep && pos < cap) out[pos] = e;
    cnt += __popcll(mask);
  }
  return cnt;
}
// Same with a strict bound first and ties filling up to `want` in log order (build: any
// deterministic choice among equal keys is fine).
__device__ __forceinline__ int collect_best(const HeapEnt* log, int n, float bound, int want, HeapEnt* out, int lane) {
  int cnt = 0;
  for (int pass = 0; pass < 2; ++pass) {
    for (int base = 0; base < n && cnt < want; base += 64) {
      const int i = base + lane;
      HeapEnt e;
      e.key = INFINITY;
      e.id = 0;
      if (i < n) e = log[i];
      const bool keep = i < n && (pass == 0 ? e.key < bound : e.key == bound);
      const unsigned long long mask = __ballot(keep);
      const int pos = cnt + lanes_below(mask);
      if (keep && pos < want) out[pos] = e;
      cnt += __popcll(mask);
    }
  }
  return cnt < want ? cnt : want;
}

}  // namespace cuhnsw_amd
