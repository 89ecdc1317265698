// Two queries per wavefront: the sorted-set search of search_level_fast with each half of the
// wavefront (32 lanes) owning one query.
//
// Why: the one-query-per-wavefront pass is bound by instruction issue — about 200 vector and 200 scalar
// instructions per expanded candidate, and a SIMD issues roughly one instruction of a wavefront every
// four cycles whatever its kind — not by memory (random 256-byte row gathers alone run five times
// faster than the search needs them).  With two queries side by side the scalar control flow, the link
// row fetch, the visited filter and the distance passes are issued once for both, a distance pass is
// always full (two 16-lane groups per query), and a CU holds twice the queries per resident wavefront.
//
// The halves run in lock step through STEPS.  A step is, for each half independently, one of
//   ENTRY    evaluate the index's entry point,
//   DESCEND  one sweep of the greedy descent on an upper level (hnswlib searchKnn upper loop;
//            cpp/include/cuda_search_kernels.cuh:22-66 in the reference),
//   SEED     offer the level-0 entry to the empty sorted set,
//   SEARCH   expand the closest waiting candidate of the sorted set (one hop of
//            cpp/include/cuda_search_kernels.cuh:99-164),
// all of which share one shape: a list of at most 32 node ids per half (a link row, filtered or not, or
// a single id) -> their keys in one joint distance pass -> a per-half consumer.  A half whose query ends
// writes its answer (or hands the query to the literal pass) and takes the next query off the batch's
// counter while the other half carries on.  Everything a half "knows" (counters, bounds, flags) is a
// vector register holding the same value in its 32 lanes; cross-lane traffic stays inside a half.
//
// The rules for equal keys are those of search_level_fast, statement for statement.
#pragma once
#include "device_core.h"

namespace cuhnsw_amd {

// ---- half-wavefront primitives ----------------------------------------------------------------------
__device__ __forceinline__ uint32_t half_ballot(bool p, int lane) {
  const unsigned long long b = __ballot(p);
  return lane < 32 ? (uint32_t)b : (uint32_t)(b >> 32);
}
__device__ __forceinline__ bool wave_any(bool p) { return __ballot(p) != 0ull; }
// value of lane `src` (0..31, the same in all lanes of a half) of the caller's half
__device__ __forceinline__ int half_read(int x, int src, int lane) {
  return __builtin_amdgcn_ds_bpermute(((lane & 32) | src) << 2, x);
}
__device__ __forceinline__ float half_read(float x, int src, int lane) {
  return __builtin_bit_cast(float, half_read(__builtin_bit_cast(int, x), src, lane));
}
// value of the half's last lane (31 / 63)
__device__ __forceinline__ float half_last(float x, int lane) {
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 31));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
  return lane < 32 ? a : b;
}
__device__ __forceinline__ float half_min(float x) {
#pragma unroll
  for (int m = 16; m >= 1; m >>= 1) x = fminf(x, __shfl_xor(x, m, 64));
  return x;
}

// ---- the sorted set on 32 lanes -----------------------------------------------------------------------
// Frontier<N> as in device_core.h, but lane hl = lane & 31 of a half holds sorted positions
// [hl*N, hl*N + N), right-aligned: position p lives in slot p + 32*N - ef.
template <int N>
__device__ __forceinline__ void pf_init(Frontier<N>& f, int ef, int hl) {
#pragma unroll
  for (int j = 0; j < N; ++j) {
    f.k[j] = (hl * N + j < 32 * N - ef) ? -INFINITY : INFINITY;
    f.v[j] = kEmpty;
  }
}
// Inserts (v, id) into the caller's half where `on`; returns 0 = inserted, 1 = inserted next to an equal key of
// another id, 2 = the id is in the set already (nothing done), 3 = not asked to.
template <int N>
__device__ __forceinline__ int pf_insert(Frontier<N>& f, float v, uint32_t id, bool on, int lane) {
  const int hl = lane & 31;
  bool eq = false;
#pragma unroll
  for (int j = 0; j < N; ++j) eq = eq || f.k[j] == v;
  const unsigned long long eqm = __ballot(eq && on);
  const bool any_eq = (lane < 32 ? (uint32_t)eqm : (uint32_t)(eqm >> 32)) != 0u;
  bool dup = false;
  if (eqm != 0ull) {  // wavefront-uniform: no half met an equal key in the usual case
    bool same = false;
#pragma unroll
    for (int j = 0; j < N; ++j) same = same || (f.k[j] == v && (f.v[j] & ~kExpanded) == id);
    dup = half_ballot(same && on, lane) != 0u;
  }
  const bool go = on && !dup;
  const float x = go ? v : INFINITY;  // +inf leaves a half's set as it is: every key is the median of (a[j-1], inf, a[j])
  float prev_k = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, f.k[N - 1]), 0x138, 0xF, 0xF, false));
  uint32_t prev_v = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)f.v[N - 1], 0x138, 0xF, 0xF, false);
  prev_k = hl == 0 ? -INFINITY : prev_k;  // (lane 32 must not take over lane 31's entry: that is the other query's)
  prev_v = hl == 0 ? 0u : prev_v;
  bool below[N + 1];
  below[0] = x < prev_k;
#pragma unroll
  for (int j = 0; j < N; ++j) below[j + 1] = x < f.k[j];
#pragma unroll
  for (int j = N - 1; j >= 0; --j) {
    const float lo_k = j > 0 ? f.k[j - 1] : prev_k;
    const uint32_t lo_v = j > 0 ? f.v[j - 1] : prev_v;
    f.k[j] = __builtin_amdgcn_fmed3f(lo_k, x, f.k[j]);
    f.v[j] = below[j + 1] ? (below[j] ? lo_v : id) : f.v[j];
  }
  return !on ? 3 : (dup ? 2 : (any_eq ? 1 : 0));
}
template <int N>
__device__ __forceinline__ float pf_max(const Frontier<N>& f, int lane) {
  return half_last(f.k[N - 1], lane);
}
template <int N>
__device__ __forceinline__ bool pf_max_twice(const Frontier<N>& f, int lane) {
  const float a = half_last(f.k[N - 1], lane);
  const float b = half_last(f.k[N > 1 ? N - 2 : 0], lane);
  return a == b;
}
// closest waiting entry of the caller's half where `on`: marks it expanded and returns its id, -1 when none
template <int N>
__device__ __forceinline__ int pf_take(Frontier<N>& f, bool on, int lane) {
  const int hl = lane & 31;
  uint32_t vf = kEmpty;
#pragma unroll
  for (int j = N - 1; j >= 0; --j) vf = (f.v[j] & kExpanded) == 0u ? f.v[j] : vf;
  const uint32_t mask = half_ballot((vf & kExpanded) == 0u, lane);
  const int L = __builtin_ctz(mask | 0x80000000u);
  const uint32_t id = (uint32_t)half_read((int)vf, L, lane);
  const bool got = on && mask != 0u;
#pragma unroll
  for (int j = 0; j < N; ++j) f.v[j] = (got && hl == L && f.v[j] == id) ? (id | kExpanded) : f.v[j];
  return got ? (int)id : -1;
}
template <int N>
__device__ __forceinline__ float pf_key_of(const Frontier<N>& f, uint32_t id, int lane) {
  float kf = 0.f;
  bool hit = false;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const bool h = (f.v[j] & ~kExpanded) == id;
    kf = h ? f.k[j] : kf;
    hit = hit || h;
  }
  const uint32_t mask = half_ballot(hit, lane);
  return half_read(kf, __builtin_ctz(mask | 0x80000000u), lane);
}
template <int N>
__device__ __forceinline__ bool pf_open_key(const Frontier<N>& f, float key, int lane) {
  bool hit = false;
#pragma unroll
  for (int j = 0; j < N; ++j) hit = hit || ((f.v[j] & kExpanded) == 0u && f.k[j] == key);
  return half_ballot(hit, lane) != 0u;
}
// do two neighbouring keys coincide among sorted positions p, p+1 with from <= p < upto and p+1 < count?
template <int N>
__device__ __forceinline__ bool pf_tie_within(const Frontier<N>& f, int ef, int upto, int count, int from, int lane) {
  const int hl = lane & 31;
  // (lane 31 reads lane 32's first key here, but its last slot is position ef - 1, which p + 1 < count excludes)
  const float next_first = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, f.k[0]), 0x130, 0xF, 0xF, false));  // wave_shl:1
  bool hit = false;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int pos = hl * N + j - (32 * N - ef);
    const float nxt = j + 1 < N ? f.k[j + 1 < N ? j + 1 : 0] : next_first;
    hit = hit || (pos >= from && pos < upto && pos + 1 < count && f.k[j] == nxt);
  }
  return half_ballot(hit, lane) != 0u;
}
template <int N>
__device__ __forceinline__ void pf_dump(const Frontier<N>& f, int ef, int count, uint32_t* out_id, float* out_key, bool on,
                                        int lane) {
  const int hl = lane & 31;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int pos = hl * N + j - (32 * N - ef);
    if (on && pos >= 0 && pos < count) {
      out_id[pos] = f.v[j] & ~kExpanded;
      out_key[pos] = f.k[j];
    }
  }
}

// ---- joint distance pass --------------------------------------------------------------------------------
// keys of ids[0..n) of either half against that half's query (registers) -> out[0..n); ids / out / n are the
// caller's half's.  Two 16-lane groups per half, U rows per group in flight.  ids[0] is always a valid id.
template <int DT, int R, int U, bool RAW, bool HALF>
__device__ __forceinline__ void pair_dist_pass(const void* rows, uint32_t rowlen, uint32_t used, const float4* q,
                                               const uint32_t* ids, int r, int n, float* out, int gg, int sub) {
  float4 v[U][R];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int idx = r + 2 * u + gg;
    const uint32_t id = ids[idx < n ? idx : (n > 0 ? n - 1 : 0)];
    const uint64_t first = (uint64_t)id * rowlen;
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const uint32_t c = sub + 16 * k;
      const uint64_t at = first + (c < used ? c : 0);  // a chunk past the row's data re-reads chunk 0 (no extra line)
      const float4 t = HALF ? load_chunk_f16(rows, at) : load_chunk_f32(rows, at);
      v[u][k] = (DT == DIST_DOT || c < used) ? t : q[k];  // the query holds zeros there: enough for a dot product
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    float ax = 0.f, ay = 0.f, az = 0.f, aw = 0.f;
#pragma unroll
    for (int k = 0; k < R; ++k) acc4<DT>(q[k], v[u][k], ax, ay, az, aw);
    const float key = finish16<DT, RAW>(ax, ay, az, aw);
    const int idx = r + 2 * u + gg;
    if (sub == 0 && idx < n) out[idx] = key;
  }
}
template <int DT, int QR, bool RAW, bool HALF>
__device__ __forceinline__ void pair_dist_t(const DevIndex& ix, const QVec<QR>& qv, const uint32_t* ids, int n, float* out,
                                            int lane) {
  const int gg = (lane >> 4) & 1, sub = lane & 15;
  const uint32_t rowlen = (uint32_t)ix.Dp >> 2, used = ((uint32_t)ix.D + 3u) >> 2;
  const int n0 = __builtin_amdgcn_readfirstlane(n), n1 = __builtin_amdgcn_readlane(n, 32);
  const int nmax = n0 > n1 ? n0 : n1;
  constexpr int UMAX = QR == 1 ? 4 : 2;
  int r = 0;
  while (r < nmax) {
    const int rem = nmax - r;
    if (UMAX >= 4 && rem > 4) {
      pair_dist_pass<DT, QR, (UMAX >= 4 ? 4 : 1), RAW, HALF>(ix.vectors, rowlen, used, qv.q, ids, r, n, out, gg, sub);
      r += 8;
    } else if (rem > 2) {
      pair_dist_pass<DT, QR, 2, RAW, HALF>(ix.vectors, rowlen, used, qv.q, ids, r, n, out, gg, sub);
      r += 4;
    } else {
      pair_dist_pass<DT, QR, 1, RAW, HALF>(ix.vectors, rowlen, used, qv.q, ids, r, n, out, gg, sub);
      r += 2;
    }
  }
}
template <int DT, int QR, bool RAW>
__device__ __forceinline__ void pair_dist(const DevIndex& ix, const QVec<QR>& qv, const uint32_t* ids, int n, float* out,
                                          int lane) {
  if (uni(ix.half) != 0) pair_dist_t<DT, QR, RAW, true>(ix, qv, ids, n, out, lane);
  else pair_dist_t<DT, QR, RAW, false>(ix, qv, ids, n, out, lane);
}

// LDS of one wavefront of the pair search: per half a visited filter and the id / key buffers
struct PairLdsPlan {
  size_t half_bytes, fcache, nbuf, dbuf, total;
};
__host__ __device__ inline PairLdsPlan plan_pair_lds(int lcap, int fc_bits) {
  PairLdsPlan p;
  size_t o = 0;
  p.fcache = o; o = (o + ((size_t)4 << fc_bits) + 15) & ~(size_t)15;
  p.nbuf = o; o = (o + (size_t)lcap * 4 + 15) & ~(size_t)15;
  p.dbuf = o; o = (o + (size_t)lcap * 4 + 15) & ~(size_t)15;
  p.half_bytes = o;
  p.total = 2 * o;
  return p;
}

enum PairPhase { PP_NEED = 0, PP_ENTRY = 1, PP_DESCEND = 2, PP_SEED = 3, PP_SEARCH = 4, PP_IDLE = 5 };

}  // namespace cuhnsw_amd
