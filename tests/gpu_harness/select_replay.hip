// GPU test harness (not part of the product library): runs the product's neighbour selection
// (select_neighbors in cuhnsw_amd/csrc/kernels.h, the counterpart of the reference's SearchHeuristic,
// cpp/include/cuda_build_kernels.cuh:68-162) on explicit candidate lists, one wavefront per list, and
// returns the rows, so that a test can compare them with the CPU oracle's statement of the same rule.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <vector>

#include "kernels.h"

using namespace cuhnsw_amd;

struct SelectCases {
  const uint32_t* cand_ids;   // concatenated candidate lists, each ascending by key
  const float* cand_keys;
  const int* cand_off;        // n_cases + 1 offsets into the two arrays
  const int* m;               // per case: row capacity
  const int* nn_num;          // per case: picks that pass untested
  const int* save_remains;    // per case
  const uint32_t* new_from;   // per case: candidates with ids from here on are newcomers to a row the rule produced (0 = none)
  uint32_t* out_ids;          // n_cases x cap
  float* out_keys;
  int* out_deg;
  int n_cases, cap, max_t, lcap;
};

template <int DT, int QR>
__global__ void __launch_bounds__(64) select_kernel(DevIndex ix, SelectCases c) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  const LdsPlan lp = plan_lds(QR, ix.Dp, -1, 0, c.lcap, c.max_t, c.cap);
  Scratch s;
  s.qlds = reinterpret_cast<float4*>(smem + lp.qlds);
  s.nbuf = reinterpret_cast<uint32_t*>(smem + lp.nbuf);
  s.dbuf = reinterpret_cast<float*>(smem + lp.dbuf);
  uint32_t* sid = reinterpret_cast<uint32_t*>(smem + lp.sorted_id);
  float* skey = reinterpret_cast<float*>(smem + lp.sorted_key);
  uint32_t* oid = reinterpret_cast<uint32_t*>(smem + lp.out_id);
  float* okey = reinterpret_cast<float*>(smem + lp.out_key);
  for (int i = blockIdx.x; i < c.n_cases; i += gridDim.x) {
    const int beg = c.cand_off[i], T = c.cand_off[i + 1] - beg;
    for (int t = lane; t < T; t += 64) {
      sid[t] = c.cand_ids[beg + t];
      skey[t] = c.cand_keys[beg + t];
    }
    wave_sync();
    const int deg = select_neighbors<DT, QR>(ix, sid, skey, T, c.m[i], c.nn_num[i], c.save_remains[i], oid, okey, s, lane,
                                             nullptr, c.new_from[i]);
    wave_sync();
    for (int j = lane; j < c.cap; j += 64) {
      c.out_ids[(size_t)i * c.cap + j] = j < deg ? oid[j] : kEmpty;
      c.out_keys[(size_t)i * c.cap + j] = j < deg ? okey[j] : 0.f;
    }
    if (lane == 0) c.out_deg[i] = deg;
    wave_sync();
  }
}

template <int DT, int QR>
static int run(const DevIndex& ix, const SelectCases& c) {
  const LdsPlan lp = plan_lds(QR, ix.Dp, -1, 0, c.lcap, c.max_t, c.cap);
  if (lp.total > 64 * 1024) return 3;
  hipLaunchKernelGGL((select_kernel<DT, QR>), dim3(std::min(c.n_cases, 1024)), dim3(64), lp.total, 0, ix, c);
  if (hipGetLastError() != hipSuccess) return 4;
  return hipDeviceSynchronize() == hipSuccess ? 0 : 2;
}
template <int DT>
static int run_qr(int qr, const DevIndex& ix, const SelectCases& c) {
  switch (qr) {
    case 1: return run<DT, 1>(ix, c);
    case 2: return run<DT, 2>(ix, c);
    case 4: return run<DT, 4>(ix, c);
    default: return run<DT, 0>(ix, c);
  }
}

template <typename T>
static T* upload(const std::vector<T>& v) {
  T* p = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&p), std::max<size_t>(v.size(), 1) * sizeof(T)) != hipSuccess) return nullptr;
  if (!v.empty() && hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return p;
}

// vectors: N x D fp32 (already rounded to fp16 values when half != 0).  Returns 0 on success.
extern "C" int select_replay(const float* vectors, int N, int D, int dist_type, int half, int n_cases, const unsigned* cand_ids,
                             const float* cand_keys, const int* cand_off, const int* m, const int* nn_num,
                             const int* save_remains, const unsigned* new_from, int cap, unsigned* out_ids, float* out_keys,
                             int* out_deg) {
  const int Dp = padded_dims(D);
  DevIndex ix{};
  void* d_vec = nullptr;
  if (half) {
    std::vector<_Float16> rows((size_t)N * Dp, (_Float16)0.f);
    for (int i = 0; i < N; ++i)
      for (int j = 0; j < D; ++j) rows[(size_t)i * Dp + j] = (_Float16)vectors[(size_t)i * D + j];
    d_vec = upload(rows);
  } else {
    std::vector<float> rows((size_t)N * Dp, 0.f);
    for (int i = 0; i < N; ++i) std::copy(vectors + (size_t)i * D, vectors + (size_t)(i + 1) * D, rows.begin() + (size_t)i * Dp);
    d_vec = upload(rows);
  }
  if (!d_vec) return 1;
  ix.vectors = d_vec;
  ix.half = half;
  ix.N = N; ix.D = D; ix.Dp = Dp;
  const int total = cand_off[n_cases];
  int max_t = 1, max_m = 1;
  for (int i = 0; i < n_cases; ++i) {
    max_t = std::max(max_t, cand_off[i + 1] - cand_off[i]);
    max_m = std::max(max_m, m[i]);
    if (m[i] > cap) return 5;
    for (int t = cand_off[i]; t < cand_off[i + 1]; ++t)
      if (cand_ids[t] >= (unsigned)N) return 6;   // operands checked on the host before anything is launched
  }
  SelectCases c{};
  c.cand_ids = upload(std::vector<uint32_t>(cand_ids, cand_ids + total));
  c.cand_keys = upload(std::vector<float>(cand_keys, cand_keys + total));
  c.cand_off = upload(std::vector<int>(cand_off, cand_off + n_cases + 1));
  c.m = upload(std::vector<int>(m, m + n_cases));
  c.nn_num = upload(std::vector<int>(nn_num, nn_num + n_cases));
  c.save_remains = upload(std::vector<int>(save_remains, save_remains + n_cases));
  c.new_from = upload(std::vector<uint32_t>(new_from, new_from + n_cases));
  c.out_ids = upload(std::vector<uint32_t>((size_t)n_cases * cap, 0u));
  c.out_keys = upload(std::vector<float>((size_t)n_cases * cap, 0.f));
  c.out_deg = upload(std::vector<int>(n_cases, 0));
  c.n_cases = n_cases; c.cap = cap; c.max_t = max_t;
  c.lcap = (std::max(max_m, 64) + 63) / 64 * 64;
  const int qr = query_regs(Dp);
  int rc = dist_type == DIST_DOT ? run_qr<DIST_DOT>(qr, ix, c) : run_qr<DIST_L2>(qr, ix, c);
  if (rc == 0) {
    if (hipMemcpy(out_ids, c.out_ids, (size_t)n_cases * cap * 4, hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(out_keys, c.out_keys, (size_t)n_cases * cap * 4, hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(out_deg, c.out_deg, (size_t)n_cases * 4, hipMemcpyDeviceToHost) != hipSuccess)
      rc = 7;
  }
  (void)hipFree(d_vec);
  (void)hipFree(const_cast<uint32_t*>(c.cand_ids)); (void)hipFree(const_cast<float*>(c.cand_keys));
  (void)hipFree(const_cast<int*>(c.cand_off)); (void)hipFree(const_cast<int*>(c.m)); (void)hipFree(const_cast<int*>(c.nn_num));
  (void)hipFree(const_cast<int*>(c.save_remains)); (void)hipFree(const_cast<uint32_t*>(c.new_from)); (void)hipFree(c.out_ids); (void)hipFree(c.out_keys); (void)hipFree(c.out_deg);
  return rc;
}
