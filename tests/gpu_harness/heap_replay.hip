// GPU test harness (not part of the product library): replays a push / pop sequence on
// the product's cooperative wavefront heap (cuhnsw_amd/csrc/heap_coop.h, through the
// LDS + global-overflow accessor the kernels use) and returns snapshots of the heap
// array, so that a test can compare them with libstdc++-literal heaps slot by slot.
#include <hip/hip_runtime.h>

#include <vector>

#include "device_core.h"

using namespace cuhnsw_amd;

template <bool MINQ>
__global__ void __launch_bounds__(64) replay_kernel(const float* keys, int n_ops, int lds_cap, HeapEnt* glob,
                                                    HeapEnt* dumps, int cap, int dump_every, int* sizes, int* popped) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x;
  SplitHeap h{reinterpret_cast<HeapEnt*>(smem), glob, lds_cap};
  const StageTree tree = make_stage_tree(lane);
  int size = 0;
  for (int op = 0; op < n_ops; ++op) {
    const float k = keys[op];
    if (k >= 0.f) {
      HeapEnt e;
      e.key = k;
      e.id = (uint32_t)op;
      coop_push<MINQ>(h, size, e, lane);
      if (lane == 0) popped[op] = -1;
    } else {
      wave_sync();
      HeapEnt root = uniform_ent(h.get(0));
      if (lane == 0) popped[op] = (int)root.id;
      coop_pop<MINQ>(h, size, tree, lane);
    }
    if ((op + 1) % dump_every == 0) {
      wave_sync();
      HeapEnt* d = dumps + (size_t)(op / dump_every) * cap;
      for (int i = lane; i < size; i += 64) d[i] = h.get(i);
      if (lane == 0) sizes[op / dump_every] = size;
    }
  }
}

extern "C" int heap_replay(const float* keys, int n_ops, int minq, int lds_cap, int cap, int dump_every, float* dump_keys,
                           unsigned* dump_ids, int* sizes, int* popped) {
  float* d_keys = nullptr;
  HeapEnt *d_glob = nullptr, *d_dumps = nullptr;
  int *d_sizes = nullptr, *d_popped = nullptr;
  const int n_dumps = n_ops / dump_every;
  if (hipMalloc(&d_keys, sizeof(float) * n_ops) != hipSuccess) return 1;
  (void)hipMalloc(&d_glob, sizeof(HeapEnt) * cap);
  (void)hipMalloc(&d_dumps, sizeof(HeapEnt) * (size_t)cap * (n_dumps + 1));
  (void)hipMalloc(&d_sizes, sizeof(int) * (n_dumps + 1));
  (void)hipMalloc(&d_popped, sizeof(int) * n_ops);
  (void)hipMemcpy(d_keys, keys, sizeof(float) * n_ops, hipMemcpyHostToDevice);
  (void)hipMemset(d_dumps, 0, sizeof(HeapEnt) * (size_t)cap * (n_dumps + 1));
  if (minq)
    hipLaunchKernelGGL(replay_kernel<true>, dim3(1), dim3(64), (size_t)lds_cap * 8, 0, d_keys, n_ops, lds_cap, d_glob,
                       d_dumps, cap, dump_every, d_sizes, d_popped);
  else
    hipLaunchKernelGGL(replay_kernel<false>, dim3(1), dim3(64), (size_t)lds_cap * 8, 0, d_keys, n_ops, lds_cap, d_glob,
                       d_dumps, cap, dump_every, d_sizes, d_popped);
  int rc = hipDeviceSynchronize() == hipSuccess ? 0 : 2;
  std::vector<HeapEnt> host((size_t)cap * n_dumps);
  (void)hipMemcpy(host.data(), d_dumps, sizeof(HeapEnt) * host.size(), hipMemcpyDeviceToHost);
  for (size_t i = 0; i < host.size(); ++i) {
    dump_keys[i] = host[i].key;
    dump_ids[i] = host[i].id;
  }
  (void)hipMemcpy(sizes, d_sizes, sizeof(int) * n_dumps, hipMemcpyDeviceToHost);
  (void)hipMemcpy(popped, d_popped, sizeof(int) * n_ops, hipMemcpyDeviceToHost);
  (void)hipFree(d_keys); (void)hipFree(d_glob); (void)hipFree(d_dumps); (void)hipFree(d_sizes); (void)hipFree(d_popped);
  return rc;
}
