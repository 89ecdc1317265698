// Binary heaps that reproduce, move for move, what libstdc++'s
// std::priority_queue<pair<float,unsigned>, vector<...>, CompareByFirst> does
// (std::push_heap / std::pop_heap, bits/stl_heap.h: __push_heap, __adjust_heap).
//
// Why literal: the search must return the ids hnswlib returns, and under equal
// distances hnswlib's answer is a function of the heap's array layout.  Any other
// priority-queue implementation is only equivalent while all keys are distinct.
//
// The code is plain C++ over an accessor (get/set by index) so that the same
// functions run on one GPU lane against LDS (+ a global-memory overflow area) and
// on the host, where a CPU test checks them against std::priority_queue itself.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define HEAP_HD __host__ __device__ __forceinline__
#else
#define HEAP_HD inline
#endif

namespace cuhnsw_amd {

struct __attribute__((aligned(8))) HeapEnt {
  float key;
  uint32_t id;
};

// MINQ = false: max-queue on key (hnswlib top_candidates).
// MINQ = true : hnswlib's candidate_set, a max-queue on (-key); comparing -a < -b
//               is exactly a > b for non-NaN floats, so the key is stored unnegated.
template <bool MINQ>
HEAP_HD bool heap_less(float a, float b) {
  return MINQ ? (a > b) : (a < b);
}

// priority_queue::emplace: push_back, then __push_heap(first, size-1, 0, value)
template <bool MINQ, class Acc>
HEAP_HD void heap_push(Acc& h, int& size, HeapEnt v) {
  int hole = size;
  size = size + 1;
  int parent = (hole - 1) / 2;
  while (hole > 0) {
    HeapEnt p = h.get(parent);
    if (!heap_less<MINQ>(p.key, v.key)) break;
    h.set(hole, p);
    hole = parent;
    parent = (hole - 1) / 2;
  }
  h.set(hole, v);
}

// priority_queue::pop: pop_heap (value = last element, hole walks from the root to
// a leaf always taking the child that is not "less", then the value is pushed up
// from there), then pop_back
template <bool MINQ, class Acc>
HEAP_HD void heap_pop(Acc& h, int& size) {
  if (size > 1) {
    const int len = size - 1;
    HeapEnt value = h.get(len);
    int hole = 0;
    int child = 0;
    while (child < (len - 1) / 2) {
      child = 2 * (child + 1);
      HeapEnt r = h.get(child);
      HeapEnt l = h.get(child - 1);
      if (heap_less<MINQ>(r.key, l.key)) {
        child--;
        r = l;
      }
      h.set(hole, r);
      hole = child;
    }
    if ((len & 1) == 0 && child == (len - 2) / 2) {
      child = 2 * (child + 1);
      h.set(hole, h.get(child - 1));
      hole = child - 1;
    }
    int parent = (hole - 1) / 2;
    while (hole > 0) {
      HeapEnt p = h.get(parent);
      if (!heap_less<MINQ>(p.key, value.key)) break;
      h.set(hole, p);
      hole = parent;
      parent = (hole - 1) / 2;
    }
    h.set(hole, value);
  }
  size = size - 1;
}

}  // namespace cuhnsw_amd
