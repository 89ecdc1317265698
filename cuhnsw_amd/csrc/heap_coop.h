// Binary heaps that reproduce, move for move, what libstdc++'s
// std::priority_queue<pair<float,unsigned>, vector<...>, CompareByFirst> does
// (std::push_heap / std::pop_heap, bits/stl_heap.h: __push_heap, __adjust_heap),
// executed cooperatively by the 64 lanes of one wavefront.
//
// Why literal: the search must return the ids hnswlib returns, and under equal
// distances hnswlib's answer is a function of the heap's array layout.  Any other
// priority-queue implementation is only equivalent while all keys are distinct.
// (Replaces the thread-0 heap of the reference, cpp/include/cuda_heap_kernels.cuh:13-49.)
//
// Why cooperative: a sift is a chain of dependent LDS reads when one lane does it.
// Here
//   * sift-up (__push_heap): lane j reads the j-th ancestor of the hole, one ballot
//     tells how far the value rises, one masked write shifts the ancestors down and
//     drops the value — one LDS round trip whatever the depth;
//   * sift-down (__adjust_heap): the hole's path always takes the child that is not
//     "less", independent of the value, so 63 lanes evaluate that choice for every
//     node of a 6-level subtree at once (one LDS round trip); a node is on the path if
//     every edge from the subtree root down to it was the chosen one, which each lane
//     tests against a ballot mask, and the lanes on the path move their chosen child
//     up.  Heaps up to 127 entries need one such stage, up to 8191 two.
//
// All functions must be called by all 64 lanes with wavefront-uniform arguments.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cuhnsw_amd {

// Every kernel here runs one wavefront per workgroup, and a wavefront's LDS (and global)
// instructions execute in program order, so lanes exchange data through memory without
// waiting: what is needed between a write by one lane and a read by another is only that
// the compiler keeps their order.  (__syncthreads() would also drain every outstanding
// global access — a full memory round trip per call.)
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

struct __attribute__((aligned(8))) HeapEnt {
  float key;
  uint32_t id;
};

// MINQ = false: max-queue on key (hnswlib top_candidates).
// MINQ = true : hnswlib's candidate_set, a max-queue on (-key); comparing -a < -b is
//               exactly a > b for non-NaN floats, so the key is stored unnegated.
template <bool MINQ>
__device__ __forceinline__ bool heap_less(float a, float b) {
  return MINQ ? (a > b) : (a < b);
}

__device__ __forceinline__ HeapEnt uniform_ent(HeapEnt e) {
  HeapEnt r;
  r.key = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, e.key)));
  r.id = (uint32_t)__builtin_amdgcn_readfirstlane((int)e.id);
  return r;
}

// __push_heap(first, holeIndex = i, topIndex = 0, value = v)
template <bool MINQ, class Acc>
__device__ __forceinline__ void coop_sift_up(Acc& h, int i, HeapEnt v, int lane) {
  wave_sync();
  const int q = lane < 31 ? ((i + 1) >> (lane + 1)) : 0;  // index + 1 of the (lane+1)-th ancestor
  const bool valid = q >= 1;
  HeapEnt e = v;
  if (valid) e = h.get(q - 1);
  const bool rises = valid && heap_less<MINQ>(e.key, v.key);
  const unsigned long long m = __ballot(rises);
  const int t = __builtin_ctzll(~m);  // ancestors passed on the way up
  if (lane <= t) {
    const int slot = ((i + 1) >> lane) - 1;
    h.set(slot, lane < t ? e : v);
  }
  // (the lanes meet again here: merged into a caller's join, the end of the some-lanes store above would make
  // the caller's size count as lane-dependent, and with it every loop over the heap)
  __builtin_amdgcn_wave_barrier();
}

// priority_queue::emplace
template <bool MINQ, class Acc>
__device__ __forceinline__ void coop_push(Acc& h, int& size, HeapEnt v, int lane) {
  coop_sift_up<MINQ>(h, size, v, lane);
  size = size + 1;
}

// per-lane constants of the 63-node stage tree used by coop_pop (lane t = t-th node in
// breadth-first order): the parent's index and the set of edges from the stage root down
// to the lane's node (bit x = edge into node x)
struct StageTree {
  int par;
  unsigned long long anc;
};
__device__ __forceinline__ StageTree make_stage_tree(int lane) {
  StageTree st;
  st.par = lane >= 1 ? ((lane - 1) >> 1) : 0;
  unsigned long long m = 0ull;
  int x = lane < 63 ? lane : 0;
  while (x > 0) {
    m |= 1ull << x;
    x = (x - 1) >> 1;
  }
  st.anc = m;
  return st;
}

// priority_queue::pop.  libstdc++ moves the hole from the root down to a leaf, always into the larger child (the
// right one when the two compare equal), and then lets the former last entry rise from there while its
// parent is smaller.  On the way down every child moved up one level, and along that path the keys do not
// grow: the entries the last one rises past are exactly the path's deepest ones that compare smaller, they end
// up where they were, and nothing below the place the last entry lands in changes at all.  So the way down
// stops at the first moved child that is smaller than the last entry, which is written there -- same array
// as the two loops of libstdc++, one pass, no second look at the path.
template <bool MINQ, class Acc>
__device__ __forceinline__ void coop_pop(Acc& h, int& size, const StageTree& tree, int lane) {
  if (size > 1) {
    wave_sync();
    const int len = size - 1;
    const HeapEnt last_ent = h.get(len);  // (the same in every lane; its read travels with the first stage's)
    // lane t < 63 stands for the t-th node (breadth first) of the subtree under the hole
    const int d = 31 - __clz(lane + 1);
    const int o = lane + 1 - (1 << d);
    int hole = 0;
    for (;;) {
      const int P = ((hole + 1) << d) - 1 + o;
      const int c1 = 2 * P + 1;
      const bool has1 = lane < 63 && c1 < len;
      const bool has2 = lane < 63 && c1 + 1 < len;
      HeapEnt L = last_ent, R = last_ent;
      if (has1) {
        L = h.get(c1);
        R = h.get(c1 + 1);  // c1 + 1 <= len is a valid slot
      }
      const bool take_left = has1 && (!has2 || heap_less<MINQ>(R.key, L.key));
      const unsigned long long mc = __ballot(has1);
      const unsigned long long ml = __ballot(take_left);
      // the edge parent -> this node is taken if the parent has children and chose this side
      // (left children have odd indices); a node is on the hole's path if every edge from the
      // stage root down to it is taken
      const bool edge = lane >= 1 && lane < 63 && ((mc >> tree.par) & 1ull) != 0ull &&
                        (int)((ml >> tree.par) & 1ull) == (lane & 1);
      const unsigned long long me = __ballot(edge);
      const bool on_path = lane < 63 && (me & tree.anc) == tree.anc;
      const unsigned long long mp = __ballot(on_path);
      const HeapEnt child = take_left ? L : R;
      // path nodes whose chosen child is smaller than the last entry (deeper nodes have higher lane numbers)
      const unsigned long long mr = __ballot(on_path && has1 && heap_less<MINQ>(child.key, last_ent.key));
      if (mr != 0ull) {
        const int first = __builtin_ctzll(mr);
        if (on_path && lane <= first) h.set(P, lane < first ? child : last_ent);
        __builtin_amdgcn_wave_barrier();
        break;
      }
      if (on_path && has1) h.set(P, child);
      const int last = 63 - __builtin_clzll(mp);  // deepest node of the path inside this stage
      const int dd = 31 - __clz(last + 1);
      const int last_abs = ((hole + 1) << dd) - 1 + (last + 1 - (1 << dd));
      if (((mc >> last) & 1ull) == 0ull) {
        if (lane == last) h.set(P, last_ent);  // no child: the hole stops here, and so does the last entry
        __builtin_amdgcn_wave_barrier();
        break;
      }
      hole = 2 * last_abs + 2 - (int)((ml >> last) & 1ull);  // its chosen child roots the next stage
      wave_sync();
    }
  }
  size = size - 1;
}

}  // namespace cuhnsw_amd
