// Host check of the product's heap emulation (cuhnsw_amd/csrc/heap_emul.h) against
// libstdc++'s std::priority_queue on tie-rich random sequences: after every push and
// pop the two underlying arrays must be identical element for element.
// usage: heap_check <seed> <ops> <key_range>; exit code 0 = identical
#include <cstdio>
#include <cstdlib>
#include <queue>
#include <random>
#include <vector>

#include "heap_emul.h"

using cuhnsw_amd::HeapEnt;
typedef std::pair<float, unsigned> DistId;
struct CompareByFirst {
  bool operator()(const DistId& a, const DistId& b) const noexcept { return a.first < b.first; }
};
struct PQ : std::priority_queue<DistId, std::vector<DistId>, CompareByFirst> {
  const std::vector<DistId>& raw() const { return c; }
};
struct VecAcc {
  std::vector<HeapEnt> v;
  HeapEnt get(int i) const { return v[i]; }
  void set(int i, HeapEnt e) { if ((int)v.size() <= i) v.resize(i + 1); v[i] = e; }
};

template <bool MINQ>
static int run(unsigned seed, int ops, int range) {
  std::mt19937 rng(seed);
  PQ ref;
  VecAcc acc;
  int size = 0;
  for (int t = 0; t < ops; ++t) {
    bool push = ref.empty() || (rng() % 100) < 58;
    if (push) {
      float key = (float)(rng() % range);
      unsigned id = (unsigned)t;
      ref.emplace(MINQ ? -key : key, id);
      cuhnsw_amd::heap_push<MINQ>(acc, size, HeapEnt{key, id});
    } else {
      ref.pop();
      cuhnsw_amd::heap_pop<MINQ>(acc, size);
    }
    if ((int)ref.size() != size) return 1;
    const std::vector<DistId>& r = ref.raw();
    for (int i = 0; i < size; ++i) {
      float k = MINQ ? -r[i].first : r[i].first;
      if (k != acc.v[i].key || r[i].second != acc.v[i].id) {
        std::fprintf(stderr, "mismatch at op %d slot %d\n", t, i);
        return 2;
      }
    }
  }
  return 0;
}

int main(int argc, char** argv) {
  unsigned seed = argc > 1 ? (unsigned)std::atoi(argv[1]) : 1;
  int ops = argc > 2 ? std::atoi(argv[2]) : 20000;
  int range = argc > 3 ? std::atoi(argv[3]) : 16;
  int a = run<false>(seed, ops, range);
  int b = run<true>(seed + 1, ops, range);
  std::printf("max-queue %d min-queue %d\n", a, b);
  return a | b;
}
