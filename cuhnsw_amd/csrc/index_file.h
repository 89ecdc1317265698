// Host model of an HNSW index and its hnswlib-compatible file format.
// Replaces CuHNSW::SaveIndex / LoadIndex (cpp/src/cuhnsw_base.cu:159-365 in the
// reference) and the host graph container LevelGraph
// (cpp/include/level_graph.hpp:23-89): adjacency is kept in the same flat,
// fixed-stride rows the GPU uses, so upload and download are plain copies.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace cuhnsw_amd {

constexpr uint32_t kEmpty = 0xFFFFFFFFu;  // unused link slot

struct HostIndex {
  int N = 0, D = 0;
  int max_m = 12, max_m0 = 24, M = 12, ef_construction = 150;
  double mult = 0.0;
  int maxlevel = 0;
  uint32_t enterpoint = 0;
  bool labelled = false;               // labels came from a file
  std::vector<float> vectors;          // N x D
  std::vector<uint64_t> labels;        // N
  std::vector<int> levels;             // N, number of upper levels of a node
  int S0 = 32, SU = 16;                // row strides (uint32 slots) of level 0 / upper levels
  std::vector<uint32_t> links0;        // N x S0, first deg slots hold ids, the rest kEmpty
  std::vector<int64_t> upper_off;      // N: index of the node's level-1 row in linksU, -1 if none
  std::vector<uint32_t> linksU;        // (sum of levels) x SU; row of (node, level) = upper_off[node] + level - 1
  int64_t upper_rows = 0;
  // hnswlib's delete marks (markDelete: bit 0 of the third byte of an element's level-0 count word), one
  // byte per element, or empty when nothing is marked.  A marked element is searched through like any
  // other and never returned.  The reference keeps no such mark: it reads the count word as a plain count
  // (cpp/src/cuhnsw_base.cu:311-312).
  std::vector<uint8_t> deleted;
  int n_deleted = 0;

  static int stride0(int max_m0) { return (max_m0 + 31) / 32 * 32; }
  static int strideU(int max_m) { return (max_m + 15) / 16 * 16; }
  // sizes strides, offsets and empty link tables from N, levels, max_m, max_m0
  void layout_links();
  // max level and entry point from levels: the first node that reaches the
  // maximal level (cpp/src/cuhnsw_base.cu:133-141; node 0 if every level is 0)
  void set_levels(const int* lv, int n);
};

// Both throw std::runtime_error with a message on I/O or format errors.
void write_index_file(const HostIndex& ix, const std::string& path);
void read_index_file(HostIndex& ix, const std::string& path);

}  // namespace cuhnsw_amd
