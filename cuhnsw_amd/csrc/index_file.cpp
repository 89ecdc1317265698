// hnswlib index file reader / writer (byte layout: 96-byte header, N level-0
// records [count | max_m0 ids | D floats | label], then per node a uint32 byte
// size followed by its upper-level link lists).  Same layout as the reference's
// CuHNSW::SaveIndex / LoadIndex (cpp/src/cuhnsw_base.cu:159-365).
#include "index_file.h"

#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>

namespace cuhnsw_amd {

void HostIndex::layout_links() {
  S0 = stride0(max_m0);
  SU = strideU(max_m);
  links0.assign((size_t)N * S0, kEmpty);
  upper_off.assign(N, -1);
  int64_t rows = 0;
  for (int i = 0; i < N; ++i) {
    if (levels[i] > 0) {
      upper_off[i] = rows;
      rows += levels[i];
    }
  }
  upper_rows = rows;
  linksU.assign((size_t)rows * SU, kEmpty);
}

void HostIndex::set_levels(const int* lv, int n) {
  levels.assign(lv, lv + n);
  maxlevel = 0;
  enterpoint = 0;
  for (int i = 0; i < n; ++i) {
    if (lv[i] < 0) throw std::runtime_error("levels must be non-negative");
    if (lv[i] > maxlevel) {
      maxlevel = lv[i];
      enterpoint = (uint32_t)i;
    }
  }
}

namespace {

struct FileCloser {
  void operator()(FILE* f) const { if (f) std::fclose(f); }
};
typedef std::unique_ptr<FILE, FileCloser> File;

struct Header {
  uint64_t offset_level0, max_elements, cur_element_count, size_data_per_element, label_offset, offset_data;
  int32_t maxlevel;
  uint32_t enterpoint;
  uint64_t max_m, max_m0, m;
  double mult;
  uint64_t ef_construction;
};

void wr(FILE* f, const void* p, size_t n) {
  if (n && std::fwrite(p, 1, n, f) != n) throw std::runtime_error("index file: write failed");
}
void rd(FILE* f, void* p, size_t n, const char* what) {
  if (n && std::fread(p, 1, n, f) != n) throw std::runtime_error(std::string("index file: truncated ") + what);
}
constexpr uint32_t kDeleteMark = 0x00010000u;  // hnswlib's DELETE_MARK as a bit of the level-0 count word

int row_degree(const uint32_t* row, int cap) {
  int d = 0;
  while (d < cap && row[d] != kEmpty) ++d;
  return d;
}

}  // namespace

void write_index_file(const HostIndex& ix, const std::string& path) {
  File f(std::fopen(path.c_str(), "wb"));
  if (!f) throw std::runtime_error("cannot open index file for writing: " + path);
  const uint64_t links0_bytes = (uint64_t)ix.max_m0 * 4 + 4;
  const uint64_t linksU_bytes = (uint64_t)ix.max_m * 4 + 4;
  Header h;
  h.offset_level0 = 0;
  h.max_elements = (uint64_t)ix.N;
  h.cur_element_count = (uint64_t)ix.N;
  h.size_data_per_element = links0_bytes + (uint64_t)ix.D * 4 + 8;
  h.label_offset = links0_bytes + (uint64_t)ix.D * 4;
  h.offset_data = links0_bytes;
  h.maxlevel = ix.maxlevel;
  h.enterpoint = ix.enterpoint;
  h.max_m = (uint64_t)ix.max_m;
  h.max_m0 = (uint64_t)ix.max_m0;
  h.m = (uint64_t)ix.M;
  h.mult = ix.mult;
  h.ef_construction = (uint64_t)ix.ef_construction;
  // field by field: the struct has padding-free natural layout here, but the file
  // layout must not depend on that
  wr(f.get(), &h.offset_level0, 8); wr(f.get(), &h.max_elements, 8); wr(f.get(), &h.cur_element_count, 8);
  wr(f.get(), &h.size_data_per_element, 8); wr(f.get(), &h.label_offset, 8); wr(f.get(), &h.offset_data, 8);
  wr(f.get(), &h.maxlevel, 4); wr(f.get(), &h.enterpoint, 4);
  wr(f.get(), &h.max_m, 8); wr(f.get(), &h.max_m0, 8); wr(f.get(), &h.m, 8);
  wr(f.get(), &h.mult, 8); wr(f.get(), &h.ef_construction, 8);

  std::vector<unsigned char> rec(h.size_data_per_element);
  for (int i = 0; i < ix.N; ++i) {
    std::memset(rec.data(), 0, rec.size());  // unused link slots are written as zeros
    const uint32_t* row = &ix.links0[(size_t)i * ix.S0];
    uint32_t deg = (uint32_t)row_degree(row, ix.max_m0);
    if (ix.n_deleted > 0 && ix.deleted[i]) deg |= kDeleteMark;
    std::memcpy(rec.data(), &deg, 4);
    std::memcpy(rec.data() + 4, row, (size_t)(deg & 0xffffu) * 4);
    std::memcpy(rec.data() + h.offset_data, &ix.vectors[(size_t)i * ix.D], (size_t)ix.D * 4);
    uint64_t label = ix.labels.empty() ? (uint64_t)i : ix.labels[i];
    std::memcpy(rec.data() + h.label_offset, &label, 8);
    wr(f.get(), rec.data(), rec.size());
  }
  std::vector<unsigned char> up;
  for (int i = 0; i < ix.N; ++i) {
    uint32_t bytes = (uint32_t)(linksU_bytes * (uint64_t)ix.levels[i]);
    wr(f.get(), &bytes, 4);
    if (!bytes) continue;
    up.assign(bytes, 0);
    for (int l = 1; l <= ix.levels[i]; ++l) {
      const uint32_t* row = &ix.linksU[(size_t)(ix.upper_off[i] + l - 1) * ix.SU];
      uint32_t deg = (uint32_t)row_degree(row, ix.max_m);
      unsigned char* dst = up.data() + (size_t)(l - 1) * linksU_bytes;
      std::memcpy(dst, &deg, 4);
      std::memcpy(dst + 4, row, (size_t)deg * 4);
    }
    wr(f.get(), up.data(), bytes);
  }
  if (std::fflush(f.get()) != 0) throw std::runtime_error("index file: flush failed");
}

void read_index_file(HostIndex& ix, const std::string& path) {
  File f(std::fopen(path.c_str(), "rb"));
  if (!f) throw std::runtime_error("cannot open index file: " + path);
  Header h;
  rd(f.get(), &h.offset_level0, 8, "header"); rd(f.get(), &h.max_elements, 8, "header");
  rd(f.get(), &h.cur_element_count, 8, "header"); rd(f.get(), &h.size_data_per_element, 8, "header");
  rd(f.get(), &h.label_offset, 8, "header"); rd(f.get(), &h.offset_data, 8, "header");
  rd(f.get(), &h.maxlevel, 4, "header"); rd(f.get(), &h.enterpoint, 4, "header");
  rd(f.get(), &h.max_m, 8, "header"); rd(f.get(), &h.max_m0, 8, "header"); rd(f.get(), &h.m, 8, "header");
  rd(f.get(), &h.mult, 8, "header"); rd(f.get(), &h.ef_construction, 8, "header");
  const uint64_t links0_bytes = h.max_m0 * 4 + 4;
  const uint64_t linksU_bytes = h.max_m * 4 + 4;
  if (h.cur_element_count > 0x7fffffffull || h.max_m == 0 || h.max_m0 == 0 || h.max_m > 65535 || h.max_m0 > 65535 ||
      h.offset_data != links0_bytes || h.label_offset <= h.offset_data || (h.label_offset - h.offset_data) % 4 != 0 ||
      h.size_data_per_element != h.label_offset + 8 || h.cur_element_count > h.max_elements || h.maxlevel < 0)
    throw std::runtime_error("index file: inconsistent header");
  ix.N = (int)h.cur_element_count;
  ix.D = (int)((h.label_offset - h.offset_data) / 4);
  ix.max_m = (int)h.max_m;
  ix.max_m0 = (int)h.max_m0;
  ix.M = (int)h.m;
  ix.mult = h.mult;
  ix.ef_construction = (int)h.ef_construction;
  ix.maxlevel = h.maxlevel;
  ix.enterpoint = h.enterpoint;
  if (ix.N > 0 && ix.enterpoint >= (uint32_t)ix.N) throw std::runtime_error("index file: entry point out of range");
  ix.labelled = true;
  ix.vectors.resize((size_t)ix.N * ix.D);
  ix.labels.resize(ix.N);
  ix.levels.assign(ix.N, 0);
  ix.deleted.clear();
  ix.n_deleted = 0;
  const int S0 = HostIndex::stride0(ix.max_m0);
  std::vector<uint32_t> l0((size_t)ix.N * S0, kEmpty);
  std::vector<unsigned char> rec(h.size_data_per_element);
  for (int i = 0; i < ix.N; ++i) {
    rd(f.get(), rec.data(), rec.size(), "level-0 block");
    uint32_t word;
    std::memcpy(&word, rec.data(), 4);
    uint32_t deg = word & 0xffffu;  // hnswlib keeps the count in the low 16 bits, flags above
    // hnswlib's markDelete sets bit 0 of the word's third byte; the other flag bits are unknown and dropped
    // (the reference reads the word as a plain count, cpp/src/cuhnsw_base.cu:311-312, and would index out
    // of its rows)
    if (word & kDeleteMark) {
      if (ix.deleted.empty()) ix.deleted.assign(ix.N, 0);
      ix.deleted[i] = 1;
      ++ix.n_deleted;
    }
    if (deg > (uint32_t)ix.max_m0) throw std::runtime_error("index file: link count above max_m0");
    uint32_t* row = &l0[(size_t)i * S0];
    std::memcpy(row, rec.data() + 4, (size_t)deg * 4);
    for (uint32_t k = 0; k < deg; ++k)
      if (row[k] >= (uint32_t)ix.N) throw std::runtime_error("index file: link id out of range");
    std::memcpy(&ix.vectors[(size_t)i * ix.D], rec.data() + h.offset_data, (size_t)ix.D * 4);
    std::memcpy(&ix.labels[i], rec.data() + h.label_offset, 8);
  }
  if (h.max_elements > h.cur_element_count) {
    uint64_t skip = (h.max_elements - h.cur_element_count) * h.size_data_per_element;
    if (fseeko(f.get(), (off_t)skip, SEEK_CUR) != 0) throw std::runtime_error("index file: truncated level-0 block");
  }
  std::vector<std::vector<uint32_t>> upper(ix.N);
  for (int i = 0; i < ix.N; ++i) {
    uint32_t bytes;
    rd(f.get(), &bytes, 4, "upper block");
    if (!bytes) continue;
    if (bytes % linksU_bytes != 0) throw std::runtime_error("index file: bad upper list size");
    ix.levels[i] = (int)(bytes / linksU_bytes);
    if (ix.levels[i] > ix.maxlevel) throw std::runtime_error("index file: node level above maxlevel");
    upper[i].resize(bytes / 4);
    rd(f.get(), upper[i].data(), bytes, "upper block");
  }
  ix.layout_links();
  ix.links0.swap(l0);
  for (int i = 0; i < ix.N; ++i)
    for (int l = 1; l <= ix.levels[i]; ++l) {
      const uint32_t* src = &upper[i][(size_t)(l - 1) * (1 + ix.max_m)];
      uint32_t deg = src[0] & 0xffffu;
      if (deg > (uint32_t)ix.max_m) throw std::runtime_error("index file: link count above max_m");
      uint32_t* row = &ix.linksU[(size_t)(ix.upper_off[i] + l - 1) * ix.SU];
      for (uint32_t k = 0; k < deg; ++k) {
        if (src[1 + k] >= (uint32_t)ix.N) throw std::runtime_error("index file: link id out of range");
        if (ix.levels[src[1 + k]] < l) throw std::runtime_error("index file: link to a node that lacks that level");
        row[k] = src[1 + k];
      }
    }
  if (ix.N > 0 && ix.levels[ix.enterpoint] < ix.maxlevel) throw std::runtime_error("index file: entry point below maxlevel");
}

}  // namespace cuhnsw_amd
