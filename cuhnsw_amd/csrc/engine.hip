// Host engine and C ABI of libcuhnsw_amd.so.
//
// Counterpart of the reference's host class cuhnsw::CuHNSW
// (cpp/include/cuhnsw.hpp:61-112, cpp/src/cuhnsw_base.cu, cpp/src/cuhnsw_build.cu).
// Differences by design: the whole multi-level index stays resident in HBM in flat
// fixed-stride rows (the reference re-flattens and re-uploads the graph on every
// search call, cpp/src/cuhnsw_build.cu:226-253, and once per upper level for the
// descent, :25-94); there is no per-level host graph container; HIP runtime calls
// are made directly (no Thrust).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/cuhnsw_amd.h"
#include "index_file.h"
#include "kernels.h"
#include "options.h"

namespace cuhnsw_amd {

#define HIP_CHECK(expr)                                                                              \
  do {                                                                                               \
    hipError_t err_ = (expr);                                                                        \
    if (err_ != hipSuccess)                                                                          \
      throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(err_) + " at " #expr); \
  } while (0)

static bool device_present() {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return n > 0;
}

// ---- scratch of the entry point that allocates nothing (cuhnsw_search_knn_device_noalloc) ----------
// Everything the two search kernels need beyond the caller's buffers, at fixed maximum sizes, in one
// array that lives in the code object: each GPU the library runs on holds its own copy from the moment
// the code object is loaded there until the process ends.  Host code never uses the array's name as an
// address (it is a host-side stand-in); the device address is looked up once per device
// (static_scratch_for_current_device) and handed to the kernels like any other buffer.
constexpr int kStaticMaxQueries = 131072;  // entries of the list of queries the first pass gives up
constexpr int kStaticMaxEf = 512;          // the sorted set in registers holds up to 512 entries
constexpr int kStaticSlots = 128;          // wavefronts of the literal pass
constexpr int kStaticGlobCap = 4096;       // per wavefront: overflow of its candidate queue beyond the LDS share
constexpr int kStaticLogCap = 8192;        // per wavefront: log of accepted entries
struct StaticScratch {
  int ctl[128];
  int redo[kStaticMaxQueries];
  HeapEnt cand_glob[(size_t)kStaticSlots * kStaticGlobCap];
  HeapEnt log[(size_t)kStaticSlots * kStaticLogCap];
};
static __device__ __align__(256) unsigned char scratch[sizeof(StaticScratch)];  // 12.5 MB

constexpr int kMaxDevices = 64;
static StaticScratch* g_static_scratch[kMaxDevices] = {};
static std::mutex g_static_scratch_mutex;             // guards the table above
static std::atomic_flag g_static_busy[kMaxDevices];   // set while a no-allocation search uses the device's array
// device address of this device's copy of `scratch`; looked up on first use, then kept
static StaticScratch* static_scratch_for_current_device(int* device = nullptr) {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) throw std::runtime_error("device ordinal beyond the table of static scratch addresses");
  if (device) *device = dev;
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (!g_static_scratch[dev]) {
    void* ptr = nullptr;
    HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    g_static_scratch[dev] = static_cast<StaticScratch*>(ptr);
  }
  return g_static_scratch[dev];
}
// One no-allocation search at a time per GPU: every engine of the process shares that GPU's array.
struct StaticScratchLease {
  int dev;
  explicit StaticScratchLease(int d) : dev(d) {
    if (g_static_busy[dev].test_and_set(std::memory_order_acquire))
      throw std::runtime_error("search_knn (no allocation): another no-allocation search is running on this GPU "
                               "(all engines of a process share the GPU's scratch array; serialise the calls)");
  }
  ~StaticScratchLease() { g_static_busy[dev].clear(std::memory_order_release); }
  StaticScratchLease(const StaticScratchLease&) = delete;
  StaticScratchLease& operator=(const StaticScratchLease&) = delete;
};

// (the no-allocation search clears its control words with this kernel: it issues no memset)
__global__ void __launch_bounds__(128) fill_ints_kernel(int* p, int n, int value) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = value;
}
// Everything a two-pass search needs cleared, in one launch: the control words (0), the list the first pass
// appends to (-1 = "no entry yet", which the literal wavefronts poll for) and, for a batch taken longest
// first, the counters of the counting sort (0).
__global__ void __launch_bounds__(256) prepare_search_kernel(int* ctl, int n_ctl, int* redo, int n_redo, int* hist, int n_hist) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_ctl) ctl[i] = 0;
  if (i < n_redo) redo[i] = -1;
  if (i < n_hist) hist[i] = 0;
}

template <typename T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    n = 0;
  }
  // grows (never shrinks); contents are not preserved
  void reserve(size_t want) {
    if (want <= n) return;
    release();
    HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&p), want * sizeof(T)));
    n = want;
  }
  // the same for a buffer the caller can do without: false (and an empty buffer) when the memory is not there
  bool try_reserve(size_t want) {
    if (want <= n) return true;
    release();
    if (hipMalloc(reinterpret_cast<void**>(&p), want * sizeof(T)) != hipSuccess) {
      (void)hipGetLastError();
      p = nullptr;
      return false;
    }
    n = want;
    return true;
  }
  ~DevBuf() { release(); }
};

class Engine {
 public:
  Options opt;
  int dist_type = DIST_DOT;
  HostIndex host;
  bool have_data = false, have_levels = false, have_graph = false;
  bool host_links_stale = false;  // device links are newer than host.links0 / linksU
  bool has_device = false;
  int num_cus = 0;
  hipStream_t stream = nullptr;
  hipStream_t stream2 = nullptr;  // the literal pass, while the sorted-set pass runs on `stream`
  hipEvent_t ev_side0 = nullptr, ev_side1 = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  std::string err;
  double last_build_seconds = 0.0;

  // tunables
  int level_first = 1;     // build: a batch hands out its nodes with upper levels first
  int build_literal = 0;   // build: 1 = the literal search (queues / sorted list in LDS) whatever ef_construction (tests)
  int build_batch = 0;     // nodes inserted per batch at most; 0 = by the size of the graph (batch_at)
  int search_slots = 0;
  int cand_lds_override = 0;
  int hnswlib_dist = 0;
  int spin_limit_override = -1;  // polls a waiting literal wavefront may spend (-1 = automatic)
  int side_per_cu = 0;         // its wavefronts per CU (0 = from the share of queries the last search gave up)
  bool share_known = false;               // last_repeat_share comes from a search of this index
  double last_repeat_share = 0.0;         // its wavefronts per CU
  int concurrent_literal = 1;  // run the literal pass beside the sorted-set pass (0: after it)
  // A literal wavefront whose bounded wait ran out (the two streams did not run side by side: a profiler that
  // serialises kernels, a saturated device) makes the next kSequentialSearches searches run their passes one
  // after the other; then the concurrent schedule is tried again.  The caller's setting above is left alone.
  static constexpr int kSequentialSearches = 8;
  int sequential_left = 0;       // searches still to run one pass after the other
  int literal_fallbacks = 0;     // how often that happened on this index
  int last_side_by_side = 0;     // the last search ran its literal pass beside the first pass
  bool trails_unavailable = false;  // the trail buffers could not be allocated: searches go on without trails
  int filter_entries = 0;  // entries of the sorted-set search's visited filter (0 = automatic)
  int first_pass_waves = 0;  // wavefronts per CU of the first pass (0 = as many as fit)
  int query_order = 1;     // first pass of 1.5 to 32 rounds of wavefronts: longest queries first (0: caller's order)
  bool fast_suspended = false;  // this index ties too often for the sorted-set search to pay (integer data)
  int lean_literal = 1;  // literal pass: 0 = always the exact visited bitmap, 1 = automatic, 2 = always the LDS filter
  bool storage_half = false;  // vectors live in HBM as fp16 (set before set_data / load_index)
  bool tight_rows = false;    // rows padded to 16-byte chunks only, not to 128-byte lines (set before set_data / load_index)
  int fast_path = 1;     // 0: search with the literal queues only; 1: sorted-set pass first when the batch is
                         // larger than one round of literal wavefronts; 2: always
  int last_repeats = 0;  // queries of the last search that were repeated with the literal queues
  int last_trails = 0;   // how many of them came with the first pass's trail
  int count_build_work = 0;    // count the work of a build on the device (cuhnsw_last_build_counters)
  unsigned long long build_counters[10] = {};
  int last_build_dropped = 0;  // reverse links of the last build that found no room in an inbox
  int keep_link_keys = 0;      // keep the keys stored with the level-0 links after a build (debugging aid)
  std::vector<float> link_keys0;  // N x max_m0, only with keep_link_keys
  int newcomer_shortcut = 1;  // build: a link row that the selection rule produced is re-selected with the shortcut for newcomers
  int own_links0 = 0;  // links a new node selects for itself on level 0: 0 = max_m0 (as the reference), else min(value, max_m0); hnswlib uses max_m
  int spill_cap = 0;  // first size of the per-slot queue overflow area (0 = automatic); the accept log is twice that
  int visited_cache = 0;  // entries of the LDS visited cache: 0 = automatic, < 0 = none

  // resident index
  int Dp = 0;
  DevBuf<float> d_vectors;
  DevBuf<uint64_t> d_labels;
  DevBuf<uint32_t> d_deleted;  // one bit per element: hnswlib's delete marks of a loaded file (used while host.n_deleted > 0)
  DevBuf<uint32_t> d_links0, d_linksU;
  DevBuf<int64_t> d_upper_off;
  DevBuf<int> d_levels;
  // per-wavefront slots
  DevBuf<uint32_t> d_bitmaps, d_undo;
  DevBuf<HeapEnt> d_cand_glob, d_log;
  SlotPool pool{};
  int pool_slots = 0;
  DevBuf<int> d_ctl;  // [0] work counter, [1] status, [2] dirty count, [32] queries given up by the
                      // sorted-set pass, [64] queries it has finished with, [96] work counter of a concurrent literal pass
  DevBuf<int> d_redo;  // their indices
  DevBuf<uint4> d_trail;      // trails of the sorted-set pass: one buffer per wavefront and the spares,
  DevBuf<int4> d_redo_trail;  // and which of them goes with which entry of d_redo
  int trails = 1;             // 0 = the literal pass searches every handed-over query from its entry point
  int trail_cap = 2048;       // records (accepted entries) per trail; a search that outgrows it leaves none
  int trail_spares = 1024;    // hand-overs with a trail per batch; the ones after that leave none
  DevBuf<uint4> d_entry;      // longest queries first: level-0 entry of every query of the batch,
  DevBuf<int> d_order_hist;   // bucket counters,
  DevBuf<int> d_order;        // and the order the first pass takes the queries in
  // staging for the host-pointer search entry point
  DevBuf<float> d_q, d_dist;
  DevBuf<int> d_nns, d_found;
  StaticScratch* static_scratch = nullptr;  // this device's copy (device address)
  int device_ordinal = 0;
  int* h_ctl = nullptr;                     // pinned: control words read back without staging
  long long wall_clock_khz = 100000;        // ticks of wall_clock64() per millisecond

  Engine() {
    has_device = device_present();
    if (has_device) {
      int dev = 0;
      HIP_CHECK(hipGetDevice(&dev));
      hipDeviceProp_t prop;
      HIP_CHECK(hipGetDeviceProperties(&prop, dev));
      num_cus = prop.multiProcessorCount;
      int khz = 0;
      if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) == hipSuccess && khz > 0) wall_clock_khz = khz;
      else (void)hipGetLastError();
      static_scratch = static_scratch_for_current_device(&device_ordinal);
      HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&h_ctl), 64 * sizeof(int), hipHostMallocDefault));
      HIP_CHECK(hipStreamCreate(&stream));
      HIP_CHECK(hipEventCreate(&ev0));
      HIP_CHECK(hipEventCreate(&ev1));
      d_ctl.reserve(128);
      HIP_CHECK(hipStreamCreate(&stream2));
      HIP_CHECK(hipEventCreate(&ev_side0));
      HIP_CHECK(hipEventCreate(&ev_side1));
    }
  }
  ~Engine() {
    if (ev0) (void)hipEventDestroy(ev0);
    if (ev1) (void)hipEventDestroy(ev1);
    if (ev_side0) (void)hipEventDestroy(ev_side0);
    if (ev_side1) (void)hipEventDestroy(ev_side1);
    if (stream2) (void)hipStreamDestroy(stream2);
    if (stream) (void)hipStreamDestroy(stream);
    if (h_ctl) (void)hipHostFree(h_ctl);
  }

  void need_device() const {
    if (!has_device) throw std::runtime_error("no HIP device available: this call needs a GPU");
  }

  int qr() const { return query_regs(Dp); }

  DevIndex dev_index(float* dists0 = nullptr, float* distsU = nullptr) const {
    DevIndex ix;
    ix.vectors = d_vectors.p;
    ix.labels = host.labelled ? d_labels.p : nullptr;
    ix.links0 = d_links0.p;
    ix.linksU = d_linksU.p;
    ix.upper_off = d_upper_off.p;
    ix.levels = d_levels.p;
    ix.dists0 = dists0;
    ix.distsU = distsU;
    ix.half = storage_half ? 1 : 0;
    ix.N = host.N; ix.D = host.D; ix.Dp = Dp; ix.S0 = host.S0; ix.SU = host.SU;
    ix.max_m = host.max_m; ix.max_m0 = host.max_m0; ix.maxlevel = host.maxlevel;
    ix.enterpoint = host.enterpoint;
    return ix;
  }

  // ---- option / data / level plumbing -------------------------------------------------
  int init(const char* path) {
    Options o;
    int dt = DIST_DOT;
    std::string why;
    int rc = load_options(path ? path : "", o, dt, why);
    if (rc == 0) {
      opt = o;
      dist_type = dt;
    }
    err = why;  // empty after a successful call
    return rc;
  }

  // vectors go up as one contiguous copy (a pitched copy from pageable memory crawls row by
  // row); rows that need padding are spread out by a small kernel on the device
  // With fp16 storage the host copy is rounded to the stored values first: everything downstream
  // (the saved file, a CPU search of that file) then sees exactly the vectors the kernels see.
  void upload_vectors() {
    Dp = padded_dims(host.D, tight_rows);
    const size_t n = (size_t)host.N;
    if (storage_half) {
      for (float& x : host.vectors) x = (float)(_Float16)x;
      d_vectors.reserve((n * Dp + 1) / 2);
      DevBuf<float> raw;
      raw.reserve(n * host.D);
      HIP_CHECK(hipMemcpyAsync(raw.p, host.vectors.data(), n * host.D * sizeof(float), hipMemcpyHostToDevice, stream));
      HIP_CHECK(hipMemsetAsync(d_vectors.p, 0, n * Dp * sizeof(_Float16), stream));
      const long long work = (long long)n * host.D;
      hipLaunchKernelGGL(pad_rows_half_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream, raw.p,
                         reinterpret_cast<_Float16*>(d_vectors.p), (long long)n, host.D, Dp);
      HIP_CHECK(hipGetLastError());
      HIP_CHECK(hipStreamSynchronize(stream));
      return;
    }
    d_vectors.reserve(n * Dp);
    if (Dp == host.D) {
      HIP_CHECK(hipMemcpyAsync(d_vectors.p, host.vectors.data(), n * Dp * sizeof(float), hipMemcpyHostToDevice, stream));
      HIP_CHECK(hipStreamSynchronize(stream));
      return;
    }
    DevBuf<float> raw;
    raw.reserve(n * host.D);
    HIP_CHECK(hipMemcpyAsync(raw.p, host.vectors.data(), n * host.D * sizeof(float), hipMemcpyHostToDevice, stream));
    HIP_CHECK(hipMemsetAsync(d_vectors.p, 0, n * Dp * sizeof(float), stream));
    const long long work = (long long)n * host.D;
    hipLaunchKernelGGL(pad_rows_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream, raw.p, d_vectors.p,
                       (long long)n, host.D, Dp);
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipStreamSynchronize(stream));
  }

  void set_data(const float* data, int n, int d) {
    if (!data || n <= 0 || d <= 0) throw std::runtime_error("set_data: empty data");
    host = HostIndex();
    host.N = n;
    host.D = d;
    host.vectors.assign(data, data + (size_t)n * d);
    have_levels = have_graph = host_links_stale = false;
    forget_search_history();
    pool_slots = 0;  // the slot pool is sized by N: rebuild it lazily
    pool = SlotPool{};
    if (has_device) upload_vectors();  // without a GPU only the host-side calls remain usable
    have_data = true;
  }

  void upload_structure() {
    d_levels.reserve((size_t)host.N);
    d_upper_off.reserve((size_t)host.N);
    d_links0.reserve((size_t)host.N * host.S0);
    d_linksU.reserve(std::max<size_t>((size_t)host.upper_rows * host.SU, 1));
    HIP_CHECK(hipMemcpyAsync(d_levels.p, host.levels.data(), (size_t)host.N * 4, hipMemcpyHostToDevice, stream));
    HIP_CHECK(hipMemcpyAsync(d_upper_off.p, host.upper_off.data(), (size_t)host.N * 8, hipMemcpyHostToDevice, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
  }
  void upload_links() {
    HIP_CHECK(hipMemcpyAsync(d_links0.p, host.links0.data(), host.links0.size() * 4, hipMemcpyHostToDevice, stream));
    if (!host.linksU.empty())
      HIP_CHECK(hipMemcpyAsync(d_linksU.p, host.linksU.data(), host.linksU.size() * 4, hipMemcpyHostToDevice, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
  }
  void download_links() {
    HIP_CHECK(hipMemcpyAsync(host.links0.data(), d_links0.p, host.links0.size() * 4, hipMemcpyDeviceToHost, stream));
    if (!host.linksU.empty())
      HIP_CHECK(hipMemcpyAsync(host.linksU.data(), d_linksU.p, host.linksU.size() * 4, hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    host_links_stale = false;
  }

  void set_random_levels(const int* levels, int n) {
    if (!have_data) throw std::runtime_error("set_random_levels: call set_data first");
    if (n != host.N) throw std::runtime_error("set_random_levels: length differs from the number of data rows");
    host.max_m = opt.max_m;
    host.max_m0 = opt.max_m0;
    host.M = opt.max_m;
    host.ef_construction = opt.ef_construction;
    host.mult = opt.level_mult;
    host.set_levels(levels, n);
    host.layout_links();
    host.labelled = false;
    host.labels.clear();
    host.deleted.clear();  // a graph built anew holds every element
    host.n_deleted = 0;
    have_levels = true;
    have_graph = false;
    if (has_device) upload_structure();
  }

  // What a search learns about an index (how many of its queries tie, whether the two passes ran side by
  // side) belongs to that index: forgotten whenever another one takes its place.
  void forget_search_history() {
    fast_suspended = false;
    share_known = false;
    last_repeat_share = 0.0;
    sequential_left = 0;
    literal_fallbacks = 0;
    last_side_by_side = 0;
    last_repeats = last_trails = 0;
  }

  // Buffers of a search that do not depend on the batch are allocated when the index becomes resident, not
  // inside the first search that wants them: the trails of the sorted-set pass (one buffer per wavefront the
  // GPU can hold plus the spares).  They are an optimisation: if the memory is not there the searches go on
  // without trails.
  size_t trail_records_wanted(int slots) const { return (size_t)(slots + trail_spares) * (size_t)trail_cap; }
  void reserve_trails(int slots) {
    if (!trails || trails_unavailable) return;
    if (!d_trail.try_reserve(trail_records_wanted(slots))) trails_unavailable = true;
  }
  void prepare_search_buffers() {
    if (!has_device) return;
    trails_unavailable = false;
    reserve_trails(28 * num_cus);  // seven wavefronts per SIMD: what the sorted-set pass holds at most where it keeps trails
  }

  // ---- slots -----------------------------------------------------------------------------
  void ensure_pool(int slots, int cand_glob_cap, int log_cap) {
    const int words = (host.N + 31) / 32;
    const int undo_cap = std::min(32768, std::max(host.N, 64));
    if (slots <= pool_slots && words == pool.bitmap_words && cand_glob_cap <= pool.cand_glob_cap &&
        log_cap <= pool.log_cap && undo_cap == pool.undo_cap)
      return;
    slots = std::max(slots, pool_slots);
    cand_glob_cap = std::max(cand_glob_cap, pool.cand_glob_cap);
    log_cap = std::max(log_cap, pool.log_cap);
    d_bitmaps.release();
    d_bitmaps.reserve((size_t)slots * words);
    HIP_CHECK(hipMemsetAsync(d_bitmaps.p, 0, (size_t)slots * words * 4, stream));
    d_undo.reserve((size_t)slots * undo_cap);
    d_cand_glob.reserve((size_t)slots * cand_glob_cap);
    d_log.reserve((size_t)slots * log_cap);
    pool.log = d_log.p;
    pool.log_cap = log_cap;
    pool.bitmaps = d_bitmaps.p;
    pool.bitmap_words = words;
    pool.undo = d_undo.p;
    pool.undo_cap = undo_cap;
    pool.cand_glob = d_cand_glob.p;
    pool.cand_glob_cap = cand_glob_cap;
    pool_slots = slots;
  }
  // a failed kernel may leave bits set: start over with clean bitmaps
  void scrub_pool() {
    HIP_CHECK(hipMemsetAsync(d_bitmaps.p, 0, (size_t)pool_slots * pool.bitmap_words * 4, stream));
  }

  // slots of sorted result keys per lane: the result set lives in registers while
  // ef < 64 * NS; 0 selects the literal LDS heap for larger ef
  static int key_slots(int ef) { return ef <= 128 ? 2 : (ef < 320 ? 5 : (ef <= 512 ? 8 : (ef < 1024 ? 16 : 0))); }

  // LDS entries of the candidate queue.  With the result keys in registers the queue is the
  // only large LDS user: 2*ef entries hold it in nearly every query (the rest spills to the
  // slot's global area) and keep ~30 wavefronts per CU resident at ef = 300.
  int auto_cand_lds(int ef, int ns, int floor_entries, size_t fixed_bytes) const {
    if (cand_lds_override > 0) return std::max(cand_lds_override, floor_entries);
    if (ns > 0) return std::max(floor_entries, std::min(std::max(2 * ef, 128), 1024));
    const size_t budget = 10240;  // ~16 resident wavefronts per CU out of 160 KB LDS
    size_t used = fixed_bytes + (size_t)(ef + 1) * 8;
    int c = used < budget ? (int)((budget - used) / 8) : 0;
    return std::max(c, std::max(floor_entries, 128));
  }

  // log2 entries of the LDS visited cache (16-bit tags: usable while N >> bits fits 16 bits
  // with 0xFFFF to spare)
  int auto_vc_bits() const {
    if (visited_cache < 0) return 0;
    int want = visited_cache > 0 ? visited_cache : 1024;
    int bits = 8;
    while ((1 << bits) < want && bits < 14) ++bits;
    if (((unsigned)host.N >> bits) >= 0xFFFFu) return 0;
    return bits;
  }

  // log2 of the size in 32-bit words (two 16-bit tags each; a set is two words, four ways) of
  // the LDS visited filter of the sorted-set search.  A search at ef = 300 evaluates 1 100 to
  // 1 300 distinct nodes on the million-point sets (max_m0 24 and 32 alike), about 800 at
  // ef = 100; the filter gets 4 * ef + 512 entries rounded up to a power of two (1 024 up to
  // ef = 128, 2 048 = 4 KB up to ef = 384), and twice as much when a repeated evaluation is
  // expensive (rows of 2 KB and more).  More costs occupancy and is slower, less repeats more.
  // 0 when ids do not fit the tags.
  int auto_fc_bits(int ef) const {
    long long want = filter_entries > 0 ? filter_entries : 4ll * ef + 512;
    if (filter_entries <= 0 && Dp >= 512) want *= 2;
    int bits = 8;
    while ((2ll << bits) < want && bits < 13) ++bits;
    if (((unsigned)host.N >> (bits - 1)) >= 0xFFFFu) return 0;  // tags are 16 bits wide, sets 64
    return bits;
  }

  template <typename K>
  int resident_slots(K kernel, size_t lds) const {
    int per_cu = 0;
    HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 64, lds));
    per_cu = std::max(1, std::min(per_cu, 32));
    return per_cu * num_cus;
  }

  // ---- search ------------------------------------------------------------------------------
  // Two passes: every query on the sorted set in registers (search_fast_kernel); the queries
  // in which equal keys met, and every query when ef exceeds the set's capacity, with the
  // literal priority queues (search_kernel).  The literal pass normally runs at the same time
  // on a second stream, on one wavefront per SIMD, and picks the given-up queries off a list
  // as the first pass appends them; should it report a problem (its bounded wait ran out, or a
  // queue overflowed) the list is answered again after the first pass.  ms covers everything.
  template <int DT, int QR, int NS>
  void launch_search(const DevIndex& ix, SearchArgs& a, int max_slots_override, float* ms) {
    a.counter = d_ctl.p;
    a.status = d_ctl.p + 1;
    a.repeats = d_ctl.p + 32;   // the counters of the two passes sit in separate 128-byte lines
    a.done = d_ctl.p + 64;
    a.redo = nullptr;
    a.live = 0;
    a.nq_total = a.nq;
    a.slot_base = 0;
    // a literal wavefront beside the first pass waits at most 2 ms for that pass to start (it is launched
    // microseconds later unless something serialises the two streams) and accepts no progress of a
    // started first pass for 100 ms (its queries finish every few microseconds)
    a.spin_limit = spin_limit_override;
    a.start_ticks = 2 * wall_clock_khz;
    a.stall_ticks = 100 * wall_clock_khz;
    a.nq_dev = nullptr;
    a.entry = nullptr;
    a.order_hist = nullptr;
    a.order = nullptr;
    a.trail = nullptr;
    a.redo_trail = nullptr;
    a.trail_next = nullptr;
    a.trail_cap = a.trail_first_spare = a.trail_spares = 0;
    last_repeats = 0;
    last_trails = 0;
    if (use_static) {
      launch_search_static<DT, QR, NS>(ix, a, ms);
      return;
    }
    HIP_CHECK(hipEventRecord(ev0, stream));
    // the literal pass runs on the sorted set with ids and the LDS filter (no bitmap) unless the
    // caller asked for literal queues only, which also means exact evaluation counters
    // ...and unless the visited bitmaps of the wavefronts at work fit the L2 caches (32 MB) together:
    // there the bitmap's atomics are cheap and the literal search with them is the faster one
    const size_t bitmap_bytes = (size_t)std::min(num_cus * 24, a.nq) * ((host.N + 31) / 32) * 4;
    const bool want_lean = lean_literal == 1 ? bitmap_bytes > ((size_t)32 << 20) : lean_literal > 1;
    a.lean = (NS > 0 && fast_path != 0 && want_lean) ? auto_fc_bits(a.ef) : 0;
    if (a.lean && filter_entries <= 0) {
      // a batch of few queries leaves most of each CU's LDS unused: give the filter what is there
      // (up to 32 KB), so that it forgets next to nothing
      const int per_cu = (a.nq + num_cus - 1) / num_cus;
      const size_t room = per_cu > 0 ? (size_t)(150 * 1024) / per_cu : 0;
      const size_t other = plan_lds(QR, ix.Dp, NS > 0 ? -1 : a.ef, a.cand_lds, a.lcap, 0, 0, 0, 0, 0).total + 256;
      while (a.lean < 13 && other + ((size_t)4 << (a.lean + 1)) <= std::min<size_t>(room, 60 * 1024) &&
             (((unsigned)host.N >> a.lean) < 0xFFFFu))
        ++a.lean;
    }
    const LdsPlan lp = plan_lds(QR, ix.Dp, NS > 0 ? -1 : a.ef, a.cand_lds, a.lcap, 0, 0, a.lean ? 0 : a.vc_bits, 0, a.lean);
    auto kernel = search_kernel<DT, QR, NS>;
    int lit_slots = resident_slots(kernel, lp.total);
    if (max_slots_override > 0) lit_slots = max_slots_override;
    int glob_cap = spill_cap > 0 ? spill_cap : std::max(4096, 8 * a.ef);
    int n_literal = a.nq;
    bool answered = false;
    bool timed = false;  // ev1 has been recorded after the last kernel of this search
    // A batch that fits the machine in one round of literal wavefronts is latency-bound: where the literal
    // search has its exact bitmaps, two passes would only add the second pass's latency to the first's, and
    // the literal pass answers alone.  Where the bitmaps do not fit the L2 (the literal search then runs on
    // the sorted set with the LDS filter) the first pass is the same search without the literal candidate
    // queue, and the faster choice even with a hand-over.
    // (Long rows — the query in LDS — go to the first pass whatever the batch: there the literal search takes twice
    // the first pass's time per expanded candidate, 2.0 against 1.0 ms for a single query on 1 M x 960.)
    if (NS > 0 && a.fast_path && a.fc_bits > 0 &&
        (a.fast_path > 1 || a.nq > lit_slots || (a.lean && a.nq > 1) || QR == 0)) {  // (reverse_cand: fast_path is 2)
      d_redo.reserve((size_t)a.nq);
      a.redo = d_redo.p;
      auto fast_kernel = search_fast_kernel<DT, QR, NS, false>;
      auto fast_lds = [&](int bits) -> size_t { return plan_fast_lds(QR, ix.Dp, a.lcap, bits).total; };
      auto fast_slots = [&](int bits) -> int { return resident_slots(fast_kernel, fast_lds(bits)); };
      // the filter must not be what limits the wavefronts per CU: half the filter repeats more
      // evaluations but is the faster choice wherever it buys 15 % more wavefronts
      while (filter_entries <= 0 && a.fc_bits > 9) {
        const int now = fast_slots(a.fc_bits);
        const int with_half = fast_slots(a.fc_bits - 1);
        if (with_half * 20 < now * 23) break;  // less than 15 % more
        --a.fc_bits;
      }
      const size_t fast_lds_bytes = fast_lds(a.fc_bits);
      int slots = fast_slots(a.fc_bits);
      const bool side = concurrent_literal && sequential_left == 0 && max_slots_override <= 0;
      last_side_by_side = side ? 1 : 0;
      int side_slots = 0;
      // few queries need the literal pass: one wavefront per CU serves them without taking room from
      // the first pass; two when the last search handed over 2 % and more (a literal wavefront's LDS
      // is that of one and a half wavefronts of the first pass, so more of them cost more than they serve)
      const int per_cu = side_per_cu > 0 ? side_per_cu : (last_repeat_share < 0.02 ? 1 : 2);
      if (side) {
        side_slots = std::min(num_cus * per_cu, a.nq);
        // an index that hands over next to nothing (the last search: under one query in a thousand) gets one
        // literal wavefront per four CUs, and the first pass the room of the others
        if (side_per_cu <= 0 && share_known && last_repeat_share < 0.001) side_slots = std::min(std::max(num_cus / 4, 1), a.nq);
        ensure_pool(std::max(side_slots, 1), glob_cap, 2 * glob_cap);
        slots = std::max(num_cus, slots - std::min(side_slots, num_cus * per_cu));  // leave the literal wavefronts their room
      }
      if (max_slots_override > 0) slots = max_slots_override;
      if (first_pass_waves > 0) slots = std::min(slots, first_pass_waves * num_cus);
      slots = std::max(1, std::min(slots, a.nq));
      // (every allocation before the literal pass is launched: growing a buffer frees the old one, and
      // hipFree waits for the device, on which that pass would be waiting for the first pass to start)
      const long long resident = slots;  // queries at work at a time
      // A handed-over query is not searched again from its entry point: the first pass leaves the entries it
      // accepted, hop by hop, and the literal pass (on the sorted set with ids: it needs no visited bitmap
      // brought up to date) replays its queue operations from them up to where the two may part.  One query per
      // wavefront, link rows of one pass of 64 lanes, and batches of under three rounds of wavefronts: keeping
      // the trail costs the first pass 9 % (the kernel instance with the trail code 4 %, writing the records the
      // rest), which only a batch short enough to wait for its last hand-over gets back.  trails = 2: whatever
      // the batch.
      bool keep_trails = (QR == 1 || QR == 2) && trails && !a.reverse && a.lean && host.S0 <= 63 &&
                         (trails > 1 || 4 * (long long)a.nq <= 11 * resident);
      if (keep_trails) {
        // (normally there since the index became resident; a changed trail_cap / trail_spares asks again)
        if (d_trail.n < trail_records_wanted(slots)) {
          trails_unavailable = false;
          reserve_trails(slots);
        }
        keep_trails = !trails_unavailable && d_trail.n >= trail_records_wanted(slots);
      }
      // (with trails a late hand-over costs less, and the order pays from one round on)
      const bool in_order = query_order && (query_order > 1 ? a.nq > resident
                                                             : (keep_trails ? a.nq > resident : 2 * a.nq >= 3 * resident) &&
                                                                   a.nq <= 32 * resident);
      if (in_order) {
        d_entry.reserve((size_t)a.nq);
        d_order.reserve((size_t)a.nq);
        d_order_hist.reserve((size_t)kOrderBuckets);
      }
      if (keep_trails) {
        d_redo_trail.reserve((size_t)a.nq);
        a.trail = d_trail.p;
        a.trail_cap = trail_cap;
        a.trail_first_spare = slots;
        a.trail_spares = trail_spares;
        a.trail_next = d_ctl.p + 48;
        a.redo_trail = d_redo_trail.p;
      }
      {
        const int n_hist = in_order ? kOrderBuckets : 0;
        const int n_fill = std::max(std::max(a.nq, n_hist), 128);
        hipLaunchKernelGGL(prepare_search_kernel, dim3((unsigned)((n_fill + 255) / 256)), dim3(256), 0, stream, d_ctl.p, 128,
                           d_redo.p, a.nq, in_order ? d_order_hist.p : nullptr, n_hist);
        HIP_CHECK(hipGetLastError());
      }
      if (side) {
        SearchArgs b = a;
        b.live = 1;
        b.entry = in_order ? d_entry.p : nullptr;  // (a query reaches that pass after the batch's descents are done)
        b.counter = d_ctl.p + 96;
        b.pool = pool;
        // one or two of these wavefronts per CU: LDS for a candidate queue that never spills costs the first
        // pass nothing (the queue of a long search outgrows 2 * ef entries)
        if (NS > 0) b.cand_lds = std::max(a.cand_lds, 1024);
        const LdsPlan lp_side = plan_lds(QR, ix.Dp, NS > 0 ? -1 : a.ef, b.cand_lds, a.lcap, 0, 0, a.lean ? 0 : a.vc_bits, 0, a.lean);
        // (the first pass starts after the batch's descents when its queries are put in order: 0.1 ms per
        // 10 000 queries of the 1.18 M x 50 set; allow ten times that on top of the usual 2 ms)
        b.start_ticks += (long long)wall_clock_khz * (a.nq / 10000 + 1);
        HIP_CHECK(hipEventRecord(ev_side0, stream));
        HIP_CHECK(hipStreamWaitEvent(stream2, ev_side0, 0));
        hipLaunchKernelGGL(kernel, dim3(side_slots), dim3(64), lp_side.total, stream2, ix, b);
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipEventRecord(ev_side1, stream2));
      }
      // more than one round of wavefronts: the batch's descents first, then its queries longest first.  (The
      // literal pass has been launched by now: launched after the first pass it would find no room until the
      // first of that pass's wavefronts leave, a third of the way through the batch.)
      if (in_order) {
        a.entry = d_entry.p;
        a.order = d_order.p;
        a.order_hist = d_order_hist.p;
        if constexpr (QR == 1 || QR == 2) {
          // four queries per wavefront, one per group of 16 lanes
          auto k_entry = entry4_kernel<DT, QR>;
          const int entry_grid = std::max(1, std::min((a.nq + 3) / 4, resident_slots(k_entry, 0)));
          hipLaunchKernelGGL(k_entry, dim3(entry_grid), dim3(64), 0, stream, ix, a);
        } else {
          auto k_entry = entry_kernel<DT, QR>;
          const size_t entry_lds = plan_fast_lds(QR, ix.Dp, a.lcap, 0).total;
          const int entry_grid = std::max(1, std::min(a.nq, resident_slots(k_entry, entry_lds)));
          hipLaunchKernelGGL(k_entry, dim3(entry_grid), dim3(64), entry_lds, stream, ix, a);
        }
        HIP_CHECK(hipGetLastError());
        hipLaunchKernelGGL(order_prefix_kernel, dim3(1), dim3(1024), 0, stream, d_order_hist.p);
        HIP_CHECK(hipGetLastError());
        hipLaunchKernelGGL(order_scatter_kernel, dim3((unsigned)((a.nq + 1023) / 1024)), dim3(1024), 0, stream, d_entry.p,
                           a.nq, d_order_hist.p, d_order.p);
        HIP_CHECK(hipGetLastError());
      }
      if constexpr (QR == 1 || QR == 2) {
        if (keep_trails) hipLaunchKernelGGL((search_fast_kernel<DT, QR, NS, true>), dim3(slots), dim3(64), fast_lds_bytes, stream, ix, a);
        else hipLaunchKernelGGL(fast_kernel, dim3(slots), dim3(64), fast_lds_bytes, stream, ix, a);
      } else {
        hipLaunchKernelGGL(fast_kernel, dim3(slots), dim3(64), fast_lds_bytes, stream, ix, a);
      }
      HIP_CHECK(hipGetLastError());
      if (side) {
        HIP_CHECK(hipStreamWaitEvent(stream, ev_side1, 0));
      }
      HIP_CHECK(hipEventRecord(ev1, stream));  // (recorded again further down if the list has to be answered after all)
      timed = true;
      int* ctl = h_ctl;  // pinned: read back without a staging copy
      HIP_CHECK(hipMemcpyAsync(ctl, d_ctl.p, 49 * sizeof(int), hipMemcpyDeviceToHost, stream));
      HIP_CHECK(hipStreamSynchronize(stream));
      n_literal = last_repeats = ctl[32];
      last_trails = ctl[48];
      last_repeat_share = (double)n_literal / a.nq;
      share_known = true;
      if (!side && sequential_left > 0) --sequential_left;
      // an index whose distances tie all the time (integer-valued data) sends most queries
      // through both passes: stop trying the sorted set on it
      if (a.nq >= 256 && (long long)n_literal * 3 > a.nq) fast_suspended = true;
      if (side) {
        answered = ctl[1] == 0;
        if (!answered) {
          scrub_pool();
          if (ctl[1] & 1) glob_cap *= 4;
          // the wait ran out: the streams of this process do not run side by side at present (a profiler
          // collecting counters, a saturated device); the next searches run one pass after the other
          if (ctl[1] & 2) {
            sequential_left = kSequentialSearches;
            ++literal_fallbacks;
          }
        }
      }
    }
    if (n_literal > 0 && !answered) {
      timed = false;
      SearchArgs b = a;
      b.nq = n_literal;
      int slots = std::max(1, std::min(lit_slots, b.nq));
      bool done = false;
      for (int attempt = 0; attempt < 8 && !done; ++attempt) {
        ensure_pool(slots, glob_cap, 2 * glob_cap);
        b.pool = pool;
        HIP_CHECK(hipMemsetAsync(d_ctl.p, 0, 3 * sizeof(int), stream));
        hipLaunchKernelGGL(kernel, dim3(slots), dim3(64), lp.total, stream, ix, b);
        HIP_CHECK(hipGetLastError());
        int ctl[2];
        HIP_CHECK(hipMemcpyAsync(ctl, d_ctl.p, sizeof(ctl), hipMemcpyDeviceToHost, stream));
        HIP_CHECK(hipStreamSynchronize(stream));
        done = ctl[1] == 0;
        if (!done) {
          scrub_pool();
          glob_cap *= 4;  // a candidate queue or accept log overflowed its global area: retry with more room
        }
      }
      if (!done) throw std::runtime_error("search: candidate queue overflow");
    }
    if (!timed) {
      HIP_CHECK(hipEventRecord(ev1, stream));
      HIP_CHECK(hipEventSynchronize(ev1));
    }
    if (ms) HIP_CHECK(hipEventElapsedTime(ms, ev0, ev1));
  }
  // The search of the entry point that allocates nothing: the sorted-set pass over every query, then the
  // literal pass over the list it left, one after the other on the engine's stream.  The length of the
  // list stays on the device (the literal kernel reads it there), so nothing is read back in between;
  // control words, list and the literal wavefronts' queue overflow and log areas live in this device's
  // copy of the static scratch array.  No hipMalloc, no hipFree, no memset: a fill kernel clears the
  // control words, the list needs no clearing (the pass after reads only the entries the count vouches
  // for).  Calls that overlap on one GPU would share the array and race.
  template <int DT, int QR, int NS>
  void launch_search_static(const DevIndex& ix, SearchArgs& a, float* ms) {
    if constexpr (NS > 0) {
      StaticScratchLease lease(device_ordinal);  // released on every way out of this function
      StaticScratch* sc = static_scratch;
      a.counter = sc->ctl;
      a.status = sc->ctl + 1;
      a.repeats = sc->ctl + 32;
      a.done = sc->ctl + 64;
      a.redo = sc->redo;
      a.fast_path = 2;
      a.lean = a.fc_bits;  // literal searches keep the LDS filter and the sorted set with ids: no bitmap in HBM
      auto kernel = search_kernel<DT, QR, NS>;
      auto fast_kernel = search_fast_kernel<DT, QR, NS, false>;
      while (filter_entries <= 0 && a.fc_bits > 9) {  // (as in the allocating search: the filter must not cost occupancy)
        const int now = resident_slots(fast_kernel, plan_fast_lds(QR, ix.Dp, a.lcap, a.fc_bits).total);
        const int with_half = resident_slots(fast_kernel, plan_fast_lds(QR, ix.Dp, a.lcap, a.fc_bits - 1).total);
        if (with_half * 20 < now * 23) break;
        --a.fc_bits;
      }
      const FastLdsPlan fp = plan_fast_lds(QR, ix.Dp, a.lcap, a.fc_bits);
      const LdsPlan lp = plan_lds(QR, ix.Dp, -1, a.cand_lds, a.lcap, 0, 0, 0, 0, a.lean);
      const int slots = std::max(1, std::min(resident_slots(fast_kernel, fp.total), a.nq));
      const int lit_slots = std::max(1, std::min(std::min(resident_slots(kernel, lp.total), kStaticSlots), a.nq));
      HIP_CHECK(hipEventRecord(ev0, stream));
      hipLaunchKernelGGL(fill_ints_kernel, dim3(1), dim3(128), 0, stream, sc->ctl, 128, 0);
      HIP_CHECK(hipGetLastError());
      hipLaunchKernelGGL(fast_kernel, dim3(slots), dim3(64), fp.total, stream, ix, a);
      HIP_CHECK(hipGetLastError());
      SearchArgs b = a;
      b.nq = 0;
      b.nq_dev = sc->ctl + 32;
      b.counter = sc->ctl + 96;
      b.pool = SlotPool{};
      b.pool.cand_glob = sc->cand_glob;
      b.pool.cand_glob_cap = kStaticGlobCap;
      b.pool.log = sc->log;
      b.pool.log_cap = kStaticLogCap;
      hipLaunchKernelGGL(kernel, dim3(lit_slots), dim3(64), lp.total, stream, ix, b);
      HIP_CHECK(hipGetLastError());
      HIP_CHECK(hipEventRecord(ev1, stream));
      HIP_CHECK(hipMemcpyAsync(h_ctl, sc->ctl, 33 * sizeof(int), hipMemcpyDeviceToHost, stream));
      HIP_CHECK(hipStreamSynchronize(stream));
      last_repeats = h_ctl[32];
      if (ms) HIP_CHECK(hipEventElapsedTime(ms, ev0, ev1));
      if (h_ctl[1] != 0)
        throw std::runtime_error("search_knn (no allocation): a literal search outgrew its share of the static scratch "
                                 "(candidate queue or accept log); use cuhnsw_search_knn_device for this batch");
    } else {
      (void)ix; (void)a; (void)ms;
      throw std::runtime_error("search_knn (no allocation): ef_search beyond the sorted set's capacity");
    }
  }

  template <int DT, int QR>
  void launch_search_ns(int ns, const DevIndex& ix, SearchArgs& a, float* ms) {
    switch (ns) {
      case 2: launch_search<DT, QR, 2>(ix, a, search_slots, ms); break;
      case 5: launch_search<DT, QR, 5>(ix, a, search_slots, ms); break;
      case 8: launch_search<DT, QR, 8>(ix, a, search_slots, ms); break;
      case 16: launch_search<DT, QR, 16>(ix, a, search_slots, ms); break;
      default: launch_search<DT, QR, 0>(ix, a, search_slots, ms); break;
    }
  }
  template <int DT>
  void launch_search_qr(int q, int ns, const DevIndex& ix, SearchArgs& a, float* ms) {
    switch (q) {
      case 1: launch_search_ns<DT, 1>(ns, ix, a, ms); break;
      case 2: launch_search_ns<DT, 2>(ns, ix, a, ms); break;
      case 4: launch_search_ns<DT, 4>(ns, ix, a, ms); break;
      default: launch_search_ns<DT, 0>(ns, ix, a, ms); break;
    }
  }

  bool use_static = false;  // the running search is the one that allocates nothing

  void search_device(const float* d_qdata, int nq, int k, int ef, int* d_nns_out, float* d_dist_out, int* d_found_out,
                     int* d_stats, float* ms, bool no_alloc = false) {
    need_device();
    if (!have_graph) throw std::runtime_error("search_knn: no index (call build_graph or load_index first)");
    if (nq <= 0) return;
    if (k <= 0) throw std::runtime_error("search_knn: topk must be positive");
    ef = std::max(ef, k);
    use_static = no_alloc;
    if (no_alloc) {
      if (nq > kStaticMaxQueries)
        throw std::runtime_error("search_knn (no allocation): at most " + std::to_string(kStaticMaxQueries) + " queries per call");
      if (ef > kStaticMaxEf)
        throw std::runtime_error("search_knn (no allocation): max(topk, ef_search) must not exceed " + std::to_string(kStaticMaxEf));
      if (auto_fc_bits(ef) == 0)
        throw std::runtime_error("search_knn (no allocation): the index has too many points for the LDS visited filter");
    }
    DevIndex ix = dev_index();
    SearchArgs a{};
    a.q = d_qdata; a.nq = nq; a.k = k; a.ef = ef;
    a.nns = d_nns_out; a.dists = d_dist_out; a.found = d_found_out; a.stats = d_stats;
    a.hnswlib_dist = hnswlib_dist;
    a.lcap = (std::max(std::max(host.S0, host.SU), std::max(k, 64)) + 63) / 64 * 64;
    const int q = qr();
    size_t fixed = (size_t)a.lcap * 8 + (q == 0 ? (size_t)query_lds_chunks(Dp) * 16 : 0);
    int ns = key_slots(ef);
    a.vc_bits = auto_vc_bits();
    a.fast_path = no_alloc ? 2 : (fast_suspended ? 0 : fast_path);
    a.reverse = opt.reverse_cand ? 1 : 0;
    // An index with deleted elements (hnswlib's marks in a loaded file) is searched by hnswlib's rule for them:
    // walked through, never returned.  Only the search on the literal queues in LDS states that rule; it takes
    // every query of such an index.
    if (host.n_deleted > 0) {
      if (no_alloc) throw std::runtime_error("search_knn (no allocation): the index holds deleted elements");
      if (a.reverse) throw std::runtime_error("search_knn: reverse_cand is not defined on an index with deleted elements");
      ns = 0;
      a.fast_path = 0;
      a.deleted = d_deleted.p;
    }
    // reverse_cand: the sorted set in registers expands its farthest entry; beyond its capacity (ef >= 1024) the
    // literal pass does, on a sorted list in LDS
    if (a.reverse) a.fast_path = ns > 0 ? 2 : 0;
    if (a.reverse && no_alloc && ns == 0) throw std::runtime_error("search_knn (no allocation): reverse_cand needs ef_search below 1024");
    a.fc_bits = (ns > 0 && a.fast_path) ? auto_fc_bits(ef) : 0;
    if (a.reverse && ns > 0 && a.fc_bits == 0)
      throw std::runtime_error("search_knn: reverse_cand needs fewer than 2^28 points");
    // with the keys in registers the queue's LDS share doubles as result buffer (lcap entries,
    // then lcap label slots) and as the replay heap (ef + 1 entries)
    const int floor_entries = ns > 0 ? std::max(ef + 1, 2 * a.lcap) : std::max(k, 64);
    a.cand_lds = auto_cand_lds(ef, ns, floor_entries, fixed);
    if (dist_type == DIST_DOT) launch_search_qr<DIST_DOT>(q, ns, ix, a, ms);
    else launch_search_qr<DIST_L2>(q, ns, ix, a, ms);
  }

  void search_host(const float* q, int nq, int k, int ef, int* nns, float* dists, int* found) {
    need_device();
    if (nq <= 0) return;
    if (!q || !nns || !dists || !found) throw std::runtime_error("search_knn: null argument");
    if (k <= 0) throw std::runtime_error("search_knn: topk must be positive");
    d_q.reserve((size_t)nq * host.D);
    d_nns.reserve((size_t)nq * k);
    d_dist.reserve((size_t)nq * k);
    d_found.reserve((size_t)nq);
    HIP_CHECK(hipMemcpyAsync(d_q.p, q, (size_t)nq * host.D * 4, hipMemcpyHostToDevice, stream));
    search_device(d_q.p, nq, k, ef, d_nns.p, d_dist.p, d_found.p, nullptr, nullptr);
    HIP_CHECK(hipMemcpyAsync(nns, d_nns.p, (size_t)nq * k * 4, hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipMemcpyAsync(dists, d_dist.p, (size_t)nq * k * 4, hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipMemcpyAsync(found, d_found.p, (size_t)nq * 4, hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
  }

  // ---- build ---------------------------------------------------------------------------------
  template <int DT, int QR, int NS>
  void build_levels() {
    const int N = host.N;
    const int cap_in = 32;
    const int bmax = build_batch > 0 ? build_batch : std::min(std::max(N, 1), 65536);
    const int m_max = std::max(host.max_m, host.max_m0);
    const size_t up_rows = std::max<size_t>((size_t)host.upper_rows, 1);
    DevBuf<float> d_dists0, d_distsU, d_sel0_keys, d_selU_keys;
    DevBuf<uint32_t> d_sel0_ids, d_selU_ids;
    DevBuf<unsigned long long> d_dirty;
    DevBuf<int> d_sel0_cnt, d_selU_cnt, d_inbox0_cnt, d_inboxU_cnt;
    DevBuf<HeapEnt> d_inbox0, d_inboxU;
    DevBuf<unsigned char> d_selected;  // per link row: the row is an output of the selection rule (kernels.h, BuildArgs)
    d_dists0.reserve((size_t)N * host.S0);
    d_distsU.reserve(up_rows * host.SU);
    d_sel0_ids.reserve((size_t)bmax * host.max_m0);
    d_sel0_keys.reserve((size_t)bmax * host.max_m0);
    d_sel0_cnt.reserve((size_t)bmax);
    d_selU_ids.reserve(up_rows * host.max_m);
    d_selU_keys.reserve(up_rows * host.max_m);
    d_selU_cnt.reserve(up_rows);
    // a batch node posts at most max_m0 links on level 0 and max_m on each upper level
    d_dirty.reserve((size_t)bmax * ((size_t)host.max_m0 + (size_t)std::max(host.maxlevel, 1) * host.max_m));
    d_inbox0.reserve((size_t)N * cap_in);
    d_inbox0_cnt.reserve((size_t)N);
    d_inboxU.reserve(up_rows * cap_in);
    d_inboxU_cnt.reserve(up_rows);
    if (newcomer_shortcut) {
      d_selected.reserve((size_t)N + up_rows);
      HIP_CHECK(hipMemsetAsync(d_selected.p, 0, (size_t)N + up_rows, stream));
    }
    HIP_CHECK(hipMemsetAsync(d_inbox0_cnt.p, 0, (size_t)N * 4, stream));
    HIP_CHECK(hipMemsetAsync(d_inboxU_cnt.p, 0, up_rows * 4, stream));
    HIP_CHECK(hipMemsetAsync(d_links0.p, 0xFF, (size_t)N * host.S0 * 4, stream));
    if (host.upper_rows > 0) HIP_CHECK(hipMemsetAsync(d_linksU.p, 0xFF, (size_t)host.upper_rows * host.SU * 4, stream));

    DevIndex ix = dev_index(d_dists0.p, d_distsU.p);
    auto k_search = build_search_kernel<DT, QR, NS>;
    auto k_reverse = reverse_kernel<DT, QR>;
    const int efc = opt.ef_construction;
    const int glob_cap = std::max(4096, 8 * efc);

    BuildArgs a{};
    a.efc = efc;
    // (the reference multiplies in single precision: `const int nn_num = max_m * heuristic_coef` with a
    // float coefficient, cpp/include/cuda_build_kernels.cuh:77,101)
    a.nn_num0 = (int)((float)host.max_m0 * (float)opt.heuristic_coef);
    a.nn_numU = (int)((float)host.max_m * (float)opt.heuristic_coef);
    a.save_remains = opt.save_remains ? 1 : 0;
    a.reverse = opt.reverse_cand ? 1 : 0;
    a.own_cap0 = own_links0 > 0 ? std::min(own_links0, host.max_m0) : host.max_m0;
    a.sel0_ids = d_sel0_ids.p; a.sel0_keys = d_sel0_keys.p; a.sel0_cnt = d_sel0_cnt.p;
    a.selU_ids = d_selU_ids.p; a.selU_keys = d_selU_keys.p; a.selU_cnt = d_selU_cnt.p;
    a.counter = d_ctl.p; a.status = d_ctl.p + 1;
    a.inbox0 = d_inbox0.p; a.inbox0_cnt = d_inbox0_cnt.p;
    a.inboxU = d_inboxU.p; a.inboxU_cnt = d_inboxU_cnt.p;
    a.cap_in = cap_in;
    a.dirty = d_dirty.p; a.dirty_cnt = d_ctl.p + 2;
    a.dropped = d_ctl.p + 3;
    a.selected0 = newcomer_shortcut ? d_selected.p : nullptr;
    a.selectedU = newcomer_shortcut ? d_selected.p + N : nullptr;
    DevBuf<unsigned long long> d_work;
    if (count_build_work) {
      d_work.reserve(10);
      HIP_CHECK(hipMemsetAsync(d_work.p, 0, 10 * sizeof(unsigned long long), stream));
    }
    a.counters = d_work.p;
    const int s_max = std::max(host.S0, host.SU);
    a.lcap = (std::max(s_max, 64) + 63) / 64 * 64;
    size_t fixed = (size_t)a.lcap * 8 + (size_t)efc * 8 + (size_t)m_max * 8 + 64 +
                   (QR == 0 ? (size_t)query_lds_chunks(Dp) * 16 : 0);
    a.fc_bits = NS > 0 ? auto_fc_bits(efc) : 0;
    const bool sorted_set = NS > 0 && a.fc_bits > 0;  // then neither queue nor literal cache is needed
    if (a.reverse && NS > 0 && !sorted_set) throw std::runtime_error("build_graph: reverse_cand needs fewer than 2^28 points");
    a.cand_lds = sorted_set ? 0 : auto_cand_lds(efc, NS, 64, fixed);
    a.vc_bits = sorted_set ? 0 : auto_vc_bits();
    const LdsPlan lp1 = plan_lds(QR, Dp, sorted_set ? -1 : efc, a.cand_lds, a.lcap, efc, m_max, a.vc_bits, a.fc_bits);
    const LdsPlan lp3 = plan_lds(QR, Dp, s_max + cap_in, 0, a.lcap, s_max + cap_in, std::max(m_max, cap_in));
    const int slots1 = resident_slots(k_search, lp1.total);
    const int slots3 = resident_slots(k_reverse, lp3.total);
    // the sorted-set search needs no per-wavefront global memory (no bitmap, no undo list, no log)
    if (!sorted_set) ensure_pool(slots1, glob_cap, 2 * glob_cap);
    a.pool = pool;

    // Nodes go in by ascending id, as hnswlib inserts them.  The graph a batch sees is the
    // one of all earlier batches: its entry point is the first node that reached the highest
    // level so far.  Batches grow with the graph — a quarter of what is already in, up to 16 384 nodes, so
    // that early nodes, which wire the long-range links, see each other; beyond half a million nodes a
    // thirty-second of the graph, up to 65 536 — because the nodes of a batch do not see each other (recall
    // falls when the share of new nodes grows), and a launch of several rounds of wavefronts loses less to
    // its last, partly filled round.
    // build_batch > 0 replaces the two caps by one.
    auto batch_at = [&](int in) {
      if (build_batch > 0) return std::max(1, std::min(build_batch, in / 4));
      return std::max(1, std::min(in / 4, std::max(16384, std::min(65536, in / 32))));
    };
    // within a batch the nodes with upper levels are handed out first (highest level first, then by id)
    DevBuf<int> d_order;
    {
      std::vector<int> order((size_t)N);
      for (int p0 = 0; p0 < N;) {
        const int b = std::min(batch_at(p0), N - p0);
        int* o = order.data() + p0;
        int n_up = 0;
        for (int i = 0; i < b; ++i)
          if (host.levels[p0 + i] > 0) o[n_up++] = i;
        std::stable_sort(o, o + n_up, [&](int x, int y) { return host.levels[p0 + x] > host.levels[p0 + y]; });
        for (int i = 0, w = n_up; i < b; ++i)
          if (host.levels[p0 + i] <= 0) o[w++] = i;
        p0 += b;
      }
      d_order.reserve((size_t)N);
      HIP_CHECK(hipMemcpyAsync(d_order.p, order.data(), (size_t)N * sizeof(int), hipMemcpyHostToDevice, stream));
      HIP_CHECK(hipStreamSynchronize(stream));
    }
    a.order = level_first ? d_order.p : nullptr;
    int cur_ep = 0, cur_max = -1;
    int pos = 0;
    while (pos < N) {
      int b = batch_at(pos);
      b = std::min(b, N - pos);
      a.begin = pos;
      a.count = b;
      a.cur_ep = cur_ep;
      a.cur_max = cur_max;
      // counter and dirty count back to zero; the status word is sticky
      HIP_CHECK(hipMemsetAsync(d_ctl.p, 0, sizeof(int), stream));
      HIP_CHECK(hipMemsetAsync(d_ctl.p + 2, 0, sizeof(int), stream));
      hipLaunchKernelGGL(k_search, dim3(std::min(b, slots1)), dim3(64), lp1.total, stream, ix, a);
      HIP_CHECK(hipGetLastError());
      if (cur_max >= 0) {
        long long work = (long long)b * m_max;
        hipLaunchKernelGGL(apply_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream, ix, a);
        HIP_CHECK(hipGetLastError());
        hipLaunchKernelGGL(k_reverse, dim3((unsigned)std::min<long long>(work, slots3)), dim3(64), lp3.total, stream, ix, a);
        HIP_CHECK(hipGetLastError());
      }
      for (int i = pos; i < pos + b; ++i)
        if (host.levels[i] > cur_max) {
          cur_max = host.levels[i];
          cur_ep = i;
        }
      pos += b;
    }
    int ctl[4];
    HIP_CHECK(hipMemcpyAsync(ctl, d_ctl.p, sizeof(ctl), hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    if (ctl[1] != 0) {
      scrub_pool();
      throw std::runtime_error("build_graph: candidate queue overflow");
    }
    last_build_dropped = ctl[3];
    std::memset(build_counters, 0, sizeof(build_counters));
    if (count_build_work) {
      HIP_CHECK(hipMemcpyAsync(build_counters, d_work.p, sizeof(build_counters), hipMemcpyDeviceToHost, stream));
      HIP_CHECK(hipStreamSynchronize(stream));
    }
    if (keep_link_keys) {
      // debugging aid: the key stored with every level-0 link, for a validator to recompute
      std::vector<float> strided((size_t)N * host.S0);
      HIP_CHECK(hipMemcpyAsync(strided.data(), d_dists0.p, strided.size() * 4, hipMemcpyDeviceToHost, stream));
      HIP_CHECK(hipStreamSynchronize(stream));
      link_keys0.assign((size_t)N * host.max_m0, 0.f);
      for (int i = 0; i < N; ++i)
        std::memcpy(&link_keys0[(size_t)i * host.max_m0], &strided[(size_t)i * host.S0], (size_t)host.max_m0 * 4);
    }
  }

  template <int DT, int QR>
  void build_ns(int ns) {
    switch (ns) {
      case 2: build_levels<DT, QR, 2>(); break;
      case 5: build_levels<DT, QR, 5>(); break;
      case 8: build_levels<DT, QR, 8>(); break;
      case 16: build_levels<DT, QR, 16>(); break;
      default: build_levels<DT, QR, 0>(); break;
    }
  }
  template <int DT>
  void build_qr(int q, int ns) {
    switch (q) {
      case 1: build_ns<DT, 1>(ns); break;
      case 2: build_ns<DT, 2>(ns); break;
      case 4: build_ns<DT, 4>(ns); break;
      default: build_ns<DT, 0>(ns); break;
    }
  }

  void build_graph() {
    need_device();
    if (!have_data || !have_levels) throw std::runtime_error("build_graph: call set_data and set_random_levels first");
    HIP_CHECK(hipMemsetAsync(d_ctl.p, 0, 4 * sizeof(int), stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    auto t0 = std::chrono::steady_clock::now();
    const int q = qr();
    const int ns = build_literal ? 0 : key_slots(opt.ef_construction);
    if (dist_type == DIST_DOT) build_qr<DIST_DOT>(q, ns);
    else build_qr<DIST_L2>(q, ns);
    last_build_seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    have_graph = true;
    forget_search_history();
    prepare_search_buffers();
    host_links_stale = true;
  }

  // ---- measurement aid --------------------------------------------------------------------------------
  // random row gathers over the resident vectors (gather_probe_kernel): returns rows fetched, ms taken
  void gather_probe(int waves_per_cu, int rows_in_flight, int dependent, double* rows, float* ms) {
    need_device();
    if (!have_data) throw std::runtime_error("gather probe: no vectors (call set_data or load_index first)");
    const int waves = std::max(1, std::min(waves_per_cu, 32)) * num_cus;
    const int batches = 2048;
    const int U = rows_in_flight >= 16 ? 4 : (rows_in_flight >= 8 ? 2 : 1);
    DevBuf<float> sink;
    sink.reserve((size_t)waves);
    DevIndex ix = dev_index();
    float best = 0.f;
    for (int it = 0; it < 3; ++it) {
      HIP_CHECK(hipEventRecord(ev0, stream));
      if (U == 4) hipLaunchKernelGGL(gather_probe_kernel<4>, dim3(waves), dim3(64), 0, stream, ix, batches, dependent, sink.p);
      else if (U == 2) hipLaunchKernelGGL(gather_probe_kernel<2>, dim3(waves), dim3(64), 0, stream, ix, batches, dependent, sink.p);
      else hipLaunchKernelGGL(gather_probe_kernel<1>, dim3(waves), dim3(64), 0, stream, ix, batches, dependent, sink.p);
      HIP_CHECK(hipGetLastError());
      HIP_CHECK(hipEventRecord(ev1, stream));
      HIP_CHECK(hipEventSynchronize(ev1));
      float t = 0.f;
      HIP_CHECK(hipEventElapsedTime(&t, ev0, ev1));
      if (it == 0 || t < best) best = t;
    }
    if (rows) *rows = (double)waves * 4.0 * U * batches;
    if (ms) *ms = best;
  }

  // ---- index file --------------------------------------------------------------------------------
  void save_index(const char* path) {
    if (!have_graph) throw std::runtime_error("save_index: no index to save");
    if (host_links_stale) download_links();
    write_index_file(host, path);
  }
  void load_index(const char* path) {
    HostIndex fresh;
    read_index_file(fresh, path);
    if (fresh.N <= 0) throw std::runtime_error("load_index: empty index");
    host = std::move(fresh);
    have_data = have_levels = have_graph = true;
    forget_search_history();
    host_links_stale = false;
    if (has_device) {
      upload_vectors();
      upload_structure();
      upload_links();
      d_labels.reserve((size_t)host.N);
      HIP_CHECK(hipMemcpyAsync(d_labels.p, host.labels.data(), (size_t)host.N * 8, hipMemcpyHostToDevice, stream));
      std::vector<uint32_t> marks;
      if (host.n_deleted > 0) {
        marks.assign(((size_t)host.N + 31) / 32, 0u);
        for (int i = 0; i < host.N; ++i)
          if (host.deleted[i]) marks[(size_t)i >> 5] |= 1u << (i & 31);
        d_deleted.reserve(marks.size());
        HIP_CHECK(hipMemcpyAsync(d_deleted.p, marks.data(), marks.size() * 4, hipMemcpyHostToDevice, stream));
      }
      HIP_CHECK(hipStreamSynchronize(stream));
      pool_slots = 0;  // N may have changed: rebuild the slot pool lazily
      pool = SlotPool{};
      prepare_search_buffers();
    }
  }
};

}  // namespace cuhnsw_amd

// ---------------------------------------------------------------------------------------------- C ABI
using cuhnsw_amd::Engine;

struct cuhnsw_engine {
  Engine impl;
  std::mutex mutex;  // calls on one engine are serialised: they share its staging buffers, slot pool and streams
};

namespace {
thread_local std::string g_create_error;

template <typename F>
int guarded(cuhnsw_engine* e, F&& f) {
  if (!e) return -1;
  std::lock_guard<std::mutex> lock(e->mutex);
  try {
    e->impl.err.clear();
    f(e->impl);
    return 0;
  } catch (const std::exception& ex) {
    e->impl.err = ex.what();
    return -1;
  } catch (...) {
    e->impl.err = "unknown error";
    return -1;
  }
}
}  // namespace

extern "C" {

int cuhnsw_create(cuhnsw_engine** out) {
  if (!out) return -1;
  try {
    *out = new cuhnsw_engine();
    return 0;
  } catch (const std::exception& ex) {
    g_create_error = ex.what();
    *out = nullptr;
    return -1;
  }
}
void cuhnsw_destroy(cuhnsw_engine* e) { delete e; }
const char* cuhnsw_last_error(cuhnsw_engine* e) { return e ? e->impl.err.c_str() : g_create_error.c_str(); }

int cuhnsw_init(cuhnsw_engine* e, const char* opt_path) {
  if (!e) return -1;
  std::lock_guard<std::mutex> lock(e->mutex);
  return e->impl.init(opt_path);
}
int cuhnsw_set_data(cuhnsw_engine* e, const float* data, int num_data, int num_dims) {
  return guarded(e, [&](Engine& g) { g.set_data(data, num_data, num_dims); });
}
int cuhnsw_set_random_levels(cuhnsw_engine* e, const int* levels, int num_levels) {
  return guarded(e, [&](Engine& g) {
    if (!levels) throw std::runtime_error("set_random_levels: null levels");
    g.set_random_levels(levels, num_levels);
  });
}
int cuhnsw_build_graph(cuhnsw_engine* e) { return guarded(e, [&](Engine& g) { g.build_graph(); }); }
int cuhnsw_save_index(cuhnsw_engine* e, const char* fpath) {
  return guarded(e, [&](Engine& g) { g.save_index(fpath ? fpath : ""); });
}
int cuhnsw_load_index(cuhnsw_engine* e, const char* fpath) {
  return guarded(e, [&](Engine& g) { g.load_index(fpath ? fpath : ""); });
}
int cuhnsw_search_knn(cuhnsw_engine* e, const float* qdata, int num_queries, int topk, int ef_search, int* nns,
                      float* distances, int* found_cnt) {
  return guarded(e, [&](Engine& g) { g.search_host(qdata, num_queries, topk, ef_search, nns, distances, found_cnt); });
}
int cuhnsw_search_knn_device(cuhnsw_engine* e, const float* d_qdata, int num_queries, int topk, int ef_search, int* d_nns,
                             float* d_distances, int* d_found_cnt, int* d_stats, float* kernel_ms) {
  return guarded(e, [&](Engine& g) {
    g.search_device(d_qdata, num_queries, topk, ef_search, d_nns, d_distances, d_found_cnt, d_stats, kernel_ms);
  });
}
int cuhnsw_search_knn_device_noalloc(cuhnsw_engine* e, const float* d_qdata, int num_queries, int topk, int ef_search,
                                     int* d_nns, float* d_distances, int* d_found_cnt, float* kernel_ms) {
  return guarded(e, [&](Engine& g) {
    g.search_device(d_qdata, num_queries, topk, ef_search, d_nns, d_distances, d_found_cnt, nullptr, kernel_ms, true);
  });
}
int cuhnsw_debug_gather_probe(cuhnsw_engine* e, int waves_per_cu, int rows_in_flight, int dependent, double* rows,
                              float* ms) {
  return guarded(e, [&](Engine& g) { g.gather_probe(waves_per_cu, rows_in_flight, dependent, rows, ms); });
}
int cuhnsw_last_build_dropped_links(cuhnsw_engine* e) { return e ? e->impl.last_build_dropped : 0; }
int cuhnsw_last_build_counters(cuhnsw_engine* e, unsigned long long* out, int n) {
  if (!e || !out || n < 10) return -1;
  std::memcpy(out, e->impl.build_counters, sizeof(e->impl.build_counters));
  return 0;
}
int cuhnsw_debug_link_keys0(cuhnsw_engine* e, float* out, long long capacity) {
  return guarded(e, [&](Engine& g) {
    if (g.link_keys0.empty()) throw std::runtime_error("link keys were not kept: set tunable keep_link_keys before build_graph");
    if (!out || capacity < (long long)g.link_keys0.size()) throw std::runtime_error("link keys: output buffer too small");
    std::memcpy(out, g.link_keys0.data(), g.link_keys0.size() * sizeof(float));
  });
}
int cuhnsw_num_data(cuhnsw_engine* e) { return e ? e->impl.host.N : 0; }
int cuhnsw_num_dims(cuhnsw_engine* e) { return e ? e->impl.host.D : 0; }
int cuhnsw_max_level(cuhnsw_engine* e) { return e ? e->impl.host.maxlevel : 0; }
int cuhnsw_enter_point(cuhnsw_engine* e) { return e ? (int)e->impl.host.enterpoint : 0; }
int cuhnsw_has_device(void) { return cuhnsw_amd::device_present() ? 1 : 0; }
double cuhnsw_last_build_seconds(cuhnsw_engine* e) { return e ? e->impl.last_build_seconds : 0.0; }
int cuhnsw_num_deleted(cuhnsw_engine* e) { return e ? e->impl.host.n_deleted : 0; }
int cuhnsw_last_search_repeats(cuhnsw_engine* e) { return e ? e->impl.last_repeats : 0; }
int cuhnsw_last_search_trails(cuhnsw_engine* e) { return e ? e->impl.last_trails : 0; }
int cuhnsw_last_search_side_by_side(cuhnsw_engine* e) { return e ? e->impl.last_side_by_side : 0; }
int cuhnsw_literal_fallbacks(cuhnsw_engine* e) { return e ? e->impl.literal_fallbacks : 0; }
int cuhnsw_trails_available(cuhnsw_engine* e) { return e ? (e->impl.trails_unavailable ? 0 : 1) : 0; }
int cuhnsw_set_tunable(cuhnsw_engine* e, const char* name, double value) {
  if (!e || !name) return -1;
  std::lock_guard<std::mutex> lock(e->mutex);
  std::string n(name);
  if (n == "build_batch") e->impl.build_batch = (int)value;
  else if (n == "level_first") e->impl.level_first = (int)value;
  else if (n == "build_literal") e->impl.build_literal = (int)value;
  else if (n == "search_slots") e->impl.search_slots = (int)value;
  else if (n == "cand_lds") e->impl.cand_lds_override = (int)value;
  else if (n == "hnswlib_dist") e->impl.hnswlib_dist = (int)value;
  else if (n == "visited_cache") e->impl.visited_cache = (int)value;
  else if (n == "own_links0") e->impl.own_links0 = (int)value;
  else if (n == "newcomer_shortcut") e->impl.newcomer_shortcut = value != 0.0;
  else if (n == "fast_path") e->impl.fast_path = (int)value;
  else if (n == "lean_literal") e->impl.lean_literal = (int)value;
  else if (n == "trails") e->impl.trails = (int)value;
  else if (n == "trail_cap") e->impl.trail_cap = std::max(1, (int)value);
  else if (n == "trail_spares") e->impl.trail_spares = std::max(0, (int)value);
  else if (n == "filter_entries") e->impl.filter_entries = (int)value;
  else if (n == "query_order") e->impl.query_order = (int)value;
  else if (n == "first_pass_waves") e->impl.first_pass_waves = (int)value;
  else if (n == "concurrent_literal") e->impl.concurrent_literal = value != 0.0;
  else if (n == "literal_spin_limit") e->impl.spin_limit_override = (int)value;
  else if (n == "literal_per_cu") e->impl.side_per_cu = std::max(0, std::min(8, (int)value));
  else if (n == "spill_cap") e->impl.spill_cap = (int)value;
  else if (n == "keep_link_keys") e->impl.keep_link_keys = value != 0.0;
  else if (n == "build_counters") e->impl.count_build_work = value != 0.0;
  else if (n == "tight_rows") {
    if (e->impl.have_data && e->impl.tight_rows != (value != 0.0)) return -2;  // only before the vectors are there
    e->impl.tight_rows = value != 0.0;
  }
  else if (n == "fp16_storage") {
    if (e->impl.have_data && e->impl.storage_half != (value != 0.0)) return -2;  // only before the vectors are there
    e->impl.storage_half = value != 0.0;
  }
  else return -1;
  return 0;
}

}  // extern "C"
