/* C ABI of the MI355X-native HNSW engine (libcuhnsw_amd.so).
 *
 * Every entry point is what a foreign-function binding of the reference's hot
 * path would bind: one call per method of the reference's host class
 * cuhnsw::CuHNSW (cpp/include/cuhnsw.hpp:61-71 in js1010/cuhnsw), which the
 * reference exposes to Python through CuHNSWBind (cuhnsw/bindings.cc:18-72).
 * Plain pointers and sizes only.
 *
 * Conventions
 *   - functions returning int: 0 = success, non-zero = failure; the message is
 *     available from cuhnsw_last_error(engine) (the reference throws
 *     std::runtime_error instead, cpp/include/cuda_base_kernels.cuh:30-37).
 *   - calls are synchronous.  Every call on an engine takes that engine's lock, so calls from several
 *     threads on ONE engine run one after the other (the reference relies on Python's GIL for that,
 *     cuhnsw/bindings.cc has no gil_scoped_release); different engines run side by side.
 *     cuhnsw_last_error reports the last failed call on the engine, whichever thread made it.
 *   - distances: dist_type "dot" -> -<q,x>, "l2" -> squared L2
 *     (cpp/include/cuda_dist_kernels.cuh:112-124).  Candidates are *ordered* by
 *     hnswlib's key (1 - <q,x> for "dot") so that ids equal hnswlib's.
 */
#ifndef CUHNSW_AMD_H_
#define CUHNSW_AMD_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cuhnsw_engine cuhnsw_engine;

/* cuhnsw::CuHNSW::CuHNSW() (cpp/src/cuhnsw_base.cu:13-16).  Works without a GPU
 * (host-side calls: init, load_index, save_index, set_random_levels); every call
 * that needs the device fails with a clear message when none is present. */
int cuhnsw_create(cuhnsw_engine** out);
/* cuhnsw::CuHNSW::~CuHNSW() (cpp/src/cuhnsw_base.cu:64) */
void cuhnsw_destroy(cuhnsw_engine* e);
/* message of the last failed call on this engine ("" if none) */
const char* cuhnsw_last_error(cuhnsw_engine* e);

/* bool CuHNSW::Init(std::string opt_path) (cpp/src/cuhnsw_base.cu:67-106):
 * opt_path names a JSON file holding the option table of
 * cuhnsw/proto/config.proto:10-26.  Returns 0 on success, 1 if the file cannot be
 * read or parsed (the reference returns false), 2 on an invalid dist_type (the
 * reference throws). */
int cuhnsw_init(cuhnsw_engine* e, const char* opt_path);

/* void CuHNSW::SetData(const float* data, int num_data, int num_dims)
 * (cpp/src/cuhnsw_base.cu:108-128).  data: row-major float32 [num_data x
 * num_dims] in host memory.  The engine keeps its own copy (the reference keeps
 * the caller's raw pointer).  Values are expected to be finite: what a search
 * returns for rows that hold infinities or NaNs is not specified. */
int cuhnsw_set_data(cuhnsw_engine* e, const float* data, int num_data, int num_dims);

/* void CuHNSW::SetRandomLevels(const int* levels) (cpp/src/cuhnsw_base.cu:130-156):
 * levels[i] = number of upper levels of node i; num_levels must equal num_data. */
int cuhnsw_set_random_levels(cuhnsw_engine* e, const int* levels, int num_levels);

/* void CuHNSW::BuildGraph() (cpp/src/cuhnsw_build.cu:96-102): builds every level
 * on the GPU; requires set_data + set_random_levels. */
int cuhnsw_build_graph(cuhnsw_engine* e);

/* void CuHNSW::SaveIndex(std::string fpath) (cpp/src/cuhnsw_base.cu:159-247):
 * hnswlib index file format. */
int cuhnsw_save_index(cuhnsw_engine* e, const char* fpath);
/* void CuHNSW::LoadIndex(std::string fpath) (cpp/src/cuhnsw_base.cu:250-365):
 * after it, search returns the file's labels instead of internal ids
 * (cpp/src/cuhnsw_build.cu:284-286).
 * A file written by hnswlib may hold deleted elements (markDelete: bit 0 of the third byte of an element's
 * level-0 count word; the reference reads that word as a plain count, cpp/src/cuhnsw_base.cu:311-312).  They
 * are honoured the way hnswlib's search honours them: walked through, never returned (found_cnt may then be
 * below topk), and cuhnsw_save_index writes the marks back.  Every query of such an index is answered by the
 * search on the literal queues (several times slower than the usual two passes); reverse_cand and
 * cuhnsw_search_knn_device_noalloc fail on it with a message.  cuhnsw_set_random_levels + cuhnsw_build_graph
 * build a new graph over every element and drop the marks. */
int cuhnsw_load_index(cuhnsw_engine* e, const char* fpath);

/* void CuHNSW::SearchGraph(const float* qdata, int num_queries, int topk,
 *   int ef_search, int* nns, float* distances, int* found_cnt)
 * (cpp/src/cuhnsw_build.cu:210-290).  All pointers are host memory, outputs are
 * caller-allocated: nns int32 [num_queries x topk], distances float32
 * [num_queries x topk] ascending, found_cnt int32 [num_queries]; only the first
 * found_cnt[i] entries of a row are defined.  ef_search is raised to topk
 * (cuhnsw/pyhnsw.py:80 does the same before the call). */
int cuhnsw_search_knn(cuhnsw_engine* e, const float* qdata, int num_queries, int topk, int ef_search,
                      int* nns, float* distances, int* found_cnt);

/* Same search with queries and outputs already in device memory (HBM); nothing
 * is copied.  Counterpart of the kernel launch inside CuHNSW::SearchGraph
 * (cpp/src/cuhnsw_build.cu:254-275).  d_stats may be null, else int32
 * [num_queries x 4]: level-0 distance evaluations (performed ones: the first pass may evaluate a
 * node again after its visited filter has forgotten it, and for a query answered from a trail the figure is
 * the first pass's count at the trail's end plus the literal pass's own; exact with tunable fast_path = 0), level-0
 * expanded candidates, upper-level distance evaluations, upper-level sweeps.  The call returns after
 * the kernel has finished; kernel_ms (may be null) receives the kernel's duration
 * measured with HIP events on the engine's stream. */
int cuhnsw_search_knn_device(cuhnsw_engine* e, const float* d_qdata, int num_queries, int topk, int ef_search,
                             int* d_nns, float* d_distances, int* d_found_cnt, int* d_stats, float* kernel_ms);

/* The same search for callers that must not allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc, code that runs beside a stream capture).  The call itself is synchronous and reads its
 * status back: it cannot be recorded into a HIP graph.  It has no counterpart in the reference, whose
 * SearchGraph allocates on every call (cpp/src/cuhnsw_build.cu:238-249).  Neither this call nor
 * anything it runs calls hipMalloc, hipFree or a memset: the scratch memory of its kernels (control
 * words, the list of queries handed from the first pass to the literal pass, the literal wavefronts'
 * queue overflow and accept log) is a fixed 12.5 MB array inside the library's code object, one copy per
 * GPU, held until the process ends.  Limits, each rejected with a message: num_queries <= 131072;
 * max(topk, ef_search) <= 512; fewer than about 2^26 points (the LDS visited filter's 16-bit tags).  A
 * literal search that outgrows its share of the array (4096 queued candidates beyond its LDS queue, 8192
 * accepted entries) makes the call fail; cuhnsw_search_knn_device answers such a batch.  The first pass
 * always runs (tunables fast_path, concurrent_literal and lean_literal do not apply) and the literal pass
 * follows it on the same stream.  All calls on one GPU share the array, so only one of them runs at a time
 * on a GPU: a call that finds another one under way — from another engine or thread of the process —
 * fails at once with a message instead of racing with it.  Same results as cuhnsw_search_knn_device, bit
 * for bit. */
int cuhnsw_search_knn_device_noalloc(cuhnsw_engine* e, const float* d_qdata, int num_queries, int topk, int ef_search,
                                     int* d_nns, float* d_distances, int* d_found_cnt, float* kernel_ms);

/* Introspection used by bindings, tests and the benchmark (the reference keeps
 * the same facts in private members num_data_, num_dims_, max_level_,
 * enter_point_, cpp/include/cuhnsw.hpp:87-108). */
int cuhnsw_num_data(cuhnsw_engine* e);
int cuhnsw_num_dims(cuhnsw_engine* e);
int cuhnsw_max_level(cuhnsw_engine* e);
int cuhnsw_enter_point(cuhnsw_engine* e);
/* elements of the loaded index that carry hnswlib's delete mark (0 for an index built here) */
int cuhnsw_num_deleted(cuhnsw_engine* e);
/* 1 if a HIP device is usable by this process, else 0 */
int cuhnsw_has_device(void);
/* seconds spent inside the last cuhnsw_build_graph (device work, event-timed) */
double cuhnsw_last_build_seconds(cuhnsw_engine* e);
/* Reverse links of the last cuhnsw_build_graph that were not considered because more than 32 nodes of one
 * insertion batch chose the same neighbour on one level; the 32 closest of them (by distance, then id) were,
 * whatever the order the GPU posted them in, so the built graph does not depend on it.  The reference
 * has no such limit: it re-runs its heuristic once per reverse link under a lock
 * (cpp/include/cuda_build_kernels.cuh:294-331).  Sets with hubs reach it: 0 on the 50- and 96-dimensional
 * benchmark configurations, about 12 600 of 25 million links on the 1 M x 128 integer-valued one. */
int cuhnsw_last_build_dropped_links(cuhnsw_engine* e);
/* Measurement aid (no counterpart in the reference): the search's memory access pattern alone.  waves_per_cu
 * wavefronts per CU fetch pseudo-random vector rows of the resident index, 16 lanes per row, rows_in_flight
 * (4, 8 or 16) rows per wavefront at a time; dependent != 0 makes every batch of loads wait for the previous
 * one, as a hop of the search waits for its rows.  rows receives the number of rows fetched, ms the kernel
 * time (best of three): rows x 4 x num_dims / ms is the rate at which this GPU delivers random rows of this
 * index, the ceiling the search's gather phase is measured against. */
int cuhnsw_debug_gather_probe(cuhnsw_engine* e, int waves_per_cu, int rows_in_flight, int dependent, double* rows,
                              float* ms);
/* Work of the last cuhnsw_build_graph, counted on the device when tunable "build_counters" = 1 was set before it
 * (all zero otherwise); the reference counts its visited nodes per level the same way
 * (cpp/src/cuhnsw_build.cu:191-195).  out[0..4] level 0, out[5..9] upper levels: distance evaluations of the
 * searches and descents, link rows read, pair tests of the selection heuristic, candidates the heuristic loaded
 * to test them, link rows written.  n must be at least 10. */
int cuhnsw_last_build_counters(cuhnsw_engine* e, unsigned long long* out, int n);
/* Debugging aid: the key (ordering distance) the build stored with every level-0 link, row-major
 * [num_data x max_m0] in list order, as the reference keeps them in its `distances` array
 * (cpp/include/cuda_build_kernels.cuh:270-278).  Needs tunable "keep_link_keys" = 1 before build_graph. */
int cuhnsw_debug_link_keys0(cuhnsw_engine* e, float* out, long long capacity);
/* number of queries of the last search in which two equal distances met and which were therefore
 * searched a second time with literal hnswlib priority queues (the first pass orders candidates
 * by distance alone, which is exact only without ties; the reference has no such distinction
 * because its kernel does not reproduce hnswlib's tie order) */
int cuhnsw_last_search_repeats(cuhnsw_engine* e);
/* how many of those queries the literal pass did not search from the entry point again: the first pass had
 * left the entries it accepted, hop by hop (its trail), and the literal pass replayed its queue operations
 * from them up to the point where the two searches may part (tunable "trails"; no counterpart in the
 * reference) */
int cuhnsw_last_search_trails(cuhnsw_engine* e);
/* 1 if the last search ran its literal pass beside the first pass (on a second stream), 0 if after it.
 * No counterpart in the reference (one kernel, one stream, cpp/src/cuhnsw_build.cu:254-275). */
int cuhnsw_last_search_side_by_side(cuhnsw_engine* e);
/* How often, since the index became resident, a literal wavefront's bounded wait for the first pass ran out
 * (the two streams were not running side by side: a profiler that serialises kernels, a saturated device).
 * Each time the batch is answered after its first pass instead, and the next 8 searches run their passes one
 * after the other before the side-by-side schedule is tried again; the "concurrent_literal" tunable itself
 * is never changed by the engine. */
int cuhnsw_literal_fallbacks(cuhnsw_engine* e);
/* 1 unless the trail buffers (tunable "trails") could not be allocated; searches then go on without trails */
int cuhnsw_trails_available(cuhnsw_engine* e);
/* tuning knobs that are not part of the reference's option table:
 *   "build_batch"   largest number of nodes inserted per batch (default 0 = by the size of the graph: a quarter
 *                   of the nodes already in, at most 16384; beyond 524288 nodes a thirty-second, at most 65536)
 *   "level_first"   1 (default) = a build batch hands out its nodes with upper levels first (they take several
 *                   searches each, and a launch ends when its last node does); 0 = by id.  Same graph either way.
 *   "build_literal" 1 = the build searches with the literal structures in LDS (two priority queues, or the
 *                   sorted list of reverse_cand) whatever ef_construction — what it does by itself from
 *                   ef_construction 1024 on; same graph as with the sorted set in registers (a testing aid)
 *   "search_slots"  resident wavefronts used by search (0 = automatic)
 *   "cand_lds"      candidate-queue entries kept in LDS (0 = automatic)
 *   "hnswlib_dist"  1 = return hnswlib distances (1-dot) instead of -dot
 *   "visited_cache" entries of the LDS cache in front of the visited bitmap (0 = automatic,
 *                   negative = none)
 *   "spill_cap"     first size (entries) of the per-wavefront queue overflow area; the search
 *                   is repeated with four times the room when it proves too small (0 = automatic)
 *   "fast_path"     0 = search with literal hnswlib priority queues only (exact evaluation
 *                   counters in d_stats); 1 = first pass on the sorted set in registers when the
 *                   batch exceeds one round of resident wavefronts, literal queues for the queries
 *                   that met equal distances (default); 2 = first pass whatever the batch size
 *   "filter_entries" entries of the first pass's LDS visited filter (0 = automatic)
 *   "query_order"   1 (default) = a search batch of 1.5 to 32 rounds of wavefronts (from one round on where the
 *                   first pass keeps trails) does its upper-level descents
 *                   first and takes its queries by descending distance of their level-0 entry point (the longest
 *                   searches first: a launch ends when its last query does); 2 = from more than one round on;
 *                   0 = in the caller's order.  Same answers and counters either way.
 *   "first_pass_waves" wavefronts per CU of the first pass (0 = as many as fit, the default)
 *   "concurrent_literal" 1 = the literal pass runs beside the first pass on a second stream
 *                   (default), 0 = after it
 *   "literal_per_cu" wavefronts per CU of that concurrent literal pass (0 = automatic: 1 or 2
 *                   depending on how many queries the previous search handed over)
 *   "literal_spin_limit" polls one of its wavefronts may spend waiting for the first pass before
 *                   it leaves and the host answers the remaining queries afterwards (-1 = no bound in
 *                   polls: it leaves when the first pass has not started within 2 ms or stalls for
 *                   100 ms; see cuhnsw_literal_fallbacks for what follows)
 *   "build_counters" 1 = count the work of the next builds on the device (cuhnsw_last_build_counters)
 *   "keep_link_keys" 1 = keep the keys stored with the level-0 links after build_graph for
 *                   cuhnsw_debug_link_keys0
 *   "lean_literal"  visited set of the literal-queue pass: 0 = exact bitmap in HBM (one bit per point and
 *                   wavefront), 2 = tag filter in LDS with the sorted set catching repeats, 1 = automatic
 *                   (the bitmap while all bitmaps at work fit the L2 caches; default)
 *   "trails"        1 = the first pass leaves, per query, the entries it accepted hop by hop while its course is
 *                   certainly hnswlib's; the literal pass starts a handed-over query from there instead of from
 *                   the entry point (cuhnsw_last_search_trails counts them).  Needs the literal pass on the tag
 *                   filter (lean_literal), one query per wavefront, link rows under 64 ids, vectors of up to
 *                   128 elements; 270 MB of device memory for 2048 accepted entries per query at work,
 *                   allocated when the index becomes resident (build_graph, load_index) — if that memory is
 *                   not there, searches go on without trails (cuhnsw_trails_available).  Keeping
 *                   the trail costs the first pass 9 %: 1 (default) = for batches of under three rounds of
 *                   wavefronts, which wait for their last hand-over; 2 = for every batch; 0 = off.
 *   "trail_cap"     accepted entries a trail holds (default 2048; a search that accepts more leaves none)
 *   "trail_spares"  handed-over queries per batch that can come with a trail (default 1024: each keeps the
 *                   buffer it was written to until the batch is over; the ones after that come without)
 *   "newcomer_shortcut" 1 (default) = a link row that the selection rule itself produced is re-selected, when
 *                   an insertion batch brings it newcomers, with the reference's new_comer shortcut
 *                   (cpp/include/cuda_build_kernels.cuh:109-138): its old entries are tested only against the
 *                   newcomers picked before them.  Same graph byte for byte, fewer pair tests; 0 = the full
 *                   rule on every re-selection.  Applies with heuristic_coef = 0 and save_remains = false.
 *   "own_links0"    most links a newly inserted node selects for itself on level 0
 *                   (0 = max_m0, as cpp/src/cuhnsw_build.cu:110 does; hnswlib's addPoint uses
 *                   max_m there and max_m0 only as the room for reverse links)
 *   "tight_rows"    1 = vector rows are padded to whole 16-byte chunks only instead of 128-byte lines (D = 50:
 *                   208 instead of 256 bytes per row).  Smaller footprint, rows no longer line-aligned; same
 *                   results.  Has to be set before set_data / load_index (returns -2 afterwards).  Default 0.
 *   "fp16_storage"  1 = the vectors are kept in device memory as fp16 (the reference's switched-off
 *                   HALF_PRECISION idea, cpp/include/types.hpp:9-28).  The index then IS an index over
 *                   the vectors rounded to fp16 (nearest even; magnitudes beyond 65504 become
 *                   infinite): queries and all arithmetic stay fp32, save_index writes the rounded
 *                   vectors, and a CPU search of that file returns the same ids and distances.
 *                   Has to be set before set_data / load_index (returns -2 afterwards).  Default 0.
 * returns -1 for an unknown name */
int cuhnsw_set_tunable(cuhnsw_engine* e, const char* name, double value);

#ifdef __cplusplus
}
#endif
#endif /* CUHNSW_AMD_H_ */
