/*
 * grab_anns.h - C ABI of the MI355X-native GRAB-ANNS hybrid vector index.
 *
 * Plain C, plain pointers and sizes.  Every entry point names the interface of the
 * reference (hxlou/GRAB-ANNS, paths relative to its root) that it stands in for.
 * All functions return GRAB_OK (0) or a GRAB_ERR_* code and never throw; the text of the
 * last error on the calling thread is available from grab_last_error().
 *
 * Two layers, as in the reference:
 *   - stateless functions on DEVICE pointers  (reference: free functions in namespace cagra,
 *     src/index/cagra.cuh, src/index/cagra_opt.cuh, src/index/insert.cuh);
 *   - an index handle taking HOST pointers     (reference: classes cagra::CagraIndex,
 *     cagra::CagraIndexOpt, src/cagraIndex.hpp, src/cagraIndexOpt.cuh).
 * Every call is synchronous on return unless stated otherwise (the reference ends each
 * wrapper in cudaDeviceSynchronize).
 */
#ifndef GRAB_ANNS_H
#define GRAB_ANNS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GRAB_OK 0
#define GRAB_ERR_INVALID 1   /* bad argument (null graph, unsupported dim, degree > 512, ...) */
#define GRAB_ERR_HIP 2       /* a HIP runtime call failed */
#define GRAB_ERR_CAPACITY 3  /* growable buffer: request exceeds the reserved capacity */
#define GRAB_ERR_IO 4        /* file open / magic / version */
#define GRAB_ERR_STATE 5     /* index not built, empty, ... */

#define GRAB_INVALID_ID 0xFFFFFFFFu
#define GRAB_MAX_DEGREE 512 /* src/index/cagra.cuh:24 */

#define GRAB_METRIC_L2 0 /* squared L2, the only metric of the reference */
#define GRAB_METRIC_IP 1 /* extension: score = -dot so that smaller is better */

/* Search flag.  By default the library fixes three defects of the reference search that can
 * only produce wrong answers: seeds bypass de-duplication and the filter
 * (src/index/compute_distance.cuh:237-266), the visited set is rebuilt from the queue before
 * the pending candidates are merged (src/index/search.cu:273-283), and an unfilled result
 * slot is reported as id 2147483647 (src/index/search.cu:351).  With this flag all three
 * behave exactly as in the reference. */
#define GRAB_FLAG_STRICT_REFERENCE 1u
/* Evaluate the filter before the visited-set insert (the reference inserts first,
 * src/index/compute_distance.cuh:560-584).  Rows outside the filter then never occupy the
 * table, so a much smaller hash_bitlen serves a selective filter; the results are the same
 * as long as the table never fills.  Meant for filter kinds that read nothing or little per
 * row (3, 2); with kind 1 every neighbour's timestamp is read (cheaply from rows laid out like
 * the graph: grab_neighbor_timestamps). */
#define GRAB_FLAG_FILTER_FIRST 2u
/* Work decomposition of the search.  Default: one 64-lane wave per query when the batch is
 * large enough to fill the device that way (>= 1024 queries) and a wave needs at most 20 KB
 * of LDS (a visited set of up to 4096 slots), else one workgroup per query (256 threads;
 * 1024 for batches of up to 256 queries).  Both give identical results. */
#define GRAB_FLAG_WAVE_PER_QUERY 4u
#define GRAB_FLAG_BLOCK_PER_QUERY 8u

const char* grab_last_error(void);
/* number of HIP devices visible; 0 when there is no GPU */
int grab_device_count(void);

/* cagra::SearchParams, src/index/cagra.cuh:35-42 */
typedef struct {
    uint32_t itopk_size;
    uint32_t search_width;
    uint32_t min_iterations; /* stored, never read by any kernel (as in the reference) */
    uint32_t max_iterations;
    uint32_t hash_bitlen;
} grab_search_params;

/* cagra::BuildParams, src/index/cagra.cuh:30-33 */
typedef struct {
    uint32_t intermediate_degree;
    uint32_t graph_degree;
} grab_build_params;

/* per-query work counters (debug / bandwidth accounting) */
typedef struct {
    uint64_t iterations;
    uint64_t seed_dists;
    uint64_t parents;
    uint64_t filter_reads;
    uint64_t child_dists;
    uint64_t hash_full;
} grab_counters;

/* ------------------------------------------------------------------------------------------
 * Host-side closed forms.  No GPU needed.
 * ---------------------------------------------------------------------------------------- */
/* cagra::detail::next_power_of_2, src/index/smem_cal.cuh:13-23 */
uint32_t grab_next_power_of_2(uint32_t n);
/* queue capacity rule, src/index/smem_cal.cuh:43-46 and src/index/cagra.cu:871-873 */
uint32_t grab_queue_capacity(uint32_t itopk, uint32_t search_width, uint32_t degree);
/* cagra::detail::calculate_and_check_smem, src/index/smem_cal.cuh:28-76 (the reference's
 * figure, kept for callers that size with it) */
size_t grab_reference_smem_bytes(uint32_t itopk, uint32_t dim, uint32_t search_width,
                                 uint32_t degree, uint32_t hash_bitlen);
/* LDS bytes that this library's workgroup-per-query search kernel uses for the same parameters on batches of more
 * than 256 queries (smaller batches add the scratch of their split merge when it fits beside queue and visited set) */
size_t grab_search_lds_bytes(uint32_t itopk, uint32_t dim, uint32_t search_width,
                             uint32_t degree, uint32_t n_seeds, uint32_t hash_bitlen);

#define GRAB_WRAP_SEARCH 0     /* clamps of cagra::search,             src/index/cagra.cu:862-887 */
#define GRAB_WRAP_SEARCH_OPT 1 /* clamps of cagra::search_opt,         src/index/cagra_opt.cu:1127-1160 */
#define GRAB_WRAP_BUCKET 2     /* clamps of cagra::search_bucket_opt,  src/index/cagra_opt.cu:1241-1276 */
#define GRAB_WRAP_RANGE 3      /* clamps of cagra::search_bucket_range, src/index/cagra_opt.cu:1352-1388 */
/* effective itopk, seed count and queue capacity that the given reference wrapper derives */
void grab_search_plan(int wrapper, uint32_t k, uint32_t itopk_param, uint32_t search_width,
                      uint32_t degree, uint32_t n_provided_seeds, uint32_t* itopk_eff,
                      uint32_t* n_seeds, uint32_t* queue_capacity);

/* ------------------------------------------------------------------------------------------
 * Stateless functions on device pointers.
 * `stream` is a hipStream_t (NULL = the default stream).
 * ---------------------------------------------------------------------------------------- */

/* cagra::search, src/index/cagra.cu:844-935.  rand_xor_mask replaces the std::random_device
 * draw of :885-886 (the reference draws 32 bits and widens them). */
int grab_search(const float* d_dataset, size_t num_dataset, uint32_t dim, const uint32_t* d_graph,
                uint32_t graph_degree, const float* d_queries, int64_t num_queries, int64_t k,
                grab_search_params params, int64_t* d_out_indices, float* d_out_dists,
                const uint32_t* d_seeds, uint32_t num_seeds_per_query, uint64_t rand_xor_mask,
                uint32_t flags, void* stream);

/* cagra::search_opt, src/index/cagra_opt.cu:1108-1210 */
int grab_search_opt(const float* d_dataset, uint32_t dim, size_t num_dataset,
                    const uint32_t* d_graph, uint32_t graph_degree, const float* d_queries,
                    int64_t num_queries, int64_t k, grab_search_params params,
                    int64_t* d_out_indices, float* d_out_dists, const uint32_t* d_seeds,
                    uint32_t num_seeds_per_query, uint64_t rand_xor_mask, uint32_t flags,
                    void* stream);

/* cagra::search_bucket_opt, src/index/cagra_opt.cu:1212-1328: only the first local_degree
 * slots of each adjacency row are followed */
int grab_search_bucket(const float* d_dataset, uint32_t dim, size_t num_dataset,
                       const uint32_t* d_graph, uint32_t total_degree, uint32_t local_degree,
                       const float* d_queries, int64_t num_queries, int64_t k,
                       grab_search_params params, int64_t* d_out_indices, float* d_out_dists,
                       const uint32_t* d_seeds, uint32_t num_seeds_per_query,
                       uint64_t rand_xor_mask, uint32_t flags, void* stream);

/* cagra::search_bucket_range, src/index/cagra_opt.cu:1330-1442: neighbours whose timestamp
 * is outside [start_bucket, end_bucket) are skipped inside the traversal */
int grab_search_range(const float* d_dataset, uint32_t dim, size_t num_dataset,
                      const uint32_t* d_graph, const uint64_t* d_ts, uint32_t total_degree,
                      uint32_t local_degree, const float* d_queries, int64_t num_queries,
                      int64_t k, uint64_t start_bucket, uint64_t end_bucket,
                      grab_search_params params, int64_t* d_out_indices, float* d_out_dists,
                      const uint32_t* d_seeds, uint32_t num_seeds_per_query,
                      uint64_t rand_xor_mask, uint32_t flags, void* stream);

typedef struct grab_entry_layer grab_entry_layer; /* entry-point layer, see grab_entry_layer_create below */

/* General form behind the four wrappers above; also carries what the reference has no
 * signature for: a window per query, a label-set filter, the inner-product metric, work
 * counters and the kernel's own duration. */
typedef struct {
    /* index */
    const float* d_dataset;   /* [num_dataset, dim] row-major fp32 */
    const uint32_t* d_graph;  /* [num_dataset, graph_degree] */
    size_t num_dataset;
    uint32_t dim;             /* multiple of 4 */
    uint32_t graph_degree;
    uint32_t active_degree;   /* slots of each row that are followed (<= graph_degree) */
    int metric;               /* GRAB_METRIC_* */
    /* queries */
    const float* d_queries;   /* [num_queries, dim] */
    size_t num_queries;
    uint32_t k;
    /* plan: already clamped values (see grab_search_plan) */
    uint32_t itopk;
    uint32_t search_width;
    uint32_t max_iterations;
    uint32_t hash_bitlen;
    uint32_t n_seeds;            /* seeds evaluated per query */
    const uint32_t* d_seeds;     /* [num_queries, n_provided] or NULL */
    uint32_t n_provided;
    uint64_t rand_xor_mask;
    /* filter */
    int filter_kind;             /* 0 none, 1 timestamp range, 2 label mask, 3 row-id range
                                  * (d_win_start/d_win_end or win_start/win_end hold id bounds) */
    const uint64_t* d_ts;        /* [num_dataset] */
    const uint64_t* d_win_start; /* [num_queries] when per_query_window, else unused */
    const uint64_t* d_win_end;
    uint64_t win_start;          /* the single window when !per_query_window */
    uint64_t win_end;
    int per_query_window;
    const uint8_t* d_labels;     /* [num_dataset], values 0..63 */
    const uint64_t* d_masks;     /* [num_queries] bit b set = label b allowed */
    uint32_t flags;              /* GRAB_FLAG_* */
    /* outputs */
    int64_t* d_out_indices;      /* [num_queries, k]; -1 for an unfilled slot */
    float* d_out_dists;          /* [num_queries, k] */
    grab_counters* d_counters;   /* [num_queries] or NULL */
    float* kernel_ms;            /* host pointer or NULL: duration of the search kernel (HIP events) */
    void* stream;
    /* optional, filter_kind 1: [num_dataset, graph_degree] timestamps of the neighbours
     * (grab_neighbor_timestamps); NULL = read d_ts[neighbour] */
    const uint64_t* d_graph_ts;
    /* optional (extension): the traversal lists its own seeds from an entry-point layer with groups, made over
     * this base with d_ids_by_ts == NULL and timestamps that never decrease with the row id.  Then filter_kind
     * must be 3, d_win_start/d_win_end (or win_start/win_end) hold TIMESTAMP windows and d_ts the base's
     * timestamps: each wave turns its window into the id interval itself (what grab_windows_to_id_ranges writes)
     * and takes as seeds the in-window members of the groups in d_entry_groups[query] (from
     * grab_entry_layer_probe), nearest group first, until entry_min_rows members are reached - the list
     * grab_entry_layer_list_grouped writes - at most n_seeds (<= 64) of them; d_seeds is not read.  Same results
     * and counters as that call followed by this search with the list as d_seeds.  Rows appended to the base
     * after the layer was made lie outside every interval.  Only the wave-per-query kernel with the queue in
     * registers does this (itopk <= 256, search_width <= 64, no GRAB_FLAG_STRICT_REFERENCE, hash_bitlen <= 15);
     * other shapes are GRAB_ERR_INVALID. */
    const grab_entry_layer* entry_layer;
    const uint32_t* d_entry_groups; /* [num_queries, entry_nprobe] */
    uint32_t entry_nprobe;          /* 1..64 */
    uint32_t entry_min_rows;
    /* optional (extension), filter_kind 3 for timestamps in any order: d_rank[id] = the row's place in ascending
     * timestamp order (the inverse of the permutation that sorts the timestamps, ties in any order).  The interval
     * [start, end) then holds places instead of ids - grab_windows_to_id_ranges over the SORTED timestamps gives
     * them - and the traversal tests d_rank[neighbour]: the answers of filter_kind 1 for 4 bytes per test instead of
     * 8.  d_graph_rank (optional with it, grab_neighbor_ranks): the places of every row's neighbours laid out like
     * the graph, [num_dataset, graph_degree], read as one row next to the adjacency row (register-queue wave kernel
     * under GRAB_FLAG_FILTER_FIRST; the other kernels read d_rank[neighbour]).  Must be rebuilt when the graph or
     * the timestamps change. */
    const uint32_t* d_rank;
    const uint32_t* d_graph_rank;
} grab_search_desc;
int grab_search_ex(const grab_search_desc* desc);
/* Same, but returns as soon as the kernel is queued on desc->stream (unless kernel_ms is asked for):
 * the caller synchronises the stream.  Lets a caller overlap the search of one batch with the
 * seed selection of the next on another stream. */
int grab_search_ex_async(const grab_search_desc* desc);
/* No counterpart in the reference, whose wrappers cudaMalloc per call (src/index/cagra.cu:876-882,
 * src/index/cagra_opt.cu:1146-1151).  For callers that cannot allocate: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  The same search as grab_search_ex_async - same
 * kernels, same results - but it calls no hipMalloc / hipFree / event creation and never waits: when the
 * visited sets do not fit LDS (one workgroup per query with hash_bitlen >= 16, or a queue that leaves the
 * table no room) the per-query tables, which grab_search_ex allocates per call, live in a fixed array of
 * GRAB_STATIC_TABLE_SLOTS uint32 (32 MiB) inside the library's device image; each GPU holds its own copy
 * until the process ends.  num_queries << hash_bitlen beyond that is GRAB_ERR_INVALID, and so is a
 * non-NULL kernel_ms.  The kernel clears the tables it uses, so nothing carries over from call to call;
 * but all calls on one GPU share the one array: two such calls that need it and overlap in time (two
 * streams, two threads) race - keep them on one stream.  The array's address is looked up on the first
 * call on a device (hipGetSymbolAddress), so make that first call outside any capture. */
#define GRAB_STATIC_TABLE_SLOTS (8u << 20)
int grab_search_ex_static(const grab_search_desc* desc);

/* Extension: d_out[row, slot] = d_ts[d_graph[row, slot]] (UINT64_MAX for an empty slot).  With it
 * (grab_search_desc.d_graph_ts) a traversal under filter_kind 1 reads the timestamps of a parent's
 * neighbours as one contiguous row next to the adjacency row, instead of one scattered 8-byte read per
 * neighbour (src/index/compute_distance.cuh:569-584 reads d_ts[neighbor_id] each time).  Same results.
 * Used by the wave-per-query kernel with the queue in registers under GRAB_FLAG_FILTER_FIRST; the other
 * kernels ignore it.  Must be rebuilt when the graph or the timestamps change.  Stream-ordered. */
int grab_neighbor_timestamps(const uint32_t* d_graph, const uint64_t* d_ts, size_t num_dataset,
                             uint32_t graph_degree, uint64_t* d_out, void* stream);

/* Extension: d_out[row, slot] = d_rank[d_graph[row, slot]] (0xFFFFFFFF for an empty slot): grab_neighbor_timestamps
 * for places in timestamp order instead of the timestamps themselves, half the bytes (grab_search_desc.d_graph_rank).
 * Stream-ordered. */
int grab_neighbor_ranks(const uint32_t* d_graph, const uint32_t* d_rank, size_t num_dataset,
                        uint32_t graph_degree, uint32_t* d_out, void* stream);

/* Extension: when timestamps never decrease with the row id (insertion order), a window
 * [start,end) is the id interval [lower_bound(start), lower_bound(end)).  Writes those bounds
 * for filter_kind 3, which tests ids instead of reading a timestamp per visited neighbour
 * (src/index/compute_distance.cuh:569-584 reads d_ts[neighbor_id] each time).
 * Stream-ordered like grab_sample_window_seeds and grab_entry_layer_select: these three only produce
 * device buffers that a search on the same stream consumes, so they return without synchronising. */
int grab_windows_to_id_ranges(const uint64_t* d_ts, size_t num_dataset, const uint64_t* d_win_start,
                              const uint64_t* d_win_end, size_t num_queries, uint64_t* d_lo,
                              uint64_t* d_hi, void* stream);

/* Extension: draws n_seeds ids per query from the ids whose timestamp lies in the query's
 * window (one per stratum of the window; all of them when the window is smaller).  Takes the
 * place of the host-side std::sample over ts_to_ids_ in CagraIndex::query_range,
 * src/cagraIndex.cu:270-295.  d_sorted_ts ascending, d_ids_by_ts the ids in that order. */
int grab_sample_window_seeds(const uint64_t* d_sorted_ts, const uint32_t* d_ids_by_ts, size_t n,
                             const uint64_t* d_win_start, const uint64_t* d_win_end,
                             uint64_t win_start, uint64_t win_end, int per_query_window,
                             size_t num_queries, uint32_t n_seeds, uint64_t seed,
                             uint32_t* d_out_seeds, void* stream);

/* Extension (the reference has no label sets, src/index/search.cu:375-586 filters one bucket): exact top-k for
 * queries that are restricted to sets of buckets, over a base whose rows are stored bucket by bucket (bucket b =
 * rows [h_bucket_offsets[b], h_bucket_offsets[b+1]), at most 64 buckets; bit b of a query's mask admits bucket b).
 * Only the admitted buckets are scanned: every (query, bucket) pair becomes a row of a contraction against that
 * bucket's rows on the matrix cores, candidates are re-scored in the canonical order and a query's partial lists
 * merged by (distance, id) - the same answers as grab_bruteforce_topk with the label-set filter (filter kind 2) on
 * labels that say which bucket a row is in, at the cost of the admitted rows instead of all rows.  Offsets and
 * masks are host arrays; k <= 128.  kernel_ms: the contraction kernel; grab_last_knn_stats / grab_last_knn_bf16_flop
 * give its FLOP, grab_last_knn_exact_rows the queries whose merged candidates proved nothing and were redone row by
 * row. */
int grab_bucket_scan_topk(const float* d_dataset, size_t num_dataset, uint32_t dim, const uint64_t* h_bucket_offsets,
                          uint32_t num_buckets, const float* d_queries, size_t num_queries, uint32_t k, int metric,
                          const uint64_t* h_masks, int64_t* d_out_indices, float* d_out_dists, float* kernel_ms,
                          void* stream);
/* Extension (the reference answers every window through the graph, src/cagraIndex.cu:257-350): exact top-k for
 * queries that are restricted to intervals of row ids, [h_id_lo[q], h_id_hi[q]) - what a timestamp window is when the
 * rows are stored in timestamp order.  Only the admitted rows are scanned: the queries go into a contraction on the
 * matrix cores in the order of their intervals' starts, a tile of 128 queries sweeps the union of their intervals,
 * candidates are re-scored in the canonical order - the same answers as grab_bruteforce_topk with the range filter.
 * For narrow windows, where a graph restricted to the window falls apart, this is both exact and faster than the
 * graph search.  Intervals are host arrays (ends beyond num_dataset are cut, an empty interval yields -1 / the
 * largest distance); k <= 128.  kernel_ms and the statistics as for grab_bucket_scan_topk. */
int grab_window_scan_topk(const float* d_dataset, size_t num_dataset, uint32_t dim, const float* d_queries,
                          size_t num_queries, uint32_t k, int metric, const uint64_t* h_id_lo, const uint64_t* h_id_hi,
                          int64_t* d_out_indices, float* d_out_dists, float* kernel_ms, void* stream);
/* The two scans above over a prepared base (no counterpart in the reference): what a call makes of the base rows -
 * their bf16 halves, norms - is made once, and the calls' scratch memory is kept between calls, so a call costs its
 * kernels and one upload of the host's tables.  The base keeps num_dataset * dim * 4 bytes more than the rows (where
 * dim is a multiple of 32 and the base has 4096 rows or more) plus the scratch of the largest call so far (at most
 * 8 GiB).  d_dataset must stay as it is while the base exists; calls on one base must not overlap.  Same answers as
 * grab_window_scan_topk / grab_bucket_scan_topk. */
typedef struct grab_scan_base grab_scan_base;
int grab_scan_base_create(const float* d_dataset, size_t num_dataset, uint32_t dim, int metric, grab_scan_base** out);
void grab_scan_base_destroy(grab_scan_base* base);
int grab_scan_base_window_topk(grab_scan_base* base, const float* d_queries, size_t num_queries, uint32_t k,
                               const uint64_t* h_id_lo, const uint64_t* h_id_hi, int64_t* d_out_indices,
                               float* d_out_dists, float* kernel_ms, void* stream);
int grab_scan_base_bucket_topk(grab_scan_base* base, const uint64_t* h_bucket_offsets, uint32_t num_buckets,
                               const float* d_queries, size_t num_queries, uint32_t k, const uint64_t* h_masks,
                               int64_t* d_out_indices, float* d_out_dists, float* kernel_ms, void* stream);
/* Exact filtered top-k (ties to the lower id): the ground-truth routine of the reference's
 * drivers, tests/test_cagra_auto.cu:57-89, as an MFMA contraction with exact re-scoring.
 * Filter arguments as in grab_search_desc. */
int grab_bruteforce_topk(const float* d_dataset, size_t num_dataset, uint32_t dim,
                         const float* d_queries, size_t num_queries, uint32_t k, int metric,
                         int filter_kind, const uint64_t* d_ts, const uint64_t* d_win_start,
                         const uint64_t* d_win_end, uint64_t win_start, uint64_t win_end,
                         int per_query_window, const uint8_t* d_labels, const uint64_t* d_masks,
                         int64_t* d_out_indices, float* d_out_dists, float* kernel_ms,
                         void* stream);

/* Extension: entry-point layer.  `num_samples` rows of the base, evenly spaced in timestamp order
 * (d_ids_by_ts: ids in ascending timestamp order, NULL when row order is timestamp order; d_ts
 * and d_labels, both per row id, may be NULL if the matching filter is never used).
 * grab_entry_layer_select writes, for each query, the n_seeds nearest sample rows that pass the
 * query's filter (row ids of the base, 0xFFFFFFFF padding) - seeds for grab_search_ex.  The
 * reference's counterpart in role is the k-means "virtual index" with entry points of
 * timestamp::TimeStampIndex (src/timeStampIndex.cu:141-238); CagraIndex::query_range seeds with a
 * random sample of the window (src/cagraIndex.cu:270-295). */
int grab_entry_layer_create(const float* d_dataset, size_t num_dataset, uint32_t dim,
                            const uint32_t* d_ids_by_ts, const uint64_t* d_ts, const uint8_t* d_labels,
                            uint32_t num_samples, grab_entry_layer** out);
void grab_entry_layer_destroy(grab_entry_layer* layer);
uint32_t grab_entry_layer_size(const grab_entry_layer* layer);
/* duration of the selection kernel of the last grab_entry_layer_select call that asked for kernel_ms
 * (range filter with n_seeds <= 64; 0 for the other paths, which select inside the contraction) */
float grab_entry_layer_last_select_ms(const grab_entry_layer* layer);
/* filter arguments as in grab_search_desc (filter_kind 0 none, 1 timestamp range, 2 label mask);
 * kernel_ms (optional): duration of the contraction kernel.  Stream-ordered: returns without
 * synchronising unless kernel_ms is asked for. */
int grab_entry_layer_select(grab_entry_layer* layer, const float* d_queries, size_t num_queries,
                            int metric, int filter_kind, const uint64_t* d_win_start,
                            const uint64_t* d_win_end, uint64_t win_start, uint64_t win_end,
                            int per_query_window, const uint64_t* d_masks, uint32_t n_seeds,
                            uint32_t* d_out_seeds, float* kernel_ms, void* stream);

/* Extension: a coarse level over the entry-point layer.  grab_entry_layer_build_groups clusters the
 * sample rows (grab_kmeans: num_groups centroids, niter Lloyd steps) and lays the rows of each group out
 * together, in timestamp order inside the group.  grab_entry_layer_select_grouped then scores, per query,
 * only the in-window rows of the groups of its nearest centroids: the nprobe (<= 64) nearest centroids are
 * found exactly, and their groups are taken nearest first until their in-window rows number min_rows (the
 * group that crosses the mark is taken whole) or the list is used up; the n_seeds (<= 64) nearest of these
 * rows are the seeds (0xFFFFFFFF padding).  With nprobe =
 * num_groups (when that is <= 64) and min_rows = UINT32_MAX the result equals grab_entry_layer_select's.  Same role in the
 * reference: the k-means virtual index of timestamp::TimeStampIndex (src/timeStampIndex.cu:141-238).
 * Window arguments as in grab_entry_layer_select with filter_kind 1 (a layer made without timestamps
 * treats every row as inside).  d_base_ts (optional, with num_base, d_id_lo, d_id_hi): the timestamps of
 * the base the layer was made from (with d_ids_by_ts == NULL), never decreasing with the row id; the call
 * then also writes what grab_windows_to_id_ranges writes, in the same kernel that turns the windows into
 * runs of sample rows.  kernel_ms: the centroid contraction; grab_entry_layer_last_select_ms: centroid
 * selection + group walk.  Stream-ordered, no synchronisation unless kernel_ms is asked for. */
int grab_entry_layer_build_groups(grab_entry_layer* layer, uint32_t num_groups, uint32_t niter, uint64_t seed);
uint32_t grab_entry_layer_num_groups(const grab_entry_layer* layer);
int grab_entry_layer_select_grouped(grab_entry_layer* layer, const float* d_queries, size_t num_queries,
                                    int metric, const uint64_t* d_win_start, const uint64_t* d_win_end,
                                    uint64_t win_start, uint64_t win_end, int per_query_window,
                                    const uint64_t* d_base_ts, size_t num_base, uint64_t* d_id_lo,
                                    uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows,
                                    uint32_t n_seeds, uint32_t* d_out_seeds, float* kernel_ms,
                                    void* stream);

/* The first half of grab_entry_layer_select_grouped alone: d_out_groups[query, 0..nprobe) = the nprobe (<= 64)
 * centroids nearest to the query, nearest first (0xFFFFFFFF padding when the layer has fewer groups), ranked by
 * |c|^2 - 2 q.c (or -q.c), ties to the lower group; at most 1024 groups.  One MFMA kernel: the inner products of 16
 * queries with every centroid, the selection in the accumulator registers.  For grab_search_desc.d_entry_groups.
 * kernel_ms: that kernel.  Stream-ordered. */
int grab_entry_layer_probe(grab_entry_layer* layer, const float* d_queries, size_t num_queries, int metric,
                           uint32_t nprobe, uint32_t* d_out_groups, float* kernel_ms, void* stream);
/* the centroids of the groups, [num_groups, dim], copied to d_out (device memory) */
int grab_entry_layer_centroids(const grab_entry_layer* layer, float* d_out);
/* the groups themselves, to host memory: the members of group g are h_member_ids[h_offsets[g] .. h_offsets[g+1])
 * (row ids of the base, ascending sample position inside a group); h_offsets has num_groups + 1 entries,
 * h_member_ids grab_entry_layer_size entries */
int grab_entry_layer_groups(const grab_entry_layer* layer, uint32_t* h_offsets, uint32_t* h_member_ids);

/* Same walk, but the in-window rows of the groups are not scored: their ids are written as they come (nearest group
 * first, timestamp order inside a group, the walk stopping as in grab_entry_layer_select_grouped), at most max_ids (<= 64)
 * per query, 0xFFFFFFFF padding.  A search that takes them as seeds scores every one of them anyway, so scoring them
 * here to keep the best few only does that work twice; the list is a superset of what the scored selection
 * returns whenever the walk ends within max_ids rows.  Stream-ordered. */
int grab_entry_layer_list_grouped(grab_entry_layer* layer, const float* d_queries, size_t num_queries,
                                  int metric, const uint64_t* d_win_start, const uint64_t* d_win_end,
                                  uint64_t win_start, uint64_t win_end, int per_query_window,
                                  const uint64_t* d_base_ts, size_t num_base, uint64_t* d_id_lo,
                                  uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows,
                                  uint32_t max_ids, uint32_t* d_out_ids, float* kernel_ms, void* stream);

/* cagra::generate_knn_graph, src/index/cagra.cu:69-210 (role also of build_batch_knn_graphs,
 * src/index/raft_help.cuh:74-172).  Exact brute force on the matrix cores instead of IVF-PQ
 * candidates (fp32 instructions, or bf16 ones on rows split into two bf16 halves - see
 * grab_last_knn_bf16_flop -, the candidates then scored exactly and checked); same
 * post-processing: ascending (dist,id), own id removed, 0xFFFFFFFF padding.
 * Unlike the reference the result stays on the device. */
int grab_generate_knn_graph(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t k,
                            int metric, uint32_t* d_knn_graph, float* kernel_ms, void* stream);
/* What the calling thread's last grab_generate_knn_graph / grab_bruteforce_topk did (no counterpart in the
 * reference): the fp32 floating-point operations of its matrix passes (whole tiles of 128 x 128) and, for a graph
 * of 16384 rows or more (4096 where grab_last_knn_bf16_flop applies), the rows that its symmetric pass handed back to
 * the plain pass.  From that size on the graph's contraction computes only the tiles on and above the diagonal - about
 * half of 2 N^2 dim - plus every row against a sample of the rows, which bounds what a tile contributes to the rows
 * behind its columns. */
int grab_last_knn_stats(double* flop, uint64_t* rows_redone);
/* The candidates of a row are picked by |a|^2+|b|^2-2ab (or -ab) on the matrix cores and only then scored exactly.
 * After the exact scoring every row is checked: its k-th exact distance must lie below the smallest GEMM-form
 * distance left outside its candidate lists minus a bound on that form's rounding error,
 * (1.25 dim + 16) 2^-24 (|a|^2 + max|b|^2).  Rows that fail (a large common offset, swarms of near-duplicates:
 * distances below the rounding error of the form) are scored against every admissible column in the canonical
 * order, which is slow and exact.  Returns how many rows of the calling thread's last grab_generate_knn_graph /
 * grab_bruteforce_topk took that path (0 on data whose neighbour distances are well above the error, such as the
 * benchmark's). */
uint64_t grab_last_knn_exact_rows(void);
/* No counterpart in the reference.  A graph of 4096 rows or more with squared L2 and up to 128 dimensions runs its
 * bounding pass and its symmetric pass on bf16 matrix instructions: the rows, centred on their mean, as two bf16 halves
 * each (16 of the 24 bits), a product as q_lo.c_hi + q_hi.c_lo + q_hi.c_hi with fp32 sums - candidates only; the exact
 * scoring and the check above (with (1.25 dim + 1596) 2^-24 for these rows, on the centred norms) decide the result.
 * Returns the bf16 floating-point operations of the calling thread's last call, which grab_last_knn_stats leaves out. */
double grab_last_knn_bf16_flop(void);
/* No counterpart in the reference.  Process-wide switch, on by default: with 0 every kNN graph forms its candidates
 * on fp32 matrix instructions (bounding pass and symmetric pass of tile_topk_kernel), whatever its metric and
 * dimension; the graphs are the same either way.  Returns the previous setting. */
int grab_knn_allow_bf16(int allow);

/* cagra::optimize_prune, src/index/cagra.cu:286-401 (detour counts + stable rank select) */
int grab_optimize_prune(const uint32_t* d_knn_graph, uint32_t* d_new_graph, size_t num_dataset,
                        uint32_t input_degree, uint32_t output_degree, void* stream);
/* detour counts alone (kern_prune, src/index/cagra.cu:219-276) */
int grab_detour_counts(const uint32_t* d_knn_graph, uint8_t* d_counts, size_t num_dataset,
                       uint32_t degree, void* stream);
/* cagra::optimize_create_reverse_graph, src/index/cagra.cu:455-548.  The order inside a
 * reverse list is the order a sequential execution gives: column by column, ascending source. */
int grab_optimize_create_reverse_graph(const uint32_t* d_input_graph, uint32_t* d_rev_graph,
                                       uint32_t* d_rev_counts, size_t num_dataset,
                                       uint32_t degree, void* stream);
/* cagra::optimize_merge_graphs, src/index/cagra.cu:574-650 */
int grab_optimize_merge_graphs(uint32_t* d_graph, const uint32_t* d_rev_graph,
                               const uint32_t* d_rev_counts, size_t num_dataset, uint32_t degree,
                               void* stream);
/* cagra::build, src/index/cagra.cu:665-711.  d_graph is caller-allocated
 * [num_dataset, params.graph_degree] (the reference allocates it and hands it over). */
int grab_build_graph(const float* d_dataset, size_t num_dataset, const uint32_t* d_raw_knn_graph,
                     grab_build_params params, uint32_t* d_graph, void* stream);

/* Time-partitioned graph (CagraIndexOpt), src/index/cagra_opt.cu.  Rows of a bucket are contiguous
 * and d_ts holds the bucket index of every row (0..B-1, non-decreasing), as CagraIndexOpt::build
 * arranges it (src/cagraIndexOpt.cu:160-205).
 *
 * grab_build_time_partitioned_graph = build_time_partitioned_graph (:928-1106): every bucket gets a
 * graph of full width total_degree from its own kNN (k = 2*total_degree) through prune / reverse /
 * merge, ids shifted to global; then grab_build_global_remote_edges.
 * grab_build_global_remote_edges = build_global_remote_edges (:796-907): global neighbours of every
 * row (global_k = grab_remote_global_k, exact here, FAISS IVF-PQ + re-ranking there), slots
 * [local_degree, total_degree) overwritten by update_remote_edges_kernel's rule (:209-303), then
 * grab_enhance_global_connectivity = enhance_global_connectivity (:739-793, kernels :457-600).
 * The reference's reverse lists are in atomic arrival order; here: ascending source id. */
uint32_t grab_remote_global_k(uint32_t total_degree, uint32_t local_degree);
int grab_update_remote_edges(uint32_t* d_graph, const uint64_t* d_ts, const uint32_t* d_candidates, size_t num_dataset,
                             uint32_t total_degree, uint32_t local_degree, uint32_t global_k, void* stream);
int grab_enhance_global_connectivity(size_t num_dataset, uint32_t* d_graph, uint32_t total_degree,
                                     uint32_t local_degree, void* stream);
int grab_build_global_remote_edges(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t* d_graph,
                                   const uint64_t* d_ts, uint32_t total_degree, uint32_t local_degree, int metric,
                                   void* stream);
int grab_build_time_partitioned_graph(const float* d_dataset, size_t total_num, uint32_t dim, uint32_t* d_graph,
                                      const uint64_t* d_ts, const size_t* bucket_sizes, size_t num_buckets,
                                      uint32_t total_degree, uint32_t local_degree, int metric, void* stream);

/* cagra::insert, src/index/cagra.cu:938-1015 with find_near_nodes and update_topology_gpu_v1,
 * src/index/insert.cu:140-440.  d_dataset holds the num_existing old rows, d_new_data the
 * num_new new ones (normally the tail of the same buffer), d_graph has room for all of them;
 * the reference's unused h_graph argument is dropped.  *rng_state supplies the rand_xor_mask of each inner search (low 32 bits of a
 * splitmix64 step per group of 64 new rows) and is advanced.  striped_sort != 0 reproduces
 * the layout mismatch of insert_sort_kernel (insert.cu:100-117). */
int grab_insert(const float* d_dataset, uint32_t dim, size_t num_existing, size_t num_new,
                const float* d_new_data, uint32_t* d_graph, uint32_t graph_degree,
                grab_search_params params, int metric, uint64_t* rng_state, uint32_t flags,
                int striped_sort, void* stream);

/* cagra::insert of the time-partitioned index, src/index/cagra_opt.cu:1674-1981, with the v1
 * branch of update_topology_gpu_opt, src/index/insert.cu:444-727, :1398-1529.  The num_new new rows
 * and their timestamps are already at [num_existing, num_existing + num_new) of d_dataset / d_ts
 * (the reference's d_queries argument points there); d_graph has room for all rows.  d_seeds is
 * [num_new, num_seeds_per_query]: ids of old rows of the bucket target_ts.  The list length of both
 * inner searches is params.itopk_size (:1693).  *rng_state supplies their rand_xor_mask (low 32
 * bits of one splitmix64 step each, the unseeded search first) and is advanced; the reference's
 * unused use_heuristic argument is dropped.  At most 1024 rows per call, and
 * itopk_size + min(num_new, itopk_size/2) <= 1024 (merge_topk_kernel's limit, :1529-1591).
 * Where the reference depends on atomic arrival order (which requests a full mailbox keeps, and
 * their order) requests are taken by ascending (new row, slot).  Slots of the new rows that
 * nothing fills are 0xFFFFFFFF (the reference leaves what the fresh mapping holds); in-batch
 * distances are the library's own instead of RAFT's, ties order by id. */
int grab_insert_partitioned(const float* d_dataset, uint32_t* d_graph, const uint64_t* d_ts,
                            const uint32_t* d_seeds, size_t num_existing, size_t num_new,
                            uint64_t target_ts, uint32_t dim, uint32_t total_degree,
                            uint32_t local_degree, grab_search_params params,
                            uint32_t num_seeds_per_query, int metric, uint64_t* rng_state,
                            uint32_t flags, void* stream);

/* ------------------------------------------------------------------------------------------
 * Device building blocks, exposed with HOST pointers so that they can be checked one by one
 * (the reference checks them in tests/test_bitonic.cu, tests/test_sort_impl.cu,
 * tests/test_hashmap.cu).
 * ---------------------------------------------------------------------------------------- */
/* sorts n (key,val) pairs ascending by (key,val) with the wave-level bitonic network that
 * the kernels use; n <= 1024.  Role of bitonic::warp_sort / load_sort_store,
 * src/index/bitonic.cuh:53-111, src/index/search.cu:110-144. */
int grab_sort_pairs(float* keys, uint32_t* vals, size_t n);
/* inserts keys[0..n) into an LDS table of 1<<bitlen slots from one 256-thread block;
 * results[i] = 1 if keys[i] was new; table_out receives the final table.
 * hashmap::insert, src/index/hashmap.cuh:59-91. */
int grab_hash_insert_many(uint32_t bitlen, const uint32_t* keys, size_t n, uint32_t* results,
                          uint32_t* table_out);
/* distances from one query to rows ids[0..n) of data, in the kernels' canonical order.
 * Role of calc_l2_dist_*, src/index/compute_distance.cuh:14-139. */
int grab_distance_many(const float* query, const float* data, size_t num_rows, uint32_t dim,
                       const uint32_t* ids, size_t n, int metric, float* out);

/* ------------------------------------------------------------------------------------------
 * Device memory helpers for callers without a HIP binding of their own (the reference's
 * callers use cudaMalloc / cudaMemcpy / cudaDeviceSynchronize directly, e.g.
 * src/cagraIndex.cu:200-213,229-234).
 * ---------------------------------------------------------------------------------------- */
int grab_device_malloc(void** out, size_t bytes);
int grab_device_free(void* p);
int grab_copy_to_device(void* dst, const void* src, size_t bytes);
int grab_copy_to_host(void* dst, const void* src, size_t bytes);
int grab_device_memset(void* dst, int value, size_t bytes);
/* page-locked host memory (hipHostMalloc): copies to and from it run at the link's rate */
int grab_host_malloc(void** out, size_t bytes);
int grab_host_free(void* p);
/* stream-ordered copies (the host side page-locked, or the copy is staged and not truly asynchronous) */
int grab_copy_to_device_async(void* dst, const void* src, size_t bytes, void* stream);
int grab_copy_to_host_async(void* dst, const void* src, size_t bytes, void* stream);
/* device-to-device copy by a plain kernel (bytes a multiple of 16): a known-size yardstick for
 * memory-traffic counters */
int grab_device_copy(void* dst, const void* src, size_t bytes);
/* free and total bytes of the current device's memory (hipMemGetInfo) */
int grab_device_memory(size_t* free_bytes, size_t* total_bytes);
int grab_device_synchronize(void);
/* HIP streams (default priority) for callers without a HIP binding of their own */
int grab_stream_create(void** out_stream);
int grab_stream_destroy(void* stream);
int grab_stream_synchronize(void* stream);
/* work queued on `stream` after this call starts once everything queued on `other` so far has completed
 * (an event recorded on `other`); the host does not wait */
int grab_stream_wait(void* stream, void* other);

/* ------------------------------------------------------------------------------------------
 * Growable device buffer.  cagra::DeviceBufferVMM, src/vmm_allocator.cuh:23-118, on
 * hipMemAddressReserve / hipMemCreate / hipMemMap / hipMemSetAccess.
 * ---------------------------------------------------------------------------------------- */
typedef struct grab_vmm grab_vmm;
int grab_vmm_create(size_t max_capacity_bytes, grab_vmm** out);
/* no-op when new_size <= mapped size; GRAB_ERR_CAPACITY when it exceeds the reservation */
int grab_vmm_resize(grab_vmm* b, size_t new_size);
void* grab_vmm_data(const grab_vmm* b);  /* stable across resize */
size_t grab_vmm_size(const grab_vmm* b); /* mapped bytes (granularity multiple) */
size_t grab_vmm_capacity(const grab_vmm* b);
void grab_vmm_destroy(grab_vmm* b);

/* ------------------------------------------------------------------------------------------
 * Index handle (host pointers).  cagra::CagraIndex, src/cagraIndex.hpp:12-119, and the
 * search surface of cagra::CagraIndexOpt, src/cagraIndexOpt.cuh:13-155.
 * ---------------------------------------------------------------------------------------- */
typedef struct grab_index grab_index;

/* CagraIndex(dim, graph_degree, vmm_max_bytes), src/cagraIndex.cu:10-41; local_degree is
 * CagraIndexOpt's third constructor argument (0 = graph_degree). */
int grab_index_create(uint32_t dim, uint32_t graph_degree, uint32_t local_degree,
                      size_t vmm_max_bytes, grab_index** out);
void grab_index_destroy(grab_index* h);
/* extension: metric (default L2), seed of the generator that replaces std::random_device */
int grab_index_set_metric(grab_index* h, int metric);
int grab_index_set_seed(grab_index* h, uint64_t seed);
int grab_index_set_flags(grab_index* h, uint32_t flags);
/* extension: the state of that generator (splitmix64; every search draws its rand_xor_mask as the low 32 bits of
 * the next output) and the query parameters in force - what a caller needs to re-derive a search of the handle */
int grab_index_get_rng_state(const grab_index* h, uint64_t* state);
int grab_index_get_query_params(const grab_index* h, grab_search_params* out);
/* CagraIndex::add, src/cagraIndex.cu:48-75; timestamps may be NULL */
int grab_index_add(grab_index* h, size_t n, const float* vectors, const uint64_t* timestamps);
/* extension for the label-set filter: one label (0..63) per added vector */
int grab_index_set_labels(grab_index* h, size_t n, const uint8_t* labels);
/* CagraIndex::build, src/cagraIndex.cu:80-124 */
int grab_index_build(grab_index* h);
/* CagraIndexOpt::build, src/cagraIndexOpt.cu:133-221: time-partitioned graph (buckets = runs of equal
 * consecutive timestamps, which must be the bucket indices 0..B-1) with the handle's local_degree */
int grab_index_build_partitioned(grab_index* h);
/* CagraIndex::insert, src/cagraIndex.cu:129-183 (64 rows per inner step).  Unlike the
 * reference the timestamps of inserted rows are recorded. */
int grab_index_insert(grab_index* h, size_t n, const float* vectors, const uint64_t* timestamps);
/* What a failed insert (either kind) leaves behind: row count, host copies of rows / timestamps / timestamp map, the
 * generator behind rand_xor_mask and the query parameters are what they were before the call, so searches answer as
 * before.  Growable device buffers keep what was mapped.  Old rows of the device graph may already hold edges to
 * ids of the failed batch: searches skip ids beyond the row count, and when later inserts reuse those ids the edges
 * lead to the rows that then carry them (legal edges, not chosen by distance).
 * grab_index_debug_fail_insert is a test hook: the next insert on the handle fails before its inner step
 * `inner_step` (64 rows a step, 32 for the partitioned insert) with GRAB_ERR_STATE; -1 disarms it. */
int grab_index_debug_fail_insert(grab_index* h, int inner_step);
/* CagraIndexOpt::insert, src/cagraIndexOpt.cu:557-652: all rows go to the bucket timestamps[0]'s
 * seeds (up to max(32, itopk_size) old rows of that bucket, one draw per 32-row step, copied to every
 * row of the step), the search parameters of the handle become 128/4/0/100/14 for good (:581-587), and
 * every 32 rows are one grab_insert_partitioned step over the rows before them.  The index must have
 * been created with 0 < local_degree < graph_degree and hold a built graph. */
int grab_index_insert_partitioned(grab_index* h, size_t n, const float* vectors, const uint64_t* timestamps);
/* Extension: seeds of grab_index_search_range / _search_range_batch come from an entry-point layer
 * (grab_entry_layer_*) of num_samples rows, seeds_per_query nearest in-window sample rows each, instead
 * of a random sample of the window (src/cagraIndex.cu:270-295).  The layer is rebuilt on the next range
 * search after rows were added.  When timestamps never decrease with the row id the traversal tests row
 * ids against the window's id interval and reads no timestamps.  num_samples = 0 switches it off. */
int grab_index_set_entry_layer(grab_index* index, uint32_t num_samples, uint32_t seeds_per_query);
/* Extension: a coarse level for that layer (grab_entry_layer_build_groups / _select_grouped): num_groups k-means
 * groups of the sample rows, nprobe nearest centroids kept per query, groups walked until min_rows in-window
 * rows were scored.  Used when seeds_per_query <= 64; num_groups = 0 switches it off. */
int grab_index_set_entry_groups(grab_index* index, uint32_t num_groups, uint32_t nprobe, uint32_t min_rows);
/* Extension: with the coarse level and timestamps that never decrease with the row id, hand the search the in-window
 * rows of the nearest groups as they are listed (at most max_rows, <= 64; grab_entry_layer_list_grouped) instead of
 * scoring them first and keeping seeds_per_query (grab_entry_layer_select_grouped).  0 (the default) = scored. */
int grab_index_set_entry_list(grab_index* index, uint32_t max_rows);
/* Extension: grab_index_search_range_batch cuts a batch of more than this many queries (default 5000; coarse level
 * set, timestamps never decreasing with the row id) into equal chunks that overlap on streams of the handle: the
 * calling thread and a helper thread of the handle stage the queries in page-locked memory, a kernel copies a chunk
 * in, its search writes the results straight into page-locked memory, and the caller's arrays are filled chunk by
 * chunk while later chunks run.  Results are those of the undivided call.  0 switches this off. */
int grab_index_set_batch_chunk(grab_index* index, size_t queries_per_chunk);
int grab_index_set_build_params(grab_index* h, uint32_t intermediate_degree, uint32_t graph_degree);
int grab_index_set_query_params(grab_index* h, uint32_t itopk, uint32_t search_width,
                                uint32_t min_iterations, uint32_t max_iterations,
                                uint32_t hash_bitlen);
int grab_index_set_insert_params(grab_index* h, uint32_t itopk, uint32_t search_width,
                                 uint32_t min_iterations, uint32_t max_iterations,
                                 uint32_t hash_bitlen);
/* CagraIndex::query, src/cagraIndex.cu:188-235 */
int grab_index_search(grab_index* h, const float* queries, size_t nq, int k, int64_t* indices,
                      float* dists, const uint32_t* seeds, size_t seeds_per_query);
/* CagraIndex::query_range, src/cagraIndex.cu:237-347: one window [start_ts,end_ts) and one
 * sampled seed set for the whole batch; range_radius >= 0.99 searches unfiltered */
int grab_index_search_range(grab_index* h, const float* queries, size_t nq, int k,
                            float range_radius, uint64_t start_ts, uint64_t end_ts,
                            int64_t* indices, float* dists, const uint32_t* seeds,
                            size_t seeds_per_query);
/* extension: a window per query, seeds drawn per query on the device */
int grab_index_search_range_batch(grab_index* h, const float* queries, size_t nq, int k,
                                  const uint64_t* start_ts, const uint64_t* end_ts,
                                  int64_t* indices, float* dists);
/* extension (the reference answers every window through the graph): the exact top-k of every query inside its window,
 * k <= 128.  With timestamps that never decrease with the row id the windows are intervals of row ids and are scanned
 * by grab_scan_base_window_topk over a base that the handle prepares once and remakes when rows were added; otherwise
 * every row is scanned with the window test.  Faster than the graph search for windows of a few percent of the rows
 * and below, where a graph cut down to the window also loses recall.  Slots that a window cannot fill: -1 / -1.0f. */
int grab_index_scan_range_batch(grab_index* h, const float* queries, size_t nq, int k,
                                const uint64_t* start_ts, const uint64_t* end_ts,
                                int64_t* indices, float* dists);
/* extension: grab_index_search_range_batch answers the queries whose window holds at most this fraction of the rows
 * through grab_index_scan_range_batch (exact) and searches the graph for the others; timestamps that never decrease
 * with the row id, k <= 128.  0 (the default): every query is a graph search, as in the reference.  On 1M x 128 the
 * scan is the faster of the two below about 2 % and the one that keeps recall@10 above 0.95 below about 5 %. */
int grab_index_set_scan_below(grab_index* h, double fraction);
/* CagraIndexOpt::query_local, src/cagraIndexOpt.cu:301-420: only rows stamped target_ts,
 * following the first local_degree slots; -1 / -1.0f when the bucket is empty */
int grab_index_search_bucket(grab_index* h, const float* queries, size_t nq, int k,
                             uint64_t target_ts, int64_t* indices, float* dists);
/* extension: label-set filter, one 64-bit mask per query */
int grab_index_search_mask(grab_index* h, const float* queries, size_t nq, int k,
                           const uint64_t* masks, int64_t* indices, float* dists);
size_t grab_index_size(const grab_index* h);
const float* grab_index_get_data(const grab_index* h);   /* host mirror, CagraIndex::get_data */
const uint32_t* grab_index_get_graph(grab_index* h);     /* host mirror refreshed from the device */
/* CagraIndexOpt::get_ids_by_timestamp, src/cagraIndexOpt.cuh: writes up to cap ids, returns count */
size_t grab_index_ids_by_timestamp(const grab_index* h, uint64_t ts, uint32_t* out, size_t cap);
/* CagraIndexOpt::sample_seeds_by_time, src/cagraIndexOpt.cu:95-131: up to `num` ids whose timestamp lies
 * in [min_ts, max_ts] (inclusive).  Returns how many were drawn; writes at most `cap` of them. */
size_t grab_index_sample_seeds_by_time(grab_index* h, uint64_t min_ts, uint64_t max_ts, size_t num, uint32_t* out, size_t cap);
/* bytes mapped into the three growable buffers (data, graph, timestamps) */
int grab_index_mapped_bytes(const grab_index* h, size_t* data, size_t* graph, size_t* ts);
/* device pointers of the resident index (valid until the next add/build/insert/load) */
int grab_index_device_ptrs(grab_index* h, const float** d_data, const uint32_t** d_graph,
                           const uint64_t** d_ts);
/* duration of the search kernel of the last search call on this handle, from HIP events */
float grab_index_last_kernel_ms(const grab_index* h);
/* seconds spent in the last build: kNN graph, optimisation, total */
int grab_index_last_build_seconds(const grab_index* h, double* knn, double* optimize, double* total);
/* CagraIndex::save / load, src/cagraIndex.cu:352-395 (same byte layout) */
int grab_index_save(grab_index* h, const char* path);
int grab_index_load(grab_index* h, const char* path);
/* CagraIndexOpt::save / load, src/cagraIndexOpt.cu:725-896: the "MCAG" version 1 layout (header,
 * timestamps, timestamp -> ids map, data, graph), byte for byte */
int grab_index_save_mcag(grab_index* h, const char* path);
int grab_index_load_mcag(grab_index* h, const char* path);

/* ---- timestamp::TimeStampIndex, src/timeStampIndex.cuh:47-63, src/timeStampIndex.cu:36-419 ----
 * One CagraIndex per timestamp plus a "virtual" CagraIndex over k-means centroids of every bucket (16*sqrt(n)
 * centroids per bucket, 5 entry points each).  grab_tsindex_query: search the virtual layer for 10*probe_buckets
 * centroids, let them vote for buckets, search the probe_buckets most voted buckets from the voters' entry points,
 * merge by distance; global ids are assigned in insertion order.  The reference clusters with faiss::Clustering
 * (30 iterations) on a GPU flat index; grab_kmeans is plain Lloyd on the exact assignment, so centroids (and with
 * them the routing) are not pinned against the reference. */
typedef struct grab_tsindex grab_tsindex;
int grab_kmeans(const float* h_data, size_t n, uint32_t dim, uint32_t k, uint32_t niter, uint64_t seed,
                float* h_centroids, int64_t* h_assign /* [n] or NULL */);
int grab_tsindex_create(uint32_t dim, uint32_t graph_degree, size_t cluster_ratio, size_t vmm_max_bytes_per_bucket,
                        grab_tsindex** out);
void grab_tsindex_destroy(grab_tsindex* t);
int grab_tsindex_set_seed(grab_tsindex* t, uint64_t seed);
int grab_tsindex_insert(grab_tsindex* t, const float* vectors, const uint64_t* timestamps, size_t num_vectors,
                        uint64_t* out_start_id);
int grab_tsindex_build_virtual_index(grab_tsindex* t);
int grab_tsindex_query(grab_tsindex* t, const float* query, size_t topk, int64_t* out_indices, float* out_dists,
                       int probe_buckets);
size_t grab_tsindex_size(const grab_tsindex* t);
size_t grab_tsindex_num_buckets(const grab_tsindex* t);
size_t grab_tsindex_num_virtual_points(const grab_tsindex* t);
int grab_tsindex_locate(const grab_tsindex* t, uint64_t global_id, uint64_t* out_ts, size_t* out_local);
/* extension, read-only views of the two levels (the reference keeps them private, src/timeStampIndex.cuh:66-93):
 * the virtual CagraIndex (NULL before build_virtual_index) and a bucket's CagraIndex (NULL if there is none) as
 * borrowed handles, valid until the next insert / build_virtual_index / destroy; the bucket timestamps in
 * ascending order (returns their number, writes at most cap); virtual point i's bucket and entry points (local
 * ids of that bucket; writes at most cap, *out_count = how many there are) */
grab_index* grab_tsindex_virtual_index(grab_tsindex* t);
grab_index* grab_tsindex_bucket_index(grab_tsindex* t, uint64_t ts);
size_t grab_tsindex_bucket_timestamps(const grab_tsindex* t, uint64_t* out, size_t cap);
int grab_tsindex_virtual_point(const grab_tsindex* t, size_t i, uint64_t* out_ts, uint32_t* out_entry_points, size_t cap,
                               size_t* out_count);

#ifdef __cplusplus
}
#endif
#endif /* GRAB_ANNS_H */
