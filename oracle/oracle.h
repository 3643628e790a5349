/*
 * CPU oracle for the GRAB-ANNS hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library is a sequential CPU restatement of the reference algorithms
 * (hxlou/GRAB-ANNS, paths relative to the reference root).  It exists so that
 * the HIP kernels can be compared against it on the same seeded inputs.  It is
 * linked / loaded only by tests, by the smoke check and by the CPU-baseline leg
 * of the benchmark.  The product library never calls into it.
 *
 * Pinning status of each function (what fixes its behaviour independently of
 * this file):
 *   orc_next_power_of_2 / orc_queue_capacity / orc_smem_bytes
 *        pinned: compiled reference header src/index/smem_cal.cuh (oracle/_ref)
 *        and the closed-form cases (64,4,64)->512, (256,6,64)->1024, (128,4,32)->256.
 *   orc_bitonic_network   pinned: recipes of tests/test_bitonic.cu:73-80 and
 *        tests/test_sort_impl.cu:64-81 (libstdc++ fixtures), 0/1 principle brute force.
 *   orc_sort_pairs        pinned: std::sort of (key,val) pairs, same fixtures.
 *   orc_hash_*            pinned: tests/test_hashmap.cu:171-187 cases + slot invariant.
 *   orc_l2_canon / orc_ip_canon   pinned: float64 cross-check (1e-5 relative),
 *        exactness on integer-valued inputs, a==b -> 0, unit-vector identity.
 *   orc_l2_natural / orc_l2_ref_warp   restate tests/test_cagra_auto.cu:48-50 and
 *        src/index/compute_distance.cuh:120-139; pinned the same way.
 *   orc_bruteforce_topk   pinned: numpy stable argsort on (dist,id), tiny-N brute force.
 *   orc_knn_graph         pinned: tests/test_knn_build.cu:32-38,58-117 (points on a line).
 *   orc_detour_counts / orc_prune   pinned: brute force on N<=64, complete-graph and
 *        no-2-hop closed forms.
 *   orc_reverse_graph     pinned: in-degree invariant + python restatement on tiny N.
 *   orc_merge_graphs      pinned: python restatement of src/index/cagra.cu:574-650 on tiny N.
 *   orc_search            pinned: a literal Python model of search_kernel / _bucket / _range
 *        and their expansion steps as written (flat queue of queue_capacity slots, seeds at
 *        slot i whatever the insert says, whole-queue sort by distance, flag bit, table rebuilt
 *        before the sort every 30 iterations, stale slots of the range variant, id & 0x7FFFFFFF)
 *        gives the same ids, distance bits and work counters on walks of 70-140 iterations,
 *        with and without table overflow (tests/ref_literal.py,
 *        tests/test_oracle_search_literal.py); plus invariants and the exhaustive case.  The
 *        compiled reference cannot run here, so end-to-end recall parity with the CUDA binary
 *        stays "parity unpinned".
 *   orc_insert_batch      pinned: the same literal model for its searches, the striped load of
 *        insert_sort_kernel and update_topology_gpu_v1 restated in Python, whole graph equal;
 *        LCG closed form; recall gate of tests/test_cagra_insert.cu:284.
 *   orc_insert_partitioned_*   pinned by an independent Python restatement on small inputs and by
 *        invariants; PARITY UNPINNED against the compiled reference (see the declarations).
 */
#ifndef GRAB_ORACLE_H
#define GRAB_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_INVALID 0xFFFFFFFFu

/* search "wrapper" kinds: which reference host wrapper's clamping rules apply */
enum {
    ORC_WRAP_SEARCH = 0,       /* cagra::search            src/index/cagra.cu:844-935      */
    ORC_WRAP_SEARCH_OPT = 1,   /* cagra::search_opt        src/index/cagra_opt.cu:1108-1210 */
    ORC_WRAP_BUCKET = 2,       /* cagra::search_bucket_opt src/index/cagra_opt.cu:1212-1328 */
    ORC_WRAP_RANGE = 3         /* cagra::search_bucket_range src/index/cagra_opt.cu:1330-1442 */
};

/* ID_RANGE: the window is given as an interval of row ids (what a timestamp window is when
 * timestamps never decrease with the row id); no filter word is read */
enum { ORC_FILTER_NONE = 0, ORC_FILTER_RANGE = 1, ORC_FILTER_MASK = 2, ORC_FILTER_ID_RANGE = 3 };
enum { ORC_METRIC_L2 = 0, ORC_METRIC_IP = 1 };

/* flag bit 0: literal reference behaviour for the quirks that the product fixes by
 * default (seeds bypass dedupe and filter, hash restore before the queue merge,
 * 0x7FFFFFFF instead of -1 for an unfilled result slot). */
#define ORC_FLAG_STRICT_REFERENCE 1u
/* evaluate the filter before the visited-set insert (extension; same results while the table has room) */
#define ORC_FLAG_FILTER_FIRST 2u

/* ---- closed forms (src/index/smem_cal.cuh:13-76) ---- */
uint32_t orc_next_power_of_2(uint32_t n);
uint32_t orc_queue_capacity(uint32_t itopk, uint32_t search_width, uint32_t degree);
size_t   orc_smem_bytes(uint32_t itopk, uint32_t dim, uint32_t search_width, uint32_t degree,
                        uint32_t hash_bitlen);

/* wrapper clamps: effective itopk and seed count for each reference wrapper */
void orc_search_plan(int wrapper, uint32_t k, uint32_t itopk_param, uint32_t search_width,
                     uint32_t degree, uint32_t n_provided_seeds,
                     uint32_t* itopk_eff, uint32_t* n_seeds, uint32_t* queue_capacity);

/* ---- sorting ---- */
/* literal model of bitonic::warp_sort (src/index/bitonic.cuh:53-111): n = lanes*per_lane
 * elements, blocked layout, no swap on equal keys. Sorts in place. */
void orc_bitonic_network(float* keys, uint32_t* vals, uint32_t lanes, uint32_t per_lane, int asc);
/* the product's ordering rule: ascending by (key, val) */
void orc_sort_pairs(float* keys, uint32_t* vals, size_t n);

/* ---- visited set (src/index/hashmap.cuh:30-117) ---- */
/* table has 1<<bitlen slots, caller fills with ORC_INVALID (or calls orc_hash_init). */
void orc_hash_init(uint32_t* table, uint32_t bitlen);
int  orc_hash_insert(uint32_t* table, uint32_t bitlen, uint32_t key); /* 1 new, 0 present or full */
void orc_hash_insert_many(uint32_t* table, uint32_t bitlen, const uint32_t* keys, size_t n,
                          uint32_t* results);

/* ---- distances ---- */
float orc_l2_canon(const float* a, const float* b, uint32_t dim);   /* canonical order of the product */
float orc_ip_canon(const float* a, const float* b, uint32_t dim);   /* -dot, same order */
float orc_l2_natural(const float* a, const float* b, uint32_t dim); /* tests/test_cagra_auto.cu:48-50 */
float orc_l2_ref_warp(const float* a, const float* b, uint32_t dim);/* compute_distance.cuh:120-139 */
void  orc_l2_canon_many(const float* q, const float* data, const uint32_t* ids, size_t n,
                        uint32_t dim, int metric, float* out);

/* ---- exact (filtered) top-k, ties to the lower id ---- */
/* win_start/win_end: nq entries when per_query_window, else 1 entry. masks: nq entries. */
void orc_bruteforce_topk(const float* data, size_t n, uint32_t dim, const float* queries, size_t nq,
                         uint32_t k, int metric, int filter_kind, const uint64_t* ts,
                         const uint64_t* win_start, const uint64_t* win_end, int per_query_window,
                         const uint8_t* labels, const uint64_t* masks,
                         int64_t* out_ids, float* out_dists, int threads);

/* ---- graph build ---- */
void orc_knn_graph(const float* data, size_t n, uint32_t dim, uint32_t k, int metric,
                   uint32_t* out_graph, int threads);
void orc_detour_counts(const uint32_t* knn, size_t n, uint32_t degree, uint8_t* counts, int threads);
void orc_prune(const uint32_t* knn, size_t n, uint32_t in_degree, uint32_t out_degree,
               uint32_t* out_graph, int threads);
void orc_reverse_graph(const uint32_t* graph, size_t n, uint32_t degree, uint32_t* rev,
                       uint32_t* rev_counts);
void orc_merge_graphs(uint32_t* graph, const uint32_t* rev, const uint32_t* rev_counts, size_t n,
                      uint32_t degree, int threads);
void orc_optimize(const uint32_t* knn, size_t n, uint32_t in_degree, uint32_t out_degree,
                  uint32_t* out_graph, int threads);

/* ---- beam search ---- */
typedef struct {
    uint64_t iterations;   /* loop iterations that reached the expansion step */
    uint64_t seed_dists;   /* S */
    uint64_t parents;      /* P */
    uint64_t filter_reads; /* F */
    uint64_t child_dists;  /* D */
    uint64_t hash_full;    /* inserts rejected because the table was full */
} orc_counters;

void orc_search(const float* data, size_t n, uint32_t dim, const uint32_t* graph, uint32_t degree,
                uint32_t active_degree, const float* queries, size_t nq, uint32_t k,
                uint32_t itopk, uint32_t search_width, uint32_t max_iterations,
                uint32_t hash_bitlen, uint32_t n_seeds, const uint32_t* seeds,
                uint32_t n_provided, uint64_t rand_xor_mask, int metric, int filter_kind,
                const uint64_t* ts, const uint64_t* win_start, const uint64_t* win_end,
                int per_query_window, const uint8_t* labels, const uint64_t* masks,
                uint32_t flags, int64_t* out_ids, float* out_dists, orc_counters* counters,
                int threads);

/* ---- seed sampling extension (stratified sample of the ids inside a window) ---- */
/* sorted_ts: timestamps ascending; ids_by_ts: ids in that order. */
void orc_sample_window_seeds(const uint64_t* sorted_ts, const uint32_t* ids_by_ts, size_t n,
                             const uint64_t* win_start, const uint64_t* win_end, size_t nq,
                             int per_query_window, uint32_t n_seeds, uint64_t seed,
                             uint32_t* out_seeds);

/* ---- rng used wherever the reference draws from std::random_device ---- */
uint64_t orc_splitmix64(uint64_t* state);

/* ---- insert (src/index/cagra.cu:938-1015, src/index/insert.cu:140-440) ---- */
/* data holds n_existing + n_new rows; graph has room for the same number of rows.
 * One call = one reference cagra::insert call (the caller does the 64-wide batching).
 * Each inner search (one per 64 new rows, insert.cu:157-176) draws its rand_xor_mask as the
 * low 32 bits of orc_splitmix64(rng_state). striped_sort!=0 reproduces the striped/blocked
 * mismatch of insert_sort_kernel (insert.cu:100-117). */
void orc_insert_batch(const float* data, uint32_t dim, size_t n_existing, size_t n_new,
                      uint32_t* graph, uint32_t degree, uint32_t itopk_param,
                      uint32_t search_width, uint32_t max_iterations, uint32_t hash_bitlen,
                      uint64_t* rng_state, int metric, uint32_t flags, int striped_sort,
                      int threads);

/* ---- insert into the time-partitioned graph (src/index/cagra_opt.cu:1674-1981,
 * src/index/insert.cu:444-727, :1398-1529) ----
 * Pinned by: an independent Python restatement of the merge and of the fill / mailbox / apply rules
 * on small inputs, and invariants (local slots hold rows of the new row's timestamp, remote slots
 * of old rows only change inside the documented slot ranges, at most cap requests reach a row).
 * PARITY UNPINNED against the compiled reference: its in-batch neighbours come from RAFT's
 * brute force (other rounding, ties in network order) and its mailboxes are in atomic arrival order;
 * here distances are the canonical ones, ties order by id and mailboxes by (new row, slot).
 * orc_insert_partitioned_batch = one cagra::insert call; data holds n_existing + n_new rows, ts
 * their timestamps; seeds is [n_new, n_seeds_per_query].  The two searches draw their
 * rand_xor_mask from orc_splitmix64(rng_state): first the global one, then the bucket one. */
void orc_merge_batch_neighbours(const float* new_data, size_t n_new, uint32_t dim, size_t n_existing, uint32_t search_k,
                                int metric, int64_t* local_ids, const float* local_dists);
void orc_insert_partitioned_update(uint32_t* graph, const uint64_t* ts, int64_t* local_ids, int64_t* global_ids,
                                   size_t n_existing, size_t n_new, uint64_t target_ts, uint32_t total_degree,
                                   uint32_t local_degree, uint32_t search_k);
void orc_insert_partitioned_batch(const float* data, uint32_t dim, const uint64_t* ts, size_t n_existing, size_t n_new,
                                  uint64_t target_ts, uint32_t* graph, uint32_t total_degree, uint32_t local_degree,
                                  const uint32_t* seeds, uint32_t n_seeds_per_query, uint32_t itopk_param,
                                  uint32_t search_width, uint32_t max_iterations, uint32_t hash_bitlen,
                                  uint64_t* rng_state, int metric, uint32_t flags, int threads);

/* ---- time-partitioned graph (src/index/cagra_opt.cu:209-303, :457-600, :739-1106) ----
 * Pinned by: closed form of global_k; brute-force re-derivation of the remote-slot rule on tiny
 * inputs (independent Python restatement in the tests); invariants (local slots stay inside the row's
 * bucket, remote slots outside it, strong half untouched by the injection).  PARITY UNPINNED against
 * the compiled reference: its candidates come from FAISS IVF-PQ and its reverse lists are in atomic
 * arrival order; here candidates are exact and the order is ascending source id. */
uint32_t orc_remote_global_k(uint32_t total_degree, uint32_t local_degree);
void orc_remote_edges(const uint32_t* cand, const uint64_t* ts, size_t n, uint32_t global_k, uint32_t total_degree,
                      uint32_t local_degree, uint32_t* graph);
void orc_inject_reverse_remote(uint32_t* graph, size_t n, uint32_t total_degree, uint32_t local_degree);
void orc_build_time_partitioned(const float* data, size_t n, uint32_t dim, const uint64_t* ts, const size_t* bucket_sizes,
                                size_t num_buckets, uint32_t total_degree, uint32_t local_degree, int metric,
                                uint32_t* graph, int threads);

/* ---- k-means of the two-level index (role of faiss::Clustering, src/timeStampIndex.cu:163-178) ----
 * Pinned by: Lloyd invariants (the objective never increases, at a fixed point every centroid is the mean of its
 * rows, every row sits with its nearest centroid by float64 numpy).  PARITY UNPINNED against
 * FAISS's centroids (absent; different initialisation and empty-cluster handling). */
void orc_kmeans(const float* data, size_t n, uint32_t dim, uint32_t k, uint32_t niter, uint64_t seed, float* centroids,
                int64_t* assign_out, int threads);

#ifdef __cplusplus
}
#endif
#endif
