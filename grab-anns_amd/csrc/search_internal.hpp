// Arguments and LDS layout of the search kernel, shared by the kernel and its host launcher.
#pragma once
#include "common.hpp"
#include "device_utils.hpp"

namespace grab {

// Seeds listed by the search kernel itself from the entry-point layer (register-queue wave kernel, id-interval filter):
// the query's window arrives as timestamps, becomes an interval of row ids through the pivot levels over the base's
// timestamps, and the members of the query's nearest groups inside that interval are the seeds.
struct EntryWalk {
    const uint32_t* groups;   // [nq, nprobe] nearest centroids, nearest first; null = seeds as given
    const uint32_t* tbl;      // [G, 65] first member of each group at or after each stretch of base ids, then the group's end
    const uint32_t* ids;      // base id of every member, group by group, ascending inside a group
    const uint64_t* piv;      // pivot levels over the base timestamps, level 0 (every 32nd row) first
    uint32_t piv_off[6], piv_cnt[6];
    uint32_t nlev, nprobe, min_rows, n_base, stretch;
};

struct SearchArgs {
    const float* data;
    const uint32_t* graph;
    const float* queries;
    const uint32_t* seeds;
    const uint64_t* ts;
    const uint64_t* graph_ts;  // optional: timestamp of every neighbour, laid out like the graph
    const uint32_t* rank_of_id;  // optional, id-interval filter: the interval is tested on rank_of_id[id] (a row's place in timestamp order)
    const uint32_t* graph_rank;  // optional with it: rank_of_id of every neighbour, laid out like the graph
    const uint64_t* win_start_arr;
    const uint64_t* win_end_arr;
    const uint8_t* labels;
    const uint64_t* masks;
    int64_t* out_ids;
    float* out_dists;
    grab_counters* counters;
    uint32_t* global_hash;  // per-query tables when the visited set does not fit LDS, else null
    uint64_t n;
    uint64_t rand_xor_mask;
    uint64_t win_start, win_end;
    uint32_t dim, degree, active_degree, nq, k, itopk, search_width, max_iterations, hash_bitlen;
    uint32_t n_seeds, n_provided, flags, cmax;
    uint32_t ccap;          // wave-per-query kernel: capacity of the candidate list (cmax = survivor list)
    int single_queue;       // wave-per-query kernel: one queue buffer, merged in place (itopk <= 64, ccap <= 128)
    int reg_queue;          // wave-per-query kernel: the queue lives in registers, 1/2/4 entries per lane (itopk <= 256, not strict)
    int per_query_window;
    int split_merge;        // workgroup-per-query kernel with 1024 threads: the merge is cut into tasks whose partial counts live in LDS
    int fixed_shape;        // register-queue kernel: rows of 64 slots all followed, <= 4 parents, <= 64 seeds, filter first, cmax >= 256
    EntryWalk entry;
};

struct SearchLdsLayout {
    uint32_t off_query, off_top0, off_top1, off_cand, off_surv, off_parents, off_misc, off_parts, off_hash, total;
};

// Batches of up to this many queries get 1024 threads a query instead of 256 (fewer queries than CUs: what counts is
// how long one query takes), and split a merge over the waves, which leave their partial counts in LDS - unless
// those counts would push the queue or the visited set out of LDS: then the plain merge runs on the 1024 threads
constexpr uint32_t kSmallBatchQueries = 256;
constexpr uint32_t kMergeChunks = 4;  // parts that the candidate list is cut into for a split merge

// cmax = capacity of the survivor / candidate lists = max(search_width*degree, n_seeds)
__host__ __device__ inline SearchLdsLayout search_lds_layout(uint32_t itopk, uint32_t dim, uint32_t cmax,
                                                            uint32_t search_width, uint32_t hash_bitlen,
                                                            bool hash_in_lds, bool split_merge) {
    SearchLdsLayout l;
    uint32_t off = 0;
    auto take = [&](uint32_t bytes) {
        uint32_t o = off;
        off += (bytes + 15u) & ~15u;
        return o;
    };
    l.off_query = take(dim * 4);
    l.off_top0 = take(itopk * 8);
    l.off_top1 = take(itopk * 8);
    l.off_cand = take(cmax * 8);
    l.off_surv = take(cmax * 4);
    l.off_parents = take(search_width * 4);
    l.off_misc = take(16 * 4);
    // split merge: per candidate one count per list part and one for the queue, per queue entry one count per list part
    l.off_parts = take(split_merge ? ((kMergeChunks + 1u) * cmax + kMergeChunks * itopk) * 4u : 0u);
    l.off_hash = take(hash_in_lds ? (1u << hash_bitlen) * 4u : 0u);
    l.total = off;
    return l;
}

// layout of the wave-per-query kernel; query_dim = 0 when the query lives in registers
struct SearchWaveLdsLayout {
    uint32_t off_top0, off_top1, off_cand, off_surv, off_parents, off_query, off_hash, total;
};

__host__ __device__ inline SearchWaveLdsLayout search_wave_lds_layout(uint32_t itopk, uint32_t query_dim, uint32_t cmax, uint32_t ccap,
                                                                     bool single_queue, uint32_t search_width,
                                                                     uint32_t hash_bitlen) {
    SearchWaveLdsLayout l;
    uint32_t off = 0;
    auto take = [&](uint32_t bytes) {
        uint32_t o = off;
        off += (bytes + 15u) & ~15u;
        return o;
    };
    l.off_top0 = take(itopk * 8);
    l.off_top1 = take(single_queue ? 0 : itopk * 8);
    l.off_cand = take(ccap * 8);
    l.off_surv = take(cmax * 4);
    l.off_parents = take(search_width * 4);
    l.off_query = take(query_dim * 4);
    l.off_hash = take((1u << hash_bitlen) * 4u);
    l.total = off;
    return l;
}

// LDS a workgroup may use on gfx950
constexpr uint32_t kMaxLdsBytes = 160 * 1024;

int launch_search(const SearchArgs& a, int metric, int filter, size_t lds_bytes, hipStream_t stream);
int launch_search_wave(const SearchArgs& a, int metric, int filter, size_t lds_bytes, hipStream_t stream);

// grab_search_ex_static: slots (uint32) of the array in the device image that holds its visited sets, 32 MiB
constexpr size_t kStaticTableSlots = (size_t)8 << 20;
// device address of that array on the current device (looked up once per device)
int static_visited_sets(uint32_t** tables);

// grab_search_ex with the option of returning before the kernel has finished, and of taking the
// visited sets that do not fit LDS from the static array instead of hipMalloc (then nothing is
// allocated, created or awaited)
int search_ex_impl(const grab_search_desc* d, bool sync, bool static_tables = false);

// fills a descriptor the way the reference wrapper `wrapper` (GRAB_WRAP_*) would: clamps of
// itopk and seed count included; filter fields are left empty
void fill_search_desc(grab_search_desc* d, int wrapper, const float* d_dataset, size_t n, uint32_t dim,
                      const uint32_t* d_graph, uint32_t degree, uint32_t active_degree, const float* d_queries,
                      size_t nq, uint32_t k, grab_search_params p, int metric, const uint32_t* d_seeds,
                      uint32_t n_provided, uint64_t mask, uint32_t flags, int64_t* d_out_indices,
                      float* d_out_dists, void* stream);

}  // namespace grab
