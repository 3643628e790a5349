// The entry-point layer as the library keeps it: a sample of the base in timestamp order, optionally grouped by
// nearest centroid, and the tables that turn a timestamp window into runs of group members.  Shared by the
// contraction kernels that build and query it, the kernel that ranks the centroids, and the search entry that
// lets the traversal list its own seeds.
#pragma once
#include <algorithm>

#include "common.hpp"

namespace grab {

// device buffer that only ever grows
struct GrowBuf {
    void* ptr = nullptr;
    size_t bytes = 0;
    int ensure(size_t need) {
        if (need <= bytes) return GRAB_OK;
        if (ptr) GRAB_HIP(hipFree(ptr));
        ptr = nullptr;
        bytes = 0;
        GRAB_HIP(hipMalloc(&ptr, std::max<size_t>(need, 4096)));
        bytes = std::max<size_t>(need, 4096);
        return GRAB_OK;
    }
    void release() {
        if (ptr) (void)hipFree(ptr);
        ptr = nullptr;
        bytes = 0;
    }
    template <class T>
    T* as() const { return static_cast<T*>(ptr); }
};

// Fan-out of the pivot levels over the base timestamps: level 1 holds the last timestamp of every block of 32 base
// rows, level 2 the last entry of every block of 32 level-1 entries, and so on until a level has at most 32
// entries.  A lower bound then takes one coalesced 256-byte read per level and one of the base itself.
constexpr uint32_t kPivotFan = 32;
constexpr uint32_t kPivotMaxLevels = 6;   // 32^7 > 2^31 rows
// a group's members are cut into this many stretches of base ids; the table holds the first member of each
constexpr uint32_t kIdStretches = 64;

// the pivot levels as a kernel argument
struct EntryPivots {
    uint32_t levels, off[kPivotMaxLevels], cnt[kPivotMaxLevels];
};

}  // namespace grab

struct grab_entry_layer {
    uint32_t S = 0, dim = 0;
    int num_cu = 0;
    bool has_ts = false, has_labels = false;
    float last_select_ms = 0.0f;  // selection kernel of the last timed select (dense path)
    grab::GrowBuf sample, norm, ids, ts, labels;                         // the layer
    grab::GrowBuf qnorm, lo, hi, keys, perm, cand, tilebuf, dense, sched, qsorted;       // grow-only scratch of select
    // optional coarse level (grab_entry_layer_build_groups): the sample rows grouped by nearest centroid
    uint32_t num_groups = 0;
    grab_entry_layer* coarse = nullptr;                          // a layer whose rows are the centroids
    // u32 [G,65] (first member at or after each of 64 stretches of sample rows, then the end), u32 [S] (sample row of
    // each member, ascending inside a group), f32 [S,dim]
    grab::GrowBuf group_tbl, group_pos, group_rows;
    grab::GrowBuf group_ids;                                     // u32 [S]: base row id of each member, in the groups' layout
    grab::GrowBuf group_tbl_id;                                  // u32 [G,65]: the same table over stretches of base ids
    grab::GrowBuf cent_pad;                                      // bf16, 2 * (G rounded up to 16) * (dim rounded up to 128) values: the centroids as hi and lo halves in the order the ranking kernel loads them
    grab::GrowBuf probe;                                         // scratch of the grouped select
    // base rows in timestamp order (made with d_ids_by_ts == NULL and timestamps): pivot levels over the base's
    // timestamps, level 1 first
    uint64_t num_base = 0;
    bool base_in_ts_order = false;
    uint32_t piv_levels = 0, piv_off[grab::kPivotMaxLevels] = {}, piv_cnt[grab::kPivotMaxLevels] = {};
    grab::GrowBuf pivots;
    // a layer of centroids is always asked with the one window that covers every row: the order of the
    // queries and the work list of the contraction then depend on the number of queries alone and are kept
    bool fixed_window = false;
    uint32_t ordered_for = 0;
};

namespace grab {

// nearest centroids of each query, nearest first (entry_probe.hip); the layer must have groups
int entry_layer_probe_async(grab_entry_layer* L, const float* d_queries, size_t nq, int metric, uint32_t nprobe,
                            uint32_t* d_out_groups, float* kernel_ms, hipStream_t st);
// The walk over the groups when the base is in timestamp order and at most 16 groups are probed: sixteen lanes a
// query, window to id interval through the pivot levels, the in-window members of the groups in d_groups listed
// (entry_probe.hip).  d_id_lo / d_id_hi may be null.
int entry_layer_list16_async(grab_entry_layer* L, const uint32_t* d_groups, size_t nq, const uint64_t* d_win_start, const uint64_t* d_win_end,
                             uint64_t win_start, uint64_t win_end, int per_query_window, const uint64_t* d_base_ts, uint64_t* d_id_lo,
                             uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows, uint32_t max_ids, uint32_t* d_out_ids, hipStream_t st);
// Seeds from the coarse level (entry_layer.hip): the nearest centroids of every query, then the in-window members of
// their groups - scored and the n_seeds nearest kept, or (list_only) listed.  d_probe: [nq, nprobe] scratch for the
// nearest centroids; null = the layer's own buffer, which calls that overlap on two streams must not share.
int entry_layer_select_grouped_async(grab_entry_layer* L, const float* d_queries, size_t nq, int metric,
                                     const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                                     uint64_t win_end, int per_query_window, const uint64_t* d_base_ts, size_t num_base,
                                     uint64_t* d_id_lo, uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows, uint32_t n_seeds,
                                     uint32_t* d_out_seeds, float* kernel_ms, hipStream_t st, bool list_only, uint32_t* d_probe);
// the zero-padded copy of the centroids that the ranking kernel reads (after the coarse layer exists)
int entry_layer_pad_centroids(grab_entry_layer* L);
// pivot levels over the base timestamps (entry_probe.hip)
int entry_layer_build_pivots(grab_entry_layer* L, const uint64_t* d_base_ts, size_t num_base);

}  // namespace grab
