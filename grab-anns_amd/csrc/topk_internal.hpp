// What the translation units around the tile contraction share (topk_gemm.hip: the kernels, exact_topk; entry_layer.hip:
// the entry-point layer; scan.hip: the exact scans of buckets and id intervals): tile geometry, the argument blocks of
// the contraction and of the re-scoring, and launchers that pick the kernel instance.
#pragma once
#include <cstdint>

#include "common.hpp"
#include "topk_gemm.hpp"

namespace grab {

constexpr int TM = 128, TN = 128, KC = 32, LDS_STRIDE = KC + 4;
constexpr int TSTRIDE = 68;               // row stride of the transposed 64x64 block: 16-byte aligned rows, conflict-free b128 reads
constexpr int CAP = 1024;                 // per-row candidate buffer (keys)
constexpr int COMPACT_AT = CAP - TN;      // a tile appends at most TN keys to a row
// layout of the work list of the dense-store mode (uint32 words)
constexpr int kSchedPer = 0, kSchedItems = 1, kSchedOff = 2, kSchedLo = kSchedOff + 129, kSchedHi = kSchedLo + 128,
              kSchedWords = kSchedHi + 128;

struct TileArgs {
    const float* A;
    const float* B;
    const float* normA;
    const float* normB;
    const uint64_t* ts;
    const uint64_t* win_start_arr;
    const uint64_t* win_end_arr;
    const uint8_t* labels;
    const uint64_t* masks;
    const uint32_t* row_perm;  // optional: tile-grid row -> row of A (rows ordered by window)
    const uint32_t* row_lo;    // kFilterColRange: per row of A, admissible columns [lo,hi)
    const uint32_t* row_hi;
    float* dense;        // STORE mode: [M][dense_pitch] distances
    uint64_t dense_pitch;
    int dense_rel;       // STORE mode: a row's distances start at the first column tile of its row tile, not at column 0
    const uint32_t* sched;  // STORE mode: work list made by bucket_order_kernel
    uint64_t* buf;       // [gridDim.x][TM][CAP]
    uint64_t* cand_out;  // [M][nsplit*kk]
    // kFilterSymmetric: what a tile above the diagonal yields for the rows behind its columns
    const float* col_bound;  // [N] a row takes a key from a column walk when its distance is <= this
    uint64_t* col_list;      // [N][col_cap] keys (distance, row of A), in arrival order
    uint32_t* col_count;     // [N] keys offered to a row (may exceed col_cap: the row is then redone the plain way)
    uint32_t col_cap;
    // optional, zero before the launch: work items are handed out through it in their order, to whichever workgroup is
    // free, instead of in equal shares (the two workgroups of a CU do not run at the same pace)
    uint32_t* work_counter;
    int cand_by_grid_row;    // cand_out is indexed by the tile-grid row instead of the row of A
    int range_by_grid_row;   // kFilterColRange: so are row_lo / row_hi (several tile-grid rows may stand for one row of A)
    uint64_t win_start, win_end;
    uint32_t M, N, dim, kk, nsplit, col_tiles, tiles_per_split, row_tiles;
    int per_query_window;
};

struct RefineArgs {
    const float* A;
    const float* B;
    const uint64_t* cand;  // [M][nc]
    uint32_t* out_u32;     // kNN mode: [M][k]
    int64_t* out_i64;      // top-k mode: [M][k]
    float* out_dist;
    uint32_t M, dim, nc, k;
    int drop_self;
    // certificate (optional): nc = nsplit lists of kk keys, each the kk smallest GEMM-form keys of its columns
    uint32_t kk;
    const float* normA;      // squared norm of every row of A
    const float* max_normB;  // one float: the largest squared norm among the rows of B
    // candidates that may (also) come from the split-bf16 pass over centred rows: the norms it used, and its error
    const float* split_normA;      // null: none do
    const float* split_max_normB;
    float split_terms;             // products that one of its fp32 sums runs over (3 * 128 + 6, or 3 * dim)
    int sorted;                    // every row's candidates are one list in ascending order (the symmetric pass leaves them so)
    const float* outside_in; // optional, per row: a bound like `outside` below that the lists themselves no longer show (they were merged)
    uint32_t* doubt;         // rows whose result the candidates do not prove, doubt[0] = how many, then the rows; null = no check
    const uint32_t* rows;    // optional: only these rows (M of them)
};

// selection inside the contraction (tile_topk_kernel<METRIC, FILTER, false, SPLIT>): a.cand_out receives kk keys per row and split
int launch_tile_any(const TileArgs& a, int metric, int filter, uint32_t grid, hipStream_t stream, bool split = false);
// distances of the swept columns to a.dense (tile_topk_kernel<METRIC, kFilterColRange, true, SPLIT>), work list in a.sched
int launch_tile_store(const TileArgs& a, int metric, uint32_t grid, hipStream_t stream, bool split = false);
int launch_refine_any(const RefineArgs& a, int metric, hipStream_t stream);
// squared norms of n rows; the largest of n non-negative floats (atomic max into *out, which the caller has zeroed);
// the mean of `count` evenly spaced rows; rows as bf16 halves per chunk of 32 dimensions (minus `mean` if given) and
// the squared norms of what was split
void launch_row_norms(const float* x, size_t n, uint32_t dim, float* out, hipStream_t stream);
void launch_max_float(const float* x, uint64_t n, uint32_t* out, hipStream_t stream);
void launch_spaced_mean(const float* data, uint64_t n, uint32_t count, uint32_t dim, float* mean, hipStream_t stream);
void launch_split_rows_chunked(const float* data, uint64_t n, uint32_t dim, const float* mean, uint16_t* out, float* norm,
                               hipStream_t stream);

// matrix work and redone rows of the calling thread's last exact_topk / scan (grab_last_knn_stats and its kin)
struct KnnStats {
    double flop = 0.0;          // fp32 matrix instructions
    double flop_bf16 = 0.0;     // bf16 matrix instructions (three per product of split rows)
    uint64_t redone_rows = 0;   // rows the symmetric pass handed to the plain pass
    uint64_t exact_rows = 0;    // rows (queries) that their candidates did not prove and an exact pass redid
};
KnnStats& knn_stats();
bool knn_bf16_allowed();  // grab_knn_allow_bf16

}  // namespace grab
