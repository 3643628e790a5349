// Exact top-k of the rows of A against the rows of B (see topk_gemm.hip).
#pragma once
#include "common.hpp"

namespace grab {

struct TopkProblem {
    const float* A = nullptr;  // [M, dim] query rows
    const float* B = nullptr;  // [N, dim] base rows
    size_t M = 0, N = 0;
    uint32_t dim = 0, k = 0;
    int metric = 0;
    int filter_kind = 0;  // applied to (row of A, row of B)
    const uint64_t* ts = nullptr;
    const uint64_t* win_start_arr = nullptr;
    const uint64_t* win_end_arr = nullptr;
    uint64_t win_start = 0, win_end = 0;
    int per_query_window = 0;
    const uint8_t* labels = nullptr;
    const uint64_t* masks = nullptr;
    const uint32_t* row_lo = nullptr;  // filter_kind 3 here: a row of A admits the columns [row_lo, row_hi) of B, and only the
    const uint32_t* row_hi = nullptr;  // column tiles that some row of a row tile admits are visited
    int drop_self = 0;            // kNN-graph mode: remove the row's own id, emit u32 ids
    uint32_t* out_u32 = nullptr;  // [M, k] when drop_self
    int64_t* out_i64 = nullptr;   // [M, k] otherwise
    float* out_dist = nullptr;
};

// kernel_ms (optional): duration of the contraction kernel from HIP events
int exact_topk(const TopkProblem& p, hipStream_t stream, float* kernel_ms);

// Per-row bounds for the symmetric pass of exact_topk, estimated with bf16 matrix instructions (bound_bf16.hip):
// for every row of `data` (n x dim fp32, dim <= 128, squared L2) about its distance to the rank-th nearest of
// n_sample evenly spaced rows.  The ranks that the estimate can stand in for end at bf16_bound_classes() / 2.
// Everything is queued on `stream`; `workspace` holds bf16_bound_workspace_bytes(n, n_sample) bytes.
// Left behind in the workspace for the symmetric pass on the same pipe: *split_rows = the centred rows as [n][272]
// bf16 (128 high halves, 128 low halves, zeros beyond dim, 16 values that carry -|row|^2/2 for a k-step of its own),
// followed by kSplitPadRows rows of zeros (that pass reads whole column tiles of 128 rows without looking at n);
// *centred_norms = the squared norms of the centred fp32 rows.
constexpr uint32_t kSplitPadRows = 128;
uint32_t bf16_bound_classes();
size_t bf16_bound_workspace_bytes(size_t n, uint32_t n_sample);
int bf16_bounds_async(const float* data, uint32_t n, uint32_t dim, uint32_t n_sample, uint32_t rank, void* workspace, float* bound,
                      hipStream_t stream, const uint16_t** split_rows, const float** centred_norms);

}  // namespace grab
