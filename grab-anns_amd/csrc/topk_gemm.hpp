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
    int drop_self = 0;            // kNN-graph mode: remove the row's own id, emit u32 ids
    uint32_t* out_u32 = nullptr;  // [M, k] when drop_self
    int64_t* out_i64 = nullptr;   // [M, k] otherwise
    float* out_dist = nullptr;
};

// kernel_ms (optional): duration of the contraction kernel from HIP events
int exact_topk(const TopkProblem& p, hipStream_t stream, float* kernel_ms);

}  // namespace grab
