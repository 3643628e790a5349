// Exact top-k of every row of A against all rows of B, as a dense fp32 MFMA contraction with
// a running per-row threshold, followed by exact re-scoring.
//
// Used twice:
//   * kNN graph (A = B = dataset): stands in for generate_knn_graph, src/index/cagra.cu:69-210
//     (IVF-PQ candidates + exact refine there) and for the RAFT brute-force self-join of
//     src/index/raft_help.cuh:74-172;
//   * filtered ground truth (A = queries): compute_ground_truth_range of the reference's
//     drivers, tests/test_cagra_auto.cu:57-89.
//
// Stage 1 (tile_topk_kernel): a 256-thread workgroup owns 128 rows of A and sweeps column
// tiles of 128 rows of B.  Both tiles are staged through LDS in 32-wide K chunks; each wave
// computes a 64x64 block with v_mfma_f32_32x32x2f32.  The epilogue turns dot products into
// distances (|a|^2 + |b|^2 - 2ab, or -ab), applies the row's filter to the column and appends
// (distance,id) keys below the row's current threshold to a workgroup-private buffer in device
// memory.  When a row's buffer is nearly full one wave sorts it, keeps the kk best and lowers
// the threshold.  The result is the exact set of the kk smallest keys under the GEMM-form
// distance.
// Stage 2 (refine_kernel): one wave per row re-scores the kept candidates in the canonical
// summation order, sorts them by (distance,id) and writes the first k.  kk carries slack so
// that rounding differences between the two distance forms cannot push a true neighbour out.
#include <algorithm>

#include "common.hpp"
#include "device_utils.hpp"
#include "topk_gemm.hpp"

namespace grab {
using namespace dev;
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int TM = 128, TN = 128, KC = 32, LDS_STRIDE = KC + 4;
constexpr int CAP = 1024;                 // per-row candidate buffer (keys)
constexpr int COMPACT_AT = CAP - TN;      // a tile appends at most TN keys to a row

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
    uint64_t* buf;       // [gridDim.x][TM][CAP]
    uint64_t* cand_out;  // [M][nsplit*kk]
    uint64_t win_start, win_end;
    uint32_t M, N, dim, kk, nsplit, col_tiles, tiles_per_split, row_tiles;
    int per_query_window;
};

struct TileLds {
    float As[TM][LDS_STRIDE];
    float Bs[TN][LDS_STRIDE];
    uint64_t thr[TM];
    uint64_t fa[TM];   // range: window start / mask: allowed-label mask
    uint64_t fb[TM];   // range: window end
    float na[TM];
    uint32_t cnt[TM];
};

// one wave: sort the row's buffer, keep the kk smallest keys, lower the threshold
__device__ __forceinline__ void compact_row(TileLds& s, uint64_t* rowbuf, int r, uint32_t kk, int lane) {
    const uint32_t n = s.cnt[r];
    uint64_t k[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t g = lane * 16 + i;
        k[i] = g < n ? rowbuf[g] : kInvalidKey;
    }
    wave_bitonic_sort<16>(k);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t g = lane * 16 + i;
        if (g < kk) rowbuf[g] = k[i];
        if (g == kk - 1) s.thr[r] = k[i];
    }
    if (lane == 0) s.cnt[r] = n < kk ? n : kk;
}

template <int METRIC, int FILTER>
// two waves per SIMD: keeps the 64 accumulator registers plus the epilogue under 256 VGPRs
__global__ void __launch_bounds__(256, 2) tile_topk_kernel(const TileArgs a) {
    __shared__ TileLds s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1, half = lane >> 5, l32 = lane & 31;
    uint64_t* myBuf = a.buf + (size_t)blockIdx.x * TM * CAP;
    const uint32_t nwork = a.row_tiles * a.nsplit;
    const uint32_t kchunks = (a.dim + KC - 1) / KC;

    for (uint32_t work = blockIdx.x; work < nwork; work += gridDim.x) {
        const uint32_t rt = work / a.nsplit, sp = work - rt * a.nsplit;
        const uint32_t row0 = rt * TM;
        const uint32_t ct_begin = sp * a.tiles_per_split;
        const uint32_t ct_end = min(a.col_tiles, ct_begin + a.tiles_per_split);

        __syncthreads();  // previous work item fully drained
        if (tid < TM) {
            const uint32_t row = row0 + tid;
            s.thr[tid] = kInvalidKey;
            s.cnt[tid] = 0;
            s.na[tid] = (METRIC == kMetricL2 && row < a.M) ? a.normA[row] : 0.0f;
            if (FILTER == kFilterRange) {
                s.fa[tid] = row < a.M ? (a.per_query_window ? a.win_start_arr[row] : a.win_start) : 0;
                s.fb[tid] = row < a.M ? (a.per_query_window ? a.win_end_arr[row] : a.win_end) : 0;
            } else if (FILTER == kFilterMask) {
                s.fa[tid] = row < a.M ? a.masks[row] : 0;
            }
        }

        for (uint32_t ct = ct_begin; ct < ct_end; ++ct) {
            const uint32_t col0 = ct * TN;
            v16f acc[2][2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int jx = 0; jx < 2; ++jx)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[i][jx][v] = 0.0f;

            for (uint32_t kc = 0; kc < kchunks; ++kc) {
                __syncthreads();
                // stage the K chunk of both tiles: 8 consecutive threads read 128 contiguous bytes
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int idx = tid + 256 * i, r = idx >> 3, c4 = idx & 7;
                    const uint32_t kcol = kc * KC + c4 * 4;
                    float4 va = make_float4(0.f, 0.f, 0.f, 0.f), vb = va;
                    if (kcol < a.dim) {
                        if (row0 + r < a.M) va = *reinterpret_cast<const float4*>(a.A + (size_t)(row0 + r) * a.dim + kcol);
                        if (col0 + r < a.N) vb = *reinterpret_cast<const float4*>(a.B + (size_t)(col0 + r) * a.dim + kcol);
                    }
                    *reinterpret_cast<float4*>(&s.As[r][c4 * 4]) = va;
                    *reinterpret_cast<float4*>(&s.Bs[r][c4 * 4]) = vb;
                }
                __syncthreads();
                // lanes 0-31 take k = 0..15 of the chunk, lanes 32-63 take k = 16..31: any
                // assignment of k to the two MFMA k-slots gives the same sum
                const float* pa0 = &s.As[wr * 64 + l32][half * 16];
                const float* pa1 = &s.As[wr * 64 + 32 + l32][half * 16];
                const float* pb0 = &s.Bs[wc * 64 + l32][half * 16];
                const float* pb1 = &s.Bs[wc * 64 + 32 + l32][half * 16];
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const float4 a0 = *reinterpret_cast<const float4*>(pa0 + q4 * 4);
                    const float4 a1 = *reinterpret_cast<const float4*>(pa1 + q4 * 4);
                    const float4 b0 = *reinterpret_cast<const float4*>(pb0 + q4 * 4);
                    const float4 b1 = *reinterpret_cast<const float4*>(pb1 + q4 * 4);
                    const float av0[4] = {a0.x, a0.y, a0.z, a0.w}, av1[4] = {a1.x, a1.y, a1.z, a1.w};
                    const float bv0[4] = {b0.x, b0.y, b0.z, b0.w}, bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv0[e], acc[0][0], 0, 0, 0);
                        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv1[e], acc[0][1], 0, 0, 0);
                        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv0[e], acc[1][0], 0, 0, 0);
                        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv1[e], acc[1][1], 0, 0, 0);
                    }
                }
            }

            // ---- epilogue: distances, filter, threshold, append ----
#pragma unroll
            for (int jx = 0; jx < 2; ++jx) {
                const uint32_t gcol = col0 + wc * 64 + jx * 32 + l32;
                const bool col_ok = gcol < a.N;
                float nb = 0.0f;
                uint64_t cts = 0;
                uint32_t clabel = 0;
                if (col_ok) {
                    if (METRIC == kMetricL2) nb = a.normB[gcol];
                    if (FILTER == kFilterRange) cts = a.ts[gcol];
                    if (FILTER == kFilterMask) clabel = a.labels[gcol] & 63;
                }
#pragma unroll
                for (int i = 0; i < 2; ++i) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int r = wr * 64 + i * 32 + (v & 3) + 4 * half + 8 * (v >> 2);
                        bool ok = col_ok && (row0 + r < a.M);
                        if (FILTER == kFilterRange) ok = ok && cts >= s.fa[r] && cts < s.fb[r];
                        if (FILTER == kFilterMask) ok = ok && ((s.fa[r] >> clabel) & 1ull);
                        float d;
                        if (METRIC == kMetricL2) {
                            d = __builtin_fmaf(-2.0f, acc[i][jx][v], s.na[r] + nb);
                            d = d < 0.0f ? 0.0f : d;
                        } else {
                            d = -acc[i][jx][v];
                        }
                        const uint64_t key = make_sel_key(d, gcol);
                        if (ok && key < s.thr[r]) {
                            const uint32_t slot = atomicAdd(&s.cnt[r], 1u);
                            myBuf[(size_t)r * CAP + slot] = key;
                        }
                    }
                }
            }
            __threadfence_block();
            __syncthreads();
            for (int r = wave; r < TM; r += 4)
                if (s.cnt[r] > COMPACT_AT) compact_row(s, myBuf + (size_t)r * CAP, r, a.kk, lane);
        }

        // ---- end of this work item: final selection, write the kk keys of every row ----
        __threadfence_block();
        __syncthreads();
        for (int r = wave; r < TM; r += 4) {
            if (row0 + r >= a.M) continue;
            uint64_t* rowbuf = myBuf + (size_t)r * CAP;
            if (s.cnt[r] > a.kk) compact_row(s, rowbuf, r, a.kk, lane);
            __threadfence_block();
            const uint32_t n = s.cnt[r];
            uint64_t* out = a.cand_out + ((size_t)(row0 + r) * a.nsplit + sp) * a.kk;
            for (uint32_t g = lane; g < a.kk; g += 64) out[g] = g < n ? rowbuf[g] : kInvalidKey;
        }
    }
}

// squared norms of the rows, 8 lanes per row
__global__ void __launch_bounds__(256) row_norms_kernel(const float* x, uint32_t n, uint32_t dim, float* out) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= n) return;
    const float4* r4 = reinterpret_cast<const float4*>(x + (size_t)g * dim);
    float s = 0.0f;
    for (uint32_t c = j; c < (dim >> 2); c += 8) {
        const float4 v = r4[c];
        s = __builtin_fmaf(v.x, v.x, s);
        s = __builtin_fmaf(v.y, v.y, s);
        s = __builtin_fmaf(v.z, v.z, s);
        s = __builtin_fmaf(v.w, v.w, s);
    }
    s = group8_sum(s);
    if (j == 0) out[g] = s;
}

struct RefineArgs {
    const float* A;
    const float* B;
    const uint64_t* cand;  // [M][nc]
    uint32_t* out_u32;     // kNN mode: [M][k]
    int64_t* out_i64;      // top-k mode: [M][k]
    float* out_dist;
    uint32_t M, dim, nc, k;
    int drop_self;
};

// one wave per row: canonical re-score, sort by (distance,id), emit
template <int METRIC, int NPL>
__global__ void __launch_bounds__(256) refine_kernel(const RefineArgs a) {
    __shared__ uint64_t keys[4][64 * NPL];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= a.M) return;  // wave-uniform
    uint64_t* mykeys = keys[wave];
    const uint64_t* cand = a.cand + (size_t)row * a.nc;
    for (uint32_t g = lane; g < 64u * NPL; g += 64) mykeys[g] = g < a.nc ? cand[g] : kInvalidKey;
    __builtin_amdgcn_wave_barrier();
    const float* q = a.A + (size_t)row * a.dim;
    const int grp = lane >> 3, j = lane & 7;
    for (uint32_t c0 = 0; c0 < a.nc; c0 += 8) {
        const uint32_t c = c0 + grp;
        const uint64_t kc = c < a.nc ? mykeys[c] : kInvalidKey;  // uniform per group of 8 lanes
        if (kc != kInvalidKey) {
            const uint32_t id = (uint32_t)(kc & 0xFFFFFFFFull);
            const float d = group8_distance<METRIC>(q, a.B + (size_t)id * a.dim, a.dim, j);
            if (j == 0) mykeys[c] = make_sel_key(d, id);
        }
    }
    __builtin_amdgcn_wave_barrier();
    uint64_t k[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) k[i] = mykeys[lane * NPL + i];
    wave_bitonic_sort<NPL>(k);
#pragma unroll
    for (int i = 0; i < NPL; ++i) mykeys[lane * NPL + i] = k[i];
    __builtin_amdgcn_wave_barrier();
    if (a.drop_self) {
        // cagra.cu:181-196: skip the row's own id, keep k, pad with 0xFFFFFFFF
        // position of self among the first k+1 sorted keys (or none)
        uint32_t self_pos = 0xFFFFFFFFu;
        for (uint32_t base = 0; base < a.k + 1 && base < 64u * NPL; base += 64) {
            const uint32_t g = base + lane;
            const bool is_self = g < 64u * NPL && mykeys[g] != kInvalidKey && (uint32_t)(mykeys[g] & 0xFFFFFFFFull) == row;
            const uint64_t b = __ballot(is_self);
            if (b != 0 && self_pos == 0xFFFFFFFFu) self_pos = base + (uint32_t)__builtin_ctzll(b);
        }
        for (uint32_t o = lane; o < a.k; o += 64) {
            const uint32_t src = o + (o >= self_pos ? 1u : 0u);
            const uint64_t kk = src < 64u * NPL ? mykeys[src] : kInvalidKey;
            a.out_u32[(size_t)row * a.k + o] = kk == kInvalidKey ? kInvalidId : (uint32_t)(kk & 0xFFFFFFFFull);
        }
    } else {
        for (uint32_t o = lane; o < a.k; o += 64) {
            const uint64_t kk = o < 64u * NPL ? mykeys[o] : kInvalidKey;
            const bool valid = kk != kInvalidKey;
            a.out_i64[(size_t)row * a.k + o] = valid ? (int64_t)(kk & 0xFFFFFFFFull) : -1;
            a.out_dist[(size_t)row * a.k + o] = valid ? ord_float((uint32_t)(kk >> 32)) : kDistMax;
        }
    }
}

template <int METRIC>
int launch_tile(const TileArgs& a, int filter, uint32_t grid, hipStream_t stream) {
    switch (filter) {
        case kFilterNone: hipLaunchKernelGGL((tile_topk_kernel<METRIC, kFilterNone>), dim3(grid), dim3(256), 0, stream, a); break;
        case kFilterRange: hipLaunchKernelGGL((tile_topk_kernel<METRIC, kFilterRange>), dim3(grid), dim3(256), 0, stream, a); break;
        case kFilterMask: hipLaunchKernelGGL((tile_topk_kernel<METRIC, kFilterMask>), dim3(grid), dim3(256), 0, stream, a); break;
        default: set_error("bad filter kind %d", filter); return GRAB_ERR_INVALID;
    }
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

template <int METRIC>
int launch_refine(const RefineArgs& a, hipStream_t stream) {
    const uint32_t grid = (a.M + 3) / 4;
    if (a.nc <= 256) hipLaunchKernelGGL((refine_kernel<METRIC, 4>), dim3(grid), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((refine_kernel<METRIC, 16>), dim3(grid), dim3(256), 0, stream, a);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace

int exact_topk(const TopkProblem& p, hipStream_t stream, float* kernel_ms) {
    GRAB_REQUIRE(p.A && p.B, "null matrix");
    GRAB_REQUIRE(p.dim >= 4 && p.dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", p.dim);
    GRAB_REQUIRE(p.M > 0 && p.N > 0 && p.N < (1ull << 31), "bad problem size");
    GRAB_REQUIRE(p.k >= 1 && p.k <= 512, "k must be in [1,512]");
    int dev = 0, num_cu = 0;
    GRAB_HIP(hipGetDevice(&dev));
    GRAB_HIP(hipDeviceGetAttribute(&num_cu, hipDeviceAttributeMultiprocessorCount, dev));

    // Candidates kept per row.  The GEMM-form distance |a|^2+|b|^2-2ab is exact on small
    // integer data but loses up to ~eps*(|a|^2+|b|^2) to cancellation on general data, so the
    // exact re-scoring needs slack beyond k: at least as many extra candidates as k itself.
    const uint32_t kk = p.drop_self ? std::min<uint32_t>(std::max<uint32_t>(2 * p.k + 33, 256), 768)
                                    : std::min<uint32_t>(std::max<uint32_t>(2 * p.k + 32, 64), 768);
    const uint32_t row_tiles = (uint32_t)((p.M + TM - 1) / TM), col_tiles = (uint32_t)((p.N + TN - 1) / TN);
    const uint32_t target = (uint32_t)num_cu * 2;  // two resident workgroups per CU
    uint32_t nsplit = 1;
    if (row_tiles < target) nsplit = std::min<uint32_t>((target + row_tiles - 1) / row_tiles, std::min<uint32_t>(col_tiles, 1024 / kk));
    nsplit = std::max(nsplit, 1u);
    uint32_t tiles_per_split = (col_tiles + nsplit - 1) / nsplit;
    nsplit = (col_tiles + tiles_per_split - 1) / tiles_per_split;
    const uint32_t nwork = row_tiles * nsplit;
    const uint32_t grid = std::min(nwork, target);

    DeviceScratch buf, cand, normA, normB;
    GRAB_HIP(buf.alloc((size_t)grid * TM * CAP * sizeof(uint64_t)));
    GRAB_HIP(cand.alloc((size_t)p.M * nsplit * kk * sizeof(uint64_t)));
    const bool same = (p.A == p.B && p.M == p.N);
    if (p.metric == kMetricL2) {
        GRAB_HIP(normB.alloc((size_t)p.N * 4));
        hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((p.N * 8 + 255) / 256)), dim3(256), 0, stream, p.B,
                           (uint32_t)p.N, p.dim, normB.as<float>());
        if (!same) {
            GRAB_HIP(normA.alloc((size_t)p.M * 4));
            hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((p.M * 8 + 255) / 256)), dim3(256), 0, stream, p.A,
                               (uint32_t)p.M, p.dim, normA.as<float>());
        }
        GRAB_HIP(hipGetLastError());
    }

    TileArgs t{};
    t.A = p.A;
    t.B = p.B;
    t.normA = same ? normB.as<float>() : normA.as<float>();
    t.normB = normB.as<float>();
    t.ts = p.ts;
    t.win_start_arr = p.win_start_arr;
    t.win_end_arr = p.win_end_arr;
    t.labels = p.labels;
    t.masks = p.masks;
    t.buf = buf.as<uint64_t>();
    t.cand_out = cand.as<uint64_t>();
    t.win_start = p.win_start;
    t.win_end = p.win_end;
    t.M = (uint32_t)p.M;
    t.N = (uint32_t)p.N;
    t.dim = p.dim;
    t.kk = kk;
    t.nsplit = nsplit;
    t.col_tiles = col_tiles;
    t.tiles_per_split = tiles_per_split;
    t.row_tiles = row_tiles;
    t.per_query_window = p.per_query_window;

    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (kernel_ms) {
        GRAB_HIP(hipEventCreate(&e0));
        GRAB_HIP(hipEventCreate(&e1));
        GRAB_HIP(hipEventRecord(e0, stream));
    }
    int rc = p.metric == kMetricIP ? launch_tile<kMetricIP>(t, p.filter_kind, grid, stream)
                                   : launch_tile<kMetricL2>(t, p.filter_kind, grid, stream);
    if (kernel_ms && rc == GRAB_OK) {
        hipError_t e = hipEventRecord(e1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(kernel_ms, e0, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the contraction kernel", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    GRAB_TRY(rc);

    RefineArgs r{};
    r.A = p.A;
    r.B = p.B;
    r.cand = cand.as<uint64_t>();
    r.out_u32 = p.out_u32;
    r.out_i64 = p.out_i64;
    r.out_dist = p.out_dist;
    r.M = (uint32_t)p.M;
    r.dim = p.dim;
    r.nc = nsplit * kk;
    r.k = p.k;
    r.drop_self = p.drop_self;
    GRAB_REQUIRE(r.nc <= 1024, "internal: too many candidates per row");
    GRAB_TRY(p.metric == kMetricIP ? launch_refine<kMetricIP>(r, stream) : launch_refine<kMetricL2>(r, stream));
    GRAB_HIP(hipStreamSynchronize(stream));
    return GRAB_OK;
}

}  // namespace grab

using namespace grab;

extern "C" {

int grab_generate_knn_graph(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t k, int metric,
                            uint32_t* d_knn_graph, float* kernel_ms, void* stream) {
    GRAB_REQUIRE(d_dataset && d_knn_graph, "null pointer");
    GRAB_REQUIRE(k >= 1 && k <= GRAB_MAX_DEGREE, "k must be in [1,%d]", GRAB_MAX_DEGREE);
    TopkProblem p{};
    p.A = d_dataset;
    p.B = d_dataset;
    p.M = num_dataset;
    p.N = num_dataset;
    p.dim = dim;
    p.k = k;
    p.metric = metric;
    p.drop_self = 1;
    p.out_u32 = d_knn_graph;
    return exact_topk(p, static_cast<hipStream_t>(stream), kernel_ms);
}

int grab_bruteforce_topk(const float* d_dataset, size_t num_dataset, uint32_t dim, const float* d_queries,
                         size_t num_queries, uint32_t k, int metric, int filter_kind, const uint64_t* d_ts,
                         const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                         uint64_t win_end, int per_query_window, const uint8_t* d_labels, const uint64_t* d_masks,
                         int64_t* d_out_indices, float* d_out_dists, float* kernel_ms, void* stream) {
    GRAB_REQUIRE(d_dataset && d_queries && d_out_indices && d_out_dists, "null pointer");
    if (filter_kind == kFilterRange) {
        GRAB_REQUIRE(d_ts != nullptr, "range filter needs timestamps");
        GRAB_REQUIRE(!per_query_window || (d_win_start && d_win_end), "per-query windows missing");
    } else if (filter_kind == kFilterMask) {
        GRAB_REQUIRE(d_labels && d_masks, "mask filter needs labels and masks");
    }
    if (num_queries == 0) return GRAB_OK;
    TopkProblem p{};
    p.A = d_queries;
    p.B = d_dataset;
    p.M = num_queries;
    p.N = num_dataset;
    p.dim = dim;
    p.k = k;
    p.metric = metric;
    p.filter_kind = filter_kind;
    p.ts = d_ts;
    p.win_start_arr = d_win_start;
    p.win_end_arr = d_win_end;
    p.win_start = win_start;
    p.win_end = win_end;
    p.per_query_window = per_query_window;
    p.labels = d_labels;
    p.masks = d_masks;
    p.out_i64 = d_out_indices;
    p.out_dist = d_out_dists;
    return exact_topk(p, static_cast<hipStream_t>(stream), kernel_ms);
}

}  // extern "C"
