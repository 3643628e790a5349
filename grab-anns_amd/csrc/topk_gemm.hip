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
// For a large row set against itself (the kNN graph) only the tiles on and above the diagonal are
// computed: a tile also yields the keys of the dataset rows behind its columns, kept in per-row
// lists in device memory when they are within a bound that a first pass against a sample of the
// rows has set; merge_symmetric_kernel puts a row's two halves together and names the rows for
// which the bound admitted too few or too many keys, which the plain pass then redoes.
// Stage 2 (refine_kernel): one wave per row re-scores the kept candidates in the canonical
// summation order, sorts them by (distance,id) and writes the first k.  kk carries slack so
// that rounding differences between the two distance forms cannot push a true neighbour out.
#include <algorithm>
#include <atomic>
#include <functional>
#include <type_traits>
#include <vector>

#include "common.hpp"
#include "device_sort.hpp"
#include "device_utils.hpp"
#include "entry_layer.hpp"
#include "topk_gemm.hpp"

namespace grab {
using namespace dev;
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __attribute__((ext_vector_type(8))) __bf16 v8bf16;

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
    int cand_by_grid_row;    // cand_out is indexed by the tile-grid row instead of the row of A
    int range_by_grid_row;   // kFilterColRange: so are row_lo / row_hi (several tile-grid rows may stand for one row of A)
    uint64_t win_start, win_end;
    uint32_t M, N, dim, kk, nsplit, col_tiles, tiles_per_split, row_tiles;
    int per_query_window;
};

struct TileLds {
    float As[2][TM][LDS_STRIDE];  // double-buffered K chunks
    float Bs[2][TN][LDS_STRIDE];
    uint64_t thr[TM];
    uint64_t fa[TM];   // range: window start / mask: allowed-label mask
    uint64_t fb[TM];   // range: window end
    float na[TM];
    uint32_t cnt[TM];
    float cnb[4][64];      // epilogue: norms of the wave's 64 columns
    uint64_t cfw[4][64];   // epilogue: filter word (timestamp or label) of the wave's 64 columns
    uint32_t arow[TM];  // row of A behind each tile row, 0xFFFFFFFF past the end
    uint32_t tlo, thi;  // kFilterColRange: union of the rows' column ranges
};

// one wave: sort the row's buffer, keep the kk smallest keys, lower the threshold
template <int NPL, class Lds>
__device__ __forceinline__ void compact_row_n(Lds& s, uint64_t* rowbuf, int r, uint32_t kk, int lane) {
    const uint32_t n = s.cnt[r];
    uint64_t k[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const uint32_t g = lane * NPL + i;
        k[i] = g < n ? rowbuf[g] : kInvalidKey;
    }
    wave_bitonic_sort<NPL>(k);
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const uint32_t g = lane * NPL + i;
        if (g < kk) rowbuf[g] = k[i];
        if (g == kk - 1) s.thr[r] = k[i];
    }
    if (lane == 0) s.cnt[r] = n < kk ? n : kk;
}
template <class Lds>
__device__ __forceinline__ void compact_row(Lds& s, uint64_t* rowbuf, int r, uint32_t kk, int lane) {
    if (s.cnt[r] <= 256) compact_row_n<4>(s, rowbuf, r, kk, lane);
    else compact_row_n<16>(s, rowbuf, r, kk, lane);
}

// STORE: instead of selecting, the distances of the visited tiles are written to a dense
// matrix a.dense[tile-grid row][column] (row pitch a.dense_pitch); a streaming kernel selects later.
// SPLIT: a.A and a.B hold rows made by split_rows_chunked_kernel - per chunk of 32 dimensions the 32 bf16 high halves,
// then the 32 low halves (x = hi + lo + what is left, |left| <= 2^-16 |x|): 128 bytes a chunk like the fp32 row, so
// the loads and the LDS tiles are the fp32 kernel's byte for byte.  The products come from v_mfma_f32_32x32x16_bf16 as
// lo.hi + hi.lo + hi.hi with fp32 sums - 24 instructions a chunk where the fp32 path issues 64 that take twice as
// long each - off the true dot product by at most 3 * 2^-16 |a||b|.  What such a pass returns are candidates; the
// exact re-scoring and the check after it (refine_kernel, which is told the larger error) decide the result.
template <int METRIC, int FILTER, bool STORE, bool SPLIT = false>
// two waves per SIMD: keeps the 64 accumulator registers plus the epilogue under 256 VGPRs
__global__ void __launch_bounds__(256, 2) tile_topk_kernel(const TileArgs a) {
    extern __shared__ __align__(16) uint8_t tile_smem[];
    TileLds& s = *reinterpret_cast<TileLds*>(tile_smem);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1, half = lane >> 5, l32 = lane & 31;
    uint64_t* myBuf = a.buf + (size_t)blockIdx.x * TM * CAP;
    const uint32_t kchunks = (a.dim + KC - 1) / KC;
    // STORE: the work list (items of `per` column tiles, all non-empty) lives in LDS that the
    // selection path would use for thresholds and filter words
    uint32_t* item_off = reinterpret_cast<uint32_t*>(s.thr);  // [row_tiles+1]
    uint32_t* tile_rng = reinterpret_cast<uint32_t*>(s.cfw);  // [0..127] first, [128..255] end column tile
    uint32_t nwork = a.row_tiles * a.nsplit, per_item = 0;
    if (STORE) {
        per_item = a.sched[kSchedPer];
        nwork = a.sched[kSchedItems];
        if (tid <= (int)a.row_tiles) item_off[tid] = a.sched[kSchedOff + tid];
        if (tid < (int)a.row_tiles) {
            tile_rng[tid] = a.sched[kSchedLo + tid];
            tile_rng[128 + tid] = a.sched[kSchedHi + tid];
        }
    }

    for (uint32_t base = 0; base < nwork; base += gridDim.x) {
        // Symmetric pass: row tile rt sweeps the column tiles from rt on, so the items shrink with rt.  Every other
        // round hands them out in reverse, which evens out the sums of a workgroup's items.
        uint32_t work = base + blockIdx.x;
        if (FILTER == kFilterSymmetric && ((base / gridDim.x) & 1u)) work = base + (gridDim.x - 1 - blockIdx.x);
        if (work >= nwork) continue;  // workgroup-uniform
        __syncthreads();  // previous work item fully drained (and the work list visible)
        uint32_t rt, sp;
        if (STORE) {
            uint32_t lo_rt = 0, hi_rt = a.row_tiles;  // largest rt with item_off[rt] <= work
            while (hi_rt - lo_rt > 1) {
                const uint32_t mid = (lo_rt + hi_rt) >> 1;
                if (item_off[mid] <= work) lo_rt = mid; else hi_rt = mid;
            }
            rt = lo_rt;
            sp = work - item_off[rt];
        } else {
            rt = work / a.nsplit;
            sp = work - rt * a.nsplit;
        }
        const uint32_t row0 = rt * TM;

        if (tid == 0) {
            s.tlo = 0xFFFFFFFFu;
            s.thi = 0;
        }
        float na_pending = 0.0f;
        if (tid < TM) {
            const uint32_t row = row0 + tid;
            const bool valid = row < a.M;
            const uint32_t ar = valid ? (a.row_perm ? a.row_perm[row] : row) : 0xFFFFFFFFu;
            s.arow[tid] = ar;
            // symmetric pass: nothing beyond the row's bound is of use (the merge drops it), so the threshold starts there
            if (!STORE) s.thr[tid] = (FILTER == kFilterSymmetric && valid) ? (((uint64_t)ord_bits(a.col_bound[ar]) << 32) | 0xFFFFFFFFull) : kInvalidKey;
            s.cnt[tid] = 0;
            // STORE: the norm is only needed by the epilogue; it goes to LDS with the first chunk
            if (STORE) na_pending = (METRIC == kMetricL2 && valid) ? a.normA[ar] : 0.0f;
            else s.na[tid] = (METRIC == kMetricL2 && valid) ? a.normA[ar] : 0.0f;
            if (STORE) {
                // nothing to filter: the selection pass applies the row's column range.  Rows that start at their row tile's
                // first column tile come with their ranges, so that what no pass will read is not written
                if (a.dense_rel) {
                    s.fa[tid] = valid ? a.row_lo[row] : 0;
                    s.fb[tid] = valid ? a.row_hi[row] : 0;
                }
            } else if (FILTER == kFilterRange) {
                s.fa[tid] = valid ? (a.per_query_window ? a.win_start_arr[ar] : a.win_start) : 0;
                s.fb[tid] = valid ? (a.per_query_window ? a.win_end_arr[ar] : a.win_end) : 0;
            } else if (FILTER == kFilterMask) {
                s.fa[tid] = valid ? a.masks[ar] : 0;
            } else if (FILTER == kFilterColRange) {
                s.fa[tid] = valid ? a.row_lo[a.range_by_grid_row ? row : ar] : 0;
                s.fb[tid] = valid ? a.row_hi[a.range_by_grid_row ? row : ar] : 0;
            }
        }
        uint32_t ct_begin = sp * a.tiles_per_split;
        uint32_t ct_end = min(a.col_tiles, ct_begin + a.tiles_per_split);
        if (FILTER == kFilterSymmetric) ct_begin = max(ct_begin, rt);  // the tiles below the diagonal are mirrored ones
        if (STORE) {
            ct_begin = tile_rng[rt] + sp * per_item;
            ct_end = min(tile_rng[128 + rt], ct_begin + per_item);
        } else if (FILTER == kFilterColRange) {
            // only the column tiles that some row of this tile admits are visited
            __syncthreads();
            if (tid < TM && s.fa[tid] < s.fb[tid]) {
                atomicMin(&s.tlo, (uint32_t)s.fa[tid]);
                atomicMax(&s.thi, (uint32_t)s.fb[tid]);
            }
            __syncthreads();
            const uint32_t c_lo = s.tlo / TN, c_hi = s.tlo < s.thi ? (s.thi + TN - 1) / TN : c_lo;
            const uint32_t per = (c_hi - c_lo + a.nsplit - 1) / a.nsplit;
            ct_begin = c_lo + sp * per;
            ct_end = min(c_hi, ct_begin + per);
            if (per == 0) ct_end = ct_begin;
        }

        // Software pipeline: the global loads of the next K chunk (or of the first chunk of the
        // next column tile) are issued before the MFMAs of the current chunk and land in
        // registers while those run; LDS is double-buffered, so one barrier per chunk suffices.
        // (On split rows a chunk is 24 short matrix instructions, far less than the way of a load.  A second chunk in
        // flight, in a second set of registers, would cover it - and does not fit: the kernel holds 234 of its 256
        // registers, and with the second set 150 of them go to scratch memory, which costs more than the waiting.)
        float4 ra[4], rb[4];
        // Whole tiles of whole chunks (all but the rim of the problem) take the short way: the thread's four row
        // pointers into A are fixed for the work item, those into B are 32 rows apart, and a chunk is a fixed step
        // along them - a few address additions per chunk instead of a bounds test and a 64-bit product per load.
        const float4* pa[4] = {nullptr, nullptr, nullptr, nullptr};
        const bool whole_rows = row0 + TM <= a.M && (a.dim % KC) == 0;
        auto load_chunk = [&](float4 (&ra)[4], float4 (&rb)[4], uint32_t col0, uint32_t kc) {
            if (whole_rows && col0 + TN <= a.N) {  // workgroup-uniform
                const float4* pb = reinterpret_cast<const float4*>(a.B + (size_t)(col0 + (tid >> 3)) * a.dim) + (tid & 7) + kc * (KC / 4);
                const size_t rows32 = (size_t)8 * a.dim;  // 32 rows, in float4
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    ra[i] = pa[i][kc * (KC / 4)];
                    rb[i] = pb[i * rows32];
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int idx = tid + 256 * i, r = idx >> 3, c4 = idx & 7;
                const uint32_t kcol = kc * KC + c4 * 4;
                ra[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                rb[i] = ra[i];
                if (kcol < a.dim) {
                    const uint32_t ar = s.arow[r];
                    if (ar != 0xFFFFFFFFu) ra[i] = *reinterpret_cast<const float4*>(a.A + (size_t)ar * a.dim + kcol);
                    if (col0 + r < a.N) rb[i] = *reinterpret_cast<const float4*>(a.B + (size_t)(col0 + r) * a.dim + kcol);
                }
            }
        };
        __syncthreads();  // row table visible
        if (whole_rows) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                pa[i] = reinterpret_cast<const float4*>(a.A + (size_t)s.arow[(tid >> 3) + 32 * i] * a.dim) + (tid & 7);
        }
        if (ct_begin < ct_end) load_chunk(ra, rb, ct_begin * TN, 0);
        int buf = 0;

        for (uint32_t ct = ct_begin; ct < ct_end; ++ct) {
            const uint32_t col0 = ct * TN;
            v16f acc[2][2];  // written by the first chunk (kchunks >= 1: dim >= 4)

            // one chunk: `xa`, `xb` hold it; the next chunk takes their place once they are parked in LDS
            auto step = [&](uint32_t kc, float4 (&xa)[4], float4 (&xb)[4]) {
                // 8 consecutive threads hold 128 contiguous bytes of a row
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int idx = tid + 256 * i, r = idx >> 3, c4 = idx & 7;
                    *reinterpret_cast<float4*>(&s.As[buf][r][c4 * 4]) = xa[i];
                    *reinterpret_cast<float4*>(&s.Bs[buf][r][c4 * 4]) = xb[i];
                }
                if (STORE && ct == ct_begin && kc == 0 && tid < TM) s.na[tid] = na_pending;
                __syncthreads();
                if (kc + 1 < kchunks) load_chunk(xa, xb, col0, kc + 1);
                else if (ct + 1 < ct_end) load_chunk(xa, xb, col0 + TN, 0);
                // lanes 0-31 take k = 0..15 of the chunk, lanes 32-63 take k = 16..31: any
                // assignment of k to the two MFMA k-slots gives the same sum
                const float* pa0 = &s.As[buf][wr * 64 + l32][half * 16];
                const float* pa1 = &s.As[buf][wr * 64 + 32 + l32][half * 16];
                const float* pb0 = &s.Bs[buf][wc * 64 + l32][half * 16];
                const float* pb1 = &s.Bs[buf][wc * 64 + 32 + l32][half * 16];
                // the first chunk of a tile starts from the constant 0 as the matrix instruction's addend, which
                // spares the 64 register moves of a zeroed accumulator block
                auto chunk = [&](auto first_chunk) {
                    constexpr bool FIRST = decltype(first_chunk)::value;
                    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    if constexpr (SPLIT) {
                        // a row's chunk in LDS: bytes 0-63 the high halves of k = 0..31, bytes 64-127 the low halves.  For
                        // k-step ks (16 values of k) lane (l32, half) holds k = 16 ks + 8 half .. + 7 of its row or column.
                        const uint8_t* ra0 = reinterpret_cast<const uint8_t*>(&s.As[buf][wr * 64 + l32][0]) + 16 * half;
                        const uint8_t* ra1 = reinterpret_cast<const uint8_t*>(&s.As[buf][wr * 64 + 32 + l32][0]) + 16 * half;
                        const uint8_t* rb0 = reinterpret_cast<const uint8_t*>(&s.Bs[buf][wc * 64 + l32][0]) + 16 * half;
                        const uint8_t* rb1 = reinterpret_cast<const uint8_t*>(&s.Bs[buf][wc * 64 + 32 + l32][0]) + 16 * half;
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const v8bf16 ah0 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(ra0 + 32 * ks));
                            const v8bf16 al0 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(ra0 + 64 + 32 * ks));
                            const v8bf16 ah1 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(ra1 + 32 * ks));
                            const v8bf16 al1 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(ra1 + 64 + 32 * ks));
                            const v8bf16 bh0 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(rb0 + 32 * ks));
                            const v8bf16 bl0 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(rb0 + 64 + 32 * ks));
                            const v8bf16 bh1 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(rb1 + 32 * ks));
                            const v8bf16 bl1 = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(rb1 + 64 + 32 * ks));
                            const bool z = FIRST && ks == 0;
                            // the small terms first; consecutive instructions go to different accumulators
                            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al0, bh0, z ? zero : acc[0][0], 0, 0, 0);
                            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al0, bh1, z ? zero : acc[0][1], 0, 0, 0);
                            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al1, bh0, z ? zero : acc[1][0], 0, 0, 0);
                            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al1, bh1, z ? zero : acc[1][1], 0, 0, 0);
                            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah0, bl0, acc[0][0], 0, 0, 0);
                            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah0, bl1, acc[0][1], 0, 0, 0);
                            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah1, bl0, acc[1][0], 0, 0, 0);
                            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah1, bl1, acc[1][1], 0, 0, 0);
                            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah0, bh0, acc[0][0], 0, 0, 0);
                            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah0, bh1, acc[0][1], 0, 0, 0);
                            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah1, bh0, acc[1][0], 0, 0, 0);
                            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah1, bh1, acc[1][1], 0, 0, 0);
                        }
                        return;
                    }
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
                            const bool z = FIRST && q4 == 0 && e == 0;
                            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv0[e], z ? zero : acc[0][0], 0, 0, 0);
                            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[e], bv1[e], z ? zero : acc[0][1], 0, 0, 0);
                            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv0[e], z ? zero : acc[1][0], 0, 0, 0);
                            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[e], bv1[e], z ? zero : acc[1][1], 0, 0, 0);
                        }
                    }
                };
                if (kc == 0) chunk(std::true_type{});
                else chunk(std::false_type{});
                buf ^= 1;
            };
            for (uint32_t kc = 0; kc < kchunks; ++kc) step(kc, ra, rb);

            // ---- epilogue: distances, filter, threshold, append ----
            // The wave's 64x64 block of dot products goes through LDS (the tile buffers are
            // idle now) so that each lane can walk ONE row: the row's norm, filter words and
            // threshold stay in registers, no two lanes of a wave append to the same row, and
            // the accumulators are dead before the next tile's prefetched chunk is stored.
            if (STORE) {
                // the wave's 64x64 block goes through LDS so that a lane owns four consecutive
                // columns of a row: 16-byte stores, 256 contiguous bytes per row and instruction
                __syncthreads();  // every wave is done reading the tile buffers
                float* T = reinterpret_cast<float*>(&s.As[0][0][0]) + wave * (64 * TSTRIDE);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int jx = 0; jx < 2; ++jx)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            T[(i * 32 + (v & 3) + 4 * half + 8 * (v >> 2)) * TSTRIDE + jx * 32 + l32] = acc[i][jx][v];
                const int c4 = lane & 15, rsub = lane >> 4;
                const uint32_t gcol = col0 + wc * 64 + c4 * 4;
                const uint32_t dcol = gcol - (a.dense_rel ? tile_rng[rt] * TN : 0u);
                float4 nb = make_float4(0.f, 0.f, 0.f, 0.f);
                if (METRIC == kMetricL2) {
                    if (gcol + 3 < a.N) {
                        nb = *reinterpret_cast<const float4*>(a.normB + gcol);
                    } else {
                        if (gcol < a.N) nb.x = a.normB[gcol];
                        if (gcol + 1 < a.N) nb.y = a.normB[gcol + 1];
                        if (gcol + 2 < a.N) nb.z = a.normB[gcol + 2];
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll 4
                for (int rr = 0; rr < 16; ++rr) {
                    const int r = rr * 4 + rsub;
                    const float4 t = *reinterpret_cast<const float4*>(T + r * TSTRIDE + c4 * 4);
                    float4 d;
                    if (METRIC == kMetricL2) {
                        const float na = s.na[wr * 64 + r];
                        d.x = __builtin_fmaf(-2.0f, t.x, na + nb.x);
                        d.y = __builtin_fmaf(-2.0f, t.y, na + nb.y);
                        d.z = __builtin_fmaf(-2.0f, t.z, na + nb.z);
                        d.w = __builtin_fmaf(-2.0f, t.w, na + nb.w);
                        d.x = d.x < 0.0f ? 0.0f : d.x;
                        d.y = d.y < 0.0f ? 0.0f : d.y;
                        d.z = d.z < 0.0f ? 0.0f : d.z;
                        d.w = d.w < 0.0f ? 0.0f : d.w;
                    } else {
                        d = make_float4(-t.x, -t.y, -t.z, -t.w);
                    }
                    // the pitch is a whole number of tiles: columns past N are written and never read
                    const uint32_t grow = row0 + wr * 64 + r;
                    bool wanted = grow < a.M;
                    if (a.dense_rel) wanted = wanted && gcol < (uint32_t)s.fb[wr * 64 + r] && gcol + 4u > (uint32_t)s.fa[wr * 64 + r];
                    if (wanted) *reinterpret_cast<float4*>(a.dense + (size_t)grow * a.dense_pitch + dcol) = d;
                }
                __syncthreads();  // the block is consumed before the next chunk lands in the tile buffers
                continue;
            }
            __syncthreads();  // every wave is done reading the tile buffers
            {
                float* T = reinterpret_cast<float*>(&s.As[0][0][0]) + wave * (64 * TSTRIDE);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int jx = 0; jx < 2; ++jx)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            T[(i * 32 + (v & 3) + 4 * half + 8 * (v >> 2)) * TSTRIDE + jx * 32 + l32] = acc[i][jx][v];
                // per-column data of the wave's 64 columns; columns past the end get +inf so that
                // they can never pass
                const uint32_t mycol = col0 + wc * 64 + lane;
                const bool col_ok = mycol < a.N;
                s.cnb[wave][lane] = col_ok ? (METRIC == kMetricL2 ? a.normB[mycol] : 0.0f) : __builtin_inff();
                if (FILTER == kFilterRange) s.cfw[wave][lane] = col_ok ? a.ts[mycol] : 0;
                if (FILTER == kFilterMask) s.cfw[wave][lane] = col_ok ? (uint64_t)(a.labels[mycol] & 63) : 0;
                // symmetric pass: the bounds of the dataset rows behind the wave's columns (in the unused filter words)
                constexpr bool SYM = FILTER == kFilterSymmetric;
                const bool mirror = SYM && ct > rt;  // the diagonal tile holds both orders of its pairs itself
                float* cbound = reinterpret_cast<float*>(s.cfw[wave]);
                if (mirror) cbound[lane] = col_ok ? a.col_bound[mycol] : -__builtin_inff();
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();

                const int r = wr * 64 + lane;
                const bool row_ok = row0 + r < a.M;
                const uint64_t thr = s.thr[r];
                // a key can only be below the threshold key if its distance is <= the threshold's
                const float thr_d = !row_ok ? -__builtin_inff() : thr == kInvalidKey ? __builtin_inff() : ord_float((uint32_t)(thr >> 32));
                const float na = s.na[r];
                const uint64_t fa = s.fa[r], fb = s.fb[r];
                constexpr float SCALE = METRIC == kMetricL2 ? -2.0f : -1.0f;
                const float4* Trow4 = reinterpret_cast<const float4*>(T + lane * TSTRIDE);
                const float4* cnb4 = reinterpret_cast<const float4*>(s.cnb[wave]);
                // Pass 1: one compare per column, the columns that may beat the threshold go into a
                // bit set.  Pass 2: every lane handles its own hits, all lanes of the wave in
                // parallel, so the wave runs the append path max-hits-per-lane times (a few) instead
                // of once per hit column.
                // Symmetric pass, tile above the diagonal: the same distances also belong to the dataset rows behind the
                // columns (d(i,j) and d(j,i) are the same bits: same products, same order of the sums), whose tile
                // below the diagonal is never computed.  Those within a column's bound are marked in a second bit set
                // and go to that row's list in device memory.
                uint64_t hits = 0, chits = 0;
                const float4* cb4 = reinterpret_cast<const float4*>(cbound);
#pragma unroll 4
                for (uint32_t c4 = 0; c4 < 16; ++c4) {
                    const float4 t = Trow4[c4], nb = cnb4[c4];
                    const float d0 = __builtin_fmaf(SCALE, t.x, na + nb.x), d1 = __builtin_fmaf(SCALE, t.y, na + nb.y);
                    const float d2 = __builtin_fmaf(SCALE, t.z, na + nb.z), d3 = __builtin_fmaf(SCALE, t.w, na + nb.w);
                    const uint32_t m = (d0 <= thr_d ? 1u : 0u) | (d1 <= thr_d ? 2u : 0u) | (d2 <= thr_d ? 4u : 0u) | (d3 <= thr_d ? 8u : 0u);
                    hits |= (uint64_t)m << (c4 * 4);
                    if (mirror) {
                        const float4 cb = cb4[c4];
                        const uint32_t m2 = (d0 <= cb.x ? 1u : 0u) | (d1 <= cb.y ? 2u : 0u) | (d2 <= cb.z ? 4u : 0u) | (d3 <= cb.w ? 8u : 0u);
                        chits |= (uint64_t)m2 << (c4 * 4);
                    }
                }
                if (FILTER == kFilterColRange) {
                    // the row's admissible columns among the wave's 64 are a run of bits: while a row has no threshold yet
                    // every column "hits", and a row whose range lies elsewhere would walk all 64 for nothing
                    const uint32_t cb = col0 + wc * 64;
                    const uint32_t lo_c = (uint32_t)fa > cb ? min((uint32_t)fa - cb, 64u) : 0u;
                    const uint32_t hi_c = (uint32_t)fb > cb ? min((uint32_t)fb - cb, 64u) : 0u;
                    const uint64_t upto = hi_c >= 64u ? ~0ull : (1ull << hi_c) - 1ull;
                    hits &= hi_c > lo_c ? upto & ~((1ull << lo_c) - 1ull) : 0ull;
                }
                const float* Trow = T + lane * TSTRIDE;
                while (hits != 0) {
                    const uint32_t c = (uint32_t)__builtin_ctzll(hits);
                    hits &= hits - 1;
                    float d = __builtin_fmaf(SCALE, Trow[c], na + s.cnb[wave][c]);
                    const uint32_t gcol = col0 + wc * 64 + c;
                    bool ok = gcol < a.N;  // +inf <= +inf while a row has no threshold yet
                    if (FILTER == kFilterRange) {
                        const uint64_t cts = s.cfw[wave][c];
                        ok = ok && cts >= fa && cts < fb;
                    }
                    if (FILTER == kFilterMask) ok = ok && ((fa >> s.cfw[wave][c]) & 1ull);
                    if (FILTER == kFilterColRange) ok = ok && gcol >= (uint32_t)fa && gcol < (uint32_t)fb;
                    if (METRIC == kMetricL2) d = d < 0.0f ? 0.0f : d;
                    const uint64_t key = make_sel_key(d, gcol);
                    if (ok && key < thr) {
                        const uint32_t slot = atomicAdd(&s.cnt[r], 1u);
                        myBuf[(size_t)r * CAP + slot] = key;
                    }
                }
                if (!row_ok) chits = 0;
                while (chits != 0) {  // symmetric pass only
                    const uint32_t c = (uint32_t)__builtin_ctzll(chits);
                    chits &= chits - 1;
                    float d = __builtin_fmaf(SCALE, Trow[c], na + s.cnb[wave][c]);
                    if (METRIC == kMetricL2) d = d < 0.0f ? 0.0f : d;
                    const uint32_t jrow = col0 + wc * 64 + c;
                    const uint32_t slot = atomicAdd(&a.col_count[jrow], 1u);
                    if (slot < a.col_cap) a.col_list[(size_t)jrow * a.col_cap + slot] = make_sel_key(d, s.arow[r]);
                }
            }
            __threadfence_block();
            __syncthreads();
            // short candidate lists are compacted (256-key sorts) as soon as 128 keys have gathered,
            // so that the threshold tightens early and a sweep over few columns stays cheap; a list of
            // 65..128 keys waits for 64 new ones (compacting after every single new key costs a sort
            // per key: ~1000 sorts per row over a million columns)
            const uint32_t trig = a.kk <= 64 ? 128u : a.kk <= 128 ? a.kk + 64u : (uint32_t)COMPACT_AT;
            {
                // wave w looks after rows w, w+4, ...: one parallel look at the 32 counters, then
                // only the rows that are due
                const uint32_t myc = lane < TM / 4 ? s.cnt[wave + 4 * lane] : 0u;
                uint64_t due = __ballot(myc >= trig && myc > a.kk);
                while (due != 0) {
                    const int r = wave + 4 * (int)__builtin_ctzll(due);
                    due &= due - 1;
                    compact_row(s, myBuf + (size_t)r * CAP, r, a.kk, lane);
                }
            }
        }

        if (STORE) continue;
        // ---- end of this work item: final selection, write the kk keys of every row ----
        __threadfence_block();
        __syncthreads();
        for (int r = wave; r < TM; r += 4) {
            if (row0 + r >= a.M) continue;
            uint64_t* rowbuf = myBuf + (size_t)r * CAP;
            if (s.cnt[r] > a.kk) compact_row(s, rowbuf, r, a.kk, lane);
            __threadfence_block();
            const uint32_t n = s.cnt[r];
            uint64_t* out = a.cand_out + ((size_t)(a.cand_by_grid_row ? row0 + r : s.arow[r]) * a.nsplit + sp) * a.kk;
            for (uint32_t g = lane; g < a.kk; g += 64) out[g] = g < n ? rowbuf[g] : kInvalidKey;
        }
    }
}


// ---- the symmetric pass on the bf16 matrix pipe --------------------------------------------------------------
// The same pass as tile_topk_kernel<kMetricL2, kFilterSymmetric> - same tiles, thresholds, lists and epilogue - with
// the inner products formed by v_mfma_f32_32x32x16_bf16, sixteen times the rate of the fp32 instruction, from rows
// split into two bf16 halves (x = hi + lo + what is left, |left| <= 2^-16 |x|): q.c is taken as
// q_lo.c_hi + q_hi.c_lo + q_hi.c_hi with fp32 accumulation, off the true product sum by at most 3 * 2^-16 |q||c|.  The
// rows are centred first (no distance notices), so that this is relative to the spread of the data, not to its
// offset.  What the pass returns are candidates: the exact re-scoring and the check after it (refine_kernel, which is
// told the larger error) decide the result, as for the fp32 pass.
// A ninth k-step adds -|q|^2/2 - |c|^2/2 (three bf16 pieces of each, against ones), so an accumulator holds g = minus
// half the squared distance when the matrix instructions are through, and the epilogue's tests are one comparison
// each: g >= -threshold/2.
// Workgroup = 8 waves, two per SIMD, a CU to itself; wave (wr, wc) owns rows wr*32..+31 and, of every column tile,
// columns wc*64..+63.  The rows' halves stay in registers for the whole sweep (64 VGPRs), the column tiles (128
// columns x 512 bytes) are staged in LDS, the next one in flight during the matrix instructions of this one.  The
// sweep runs from the last column tile down to the diagonal, so that the workgroups of a round read the same tiles at
// about the same time and share them in L2.
constexpr uint32_t kSplitRow = 272;      // bf16 values of a split row: 128 high halves, 128 low halves, 8 of the norm as a column, 8 as a row
constexpr uint32_t kSplitPitch = 560;    // bytes of a column in LDS: 528 of data, 32 so that 16-byte reads of 8 consecutive columns cover all banks
constexpr uint32_t kSplitWaves = 8;
constexpr uint32_t kSplitT = 68;         // row stride of a wave's transposed 32 x 64 block: 16-byte aligned rows, conflict-free b128 reads
constexpr uint32_t kSplitSlot = TN * kSplitPitch;  // a tile buffer, which the epilogue's transposed blocks (smaller by 2 KB) take over
static_assert(kSplitSlot >= kSplitWaves * 32 * kSplitT * 4, "the transposed blocks fit a tile buffer");

struct SplitLds {
    uint8_t b[2][kSplitSlot];
    uint64_t thr[TM];
    uint32_t cnt[TM];
    float cbound[kSplitWaves][64];  // -bound/2 of the wave's columns
};

// Sorting a row's buffer needs some 60 registers that the sweep, with the rows' halves in 128 of its 256, does not
// have: as a function of its own it saves and restores what it uses when it runs - once in hundreds of steps -
// instead of the sweep keeping part of the halves in scratch memory and fetching them in every step.
__device__ __attribute__((noinline)) void compact_row_split(SplitLds& s, uint64_t* rowbuf, int r, uint32_t kk, int lane) {
    compact_row(s, rowbuf, r, kk, lane);
}

__global__ void __launch_bounds__(64 * kSplitWaves, 1) sym_split_kernel(const TileArgs a, const uint16_t* __restrict__ rows) {
    extern __shared__ __align__(16) uint8_t tile_smem[];
    SplitLds& s = *reinterpret_cast<SplitLds*>(tile_smem);
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wr = wave >> 1, wc = wave & 1, half = lane >> 5, l32 = lane & 31;
    uint64_t* myBuf = a.buf + (size_t)blockIdx.x * TM * CAP;
    const uint32_t nwork = a.row_tiles;

    for (uint32_t base = 0; base < nwork; base += gridDim.x) {
        // row tile rt sweeps the column tiles from rt on, so the items shrink with rt; every other round hands them out in reverse
        uint32_t work = base + blockIdx.x;
        if ((base / gridDim.x) & 1u) work = base + (gridDim.x - 1 - blockIdx.x);
        if (work >= nwork) continue;  // workgroup-uniform
        __syncthreads();              // the item before is fully drained
        const uint32_t rt = work, row0 = rt * TM;
        if (tid < TM) {
            const uint32_t row = row0 + tid;
            const bool valid = row < a.M;
            s.thr[tid] = valid ? (((uint64_t)ord_bits(a.col_bound[min(row, a.M - 1u)]) << 32) | 0xFFFFFFFFull) : kInvalidKey;
            s.cnt[tid] = 0;
        }
        // lane (l32, half) holds, for k-step ks, the 8 values k = 16 ks + 8 half .. + 7 of row l32 of the wave's block, both halves
        v8bf16 ah[8], al[8], anorm;
        {
            const uint16_t* x = rows + (size_t)min(row0 + wr * 32 + l32, a.M - 1u) * kSplitRow + 8u * half;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                ah[ks] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(x + 16 * ks));
                al[ks] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(x + 128 + 16 * ks));
            }
            // the ninth k-step: its first 8 values are the norm's pieces and ones, the other 8 (the lanes of half 1) nothing
            uint4 e = *reinterpret_cast<const uint4*>(x - 8u * half + 264);
            if (half) e = make_uint4(0u, 0u, 0u, 0u);
            anorm = __builtin_bit_cast(v8bf16, e);
        }

        // a column tile: 128 x 32 pieces of 16 bytes, 8 pieces a thread in two lots of 4, a column's pieces by consecutive
        // threads; and the 128 pieces of the ninth k-step, which travel with the second lot
        const uint32_t steps = a.col_tiles - rt;
        uint4 st0, st1, st2, st3, st4 = make_uint4(0u, 0u, 0u, 0u);
        auto piece_of = [&](uint32_t lot, uint32_t u) { return tid + 64u * kSplitWaves * (4u * lot + u); };
        auto load_piece = [&](uint32_t ct, uint32_t piece) {
            const uint32_t col = ct * TN + (piece >> 5);
            return *reinterpret_cast<const uint4*>(rows + (size_t)min(col, a.N - 1u) * kSplitRow + 8u * (piece & 31u));
        };
        auto store_piece = [&](uint32_t buf, uint32_t piece, uint4 v) {
            *reinterpret_cast<uint4*>(&s.b[buf][(piece >> 5) * kSplitPitch + 16u * (piece & 31u)]) = v;
        };
#define fetch(ct_, lot_)                             \
    do {                                             \
        st0 = load_piece(ct_, piece_of(lot_, 0));    \
        st1 = load_piece(ct_, piece_of(lot_, 1));    \
        st2 = load_piece(ct_, piece_of(lot_, 2));    \
        st3 = load_piece(ct_, piece_of(lot_, 3));    \
    } while (0)
#define park(buf_, lot_)                             \
    do {                                             \
        store_piece(buf_, piece_of(lot_, 0), st0);   \
        store_piece(buf_, piece_of(lot_, 1), st1);   \
        store_piece(buf_, piece_of(lot_, 2), st2);   \
        store_piece(buf_, piece_of(lot_, 3), st3);   \
    } while (0)
#define fetch_norms(ct_) st4 = *reinterpret_cast<const uint4*>(rows + (size_t)min((ct_) * TN + (tid & 127u), a.N - 1u) * kSplitRow + 256)
#define park_norms(buf_)                                                                                       \
    do {                                                                                                       \
        if (tid < 128u) *reinterpret_cast<uint4*>(&s.b[buf_][tid * kSplitPitch + 512u]) = st4;                 \
    } while (0)
        // The tile after this one travels in two lots: the first is fetched during the epilogue of the step before and
        // parked at the start of this step, the second is fetched then and parked after the matrix instructions - each
        // has thousands of cycles for its way, and no wait for memory stands inside the loop of matrix instructions.
        // (Past the end of the sweep a tile is fetched once more, into the buffer nobody reads.)
        auto tile_of = [&](uint32_t step) { return a.col_tiles - 1u - min(step, steps - 1u); };
        fetch(tile_of(0), 0);
        park(0, 0);
        fetch(tile_of(0), 1);
        fetch_norms(tile_of(0));
        park(0, 1);
        park_norms(0);
        fetch(tile_of(1), 0);
        // a key for a column's list waits one step for its place: the addition that reserves it is on its way during the
        // matrix instructions of the next step instead of being waited for (most lanes have at most one such key a step)
        bool pend = false;
        uint32_t pend_slot = 0, pend_row = 0;
        uint64_t pend_key = 0;
        __syncthreads();  // first tile and row table visible
        for (uint32_t step = 0; step < steps; ++step) {
            const uint32_t buf = step & 1u;
            const uint32_t ct = tile_of(step), col0 = ct * TN;
            v16f acc[2];  // the wave's two blocks of 32 columns; the first k-step starts them from the constant 0 (no 32 register moves)
            const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            park(buf ^ 1u, 0);
            fetch(tile_of(step + 1), 1);
            fetch_norms(tile_of(step + 1));
            // what the epilogue wants of the wave's columns, on its way during the matrix instructions
            const uint32_t mycol = col0 + wc * 64 + lane;
            const float cbv = a.col_bound[min(mycol, a.N - 1u)];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                v8bf16 bh[2], bl[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint8_t* colp = &s.b[buf][(wc * 64 + j * 32 + l32) * kSplitPitch + 32u * ks + 16u * half];
                    bh[j] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(colp));
                    bl[j] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(colp + 256));
                }
                // the small terms first; consecutive instructions go to different accumulators
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[ks], bh[0], ks == 0 ? zero : acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[ks], bh[1], ks == 0 ? zero : acc[1], 0, 0, 0);
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bl[0], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bl[1], acc[1], 0, 0, 0);
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bh[0], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ks], bh[1], acc[1], 0, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {  // the norms last: they are added to the finished sum of products
                const v8bf16 bn = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(&s.b[buf][(wc * 64 + j * 32 + l32) * kSplitPitch + 512u]));
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(anorm, bn, acc[j], 0, 0, 0);
            }
            park(buf ^ 1u, 1);
            park_norms(buf ^ 1u);
            __syncthreads();  // every wave is done reading this tile: its buffer becomes the transposed blocks
            fetch(tile_of(step + 2), 0);

            // ---- epilogue, as in tile_topk_kernel: the wave's 32 x 64 block goes through LDS, and each lane walks half a row ----
            {
                float* T = reinterpret_cast<float*>(s.b[buf]) + wave * (32 * kSplitT);
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) T[((v & 3) + 4 * half + 8 * (v >> 2)) * kSplitT + j * 32 + l32] = acc[j][v];
                const bool col_ok = mycol < a.N;
                const bool mirror = ct > rt;  // the diagonal tile holds both orders of its pairs itself
                s.cbound[wave][lane] = col_ok ? -0.5f * cbv : __builtin_inff();  // columns past the end can never pass
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();

                // lane (l32, half): row l32 of the block, columns 32 half .. + 31 of the wave's 64
                const uint32_t r = wr * 32 + l32;
                const bool row_ok = row0 + r < a.M;
                const uint64_t thr = s.thr[r];
                // a key can only be below the threshold key if its distance is <= the threshold's: g >= -that/2
                const float thr_g = !row_ok ? __builtin_inff() : thr == kInvalidKey ? -__builtin_inff() : -0.5f * ord_float((uint32_t)(thr >> 32));
                const float4* Trow4 = reinterpret_cast<const float4*>(T + l32 * kSplitT + 32u * half);
                const float4* cb4 = reinterpret_cast<const float4*>(s.cbound[wave] + 32u * half);
                // Four columns at a time, two comparisons a value; their results are put together lane by lane only where
                // some lane of the wave has a mark among the four (the comparisons leave wave-wide masks, which the scalar
                // unit joins and tests)
                uint32_t hits = 0, chits = 0;
#pragma unroll
                for (uint32_t c4 = 0; c4 < 8; ++c4) {
                    const float4 t = Trow4[c4], cb = cb4[c4];
                    const bool o0 = t.x >= thr_g, o1 = t.y >= thr_g, o2 = t.z >= thr_g, o3 = t.w >= thr_g;
                    const bool m0 = t.x >= cb.x, m1 = t.y >= cb.y, m2 = t.z >= cb.z, m3 = t.w >= cb.w;
                    if (__ballot(o0 | o1 | o2 | o3 | m0 | m1 | m2 | m3) != 0) {
                        hits |= ((o0 ? 1u : 0u) | (o1 ? 2u : 0u) | (o2 ? 4u : 0u) | (o3 ? 8u : 0u)) << (c4 * 4);
                        chits |= ((m0 ? 1u : 0u) | (m1 ? 2u : 0u) | (m2 ? 4u : 0u) | (m3 ? 8u : 0u)) << (c4 * 4);
                    }
                }
                if (!mirror || !row_ok) chits = 0;
                if (pend) {
                    if (pend_slot < a.col_cap) a.col_list[(size_t)pend_row * a.col_cap + pend_slot] = pend_key;
                    pend = false;
                }
                const float* Trow = T + l32 * kSplitT + 32u * half;
                while (hits != 0) {
                    const uint32_t c = (uint32_t)__builtin_ctz(hits);
                    hits &= hits - 1;
                    float d = -2.0f * Trow[c];
                    const uint32_t gcol = col0 + wc * 64 + 32u * half + c;
                    d = d < 0.0f ? 0.0f : d;
                    const uint64_t key = make_sel_key(d, gcol);
                    if (gcol < a.N && key < thr) {
                        const uint32_t slot = atomicAdd(&s.cnt[r], 1u);
                        myBuf[(size_t)r * CAP + slot] = key;
                    }
                }
                while (chits != 0) {
                    const uint32_t c = (uint32_t)__builtin_ctz(chits);
                    chits &= chits - 1;
                    float d = -2.0f * Trow[c];
                    d = d < 0.0f ? 0.0f : d;
                    const uint32_t jrow = col0 + wc * 64 + 32u * half + c;
                    const uint32_t slot = atomicAdd(&a.col_count[jrow], 1u);
                    const uint64_t key = make_sel_key(d, row0 + r);
                    if (!pend) {
                        pend = true;
                        pend_slot = slot;
                        pend_row = jrow;
                        pend_key = key;
                    } else if (slot < a.col_cap) {
                        a.col_list[(size_t)jrow * a.col_cap + slot] = key;
                    }
                }
            }
            __threadfence_block();
            __syncthreads();  // the blocks are consumed: the buffer may take the tile after next; appended keys are visible
            const uint32_t trig = a.kk <= 64 ? 128u : a.kk <= 128 ? a.kk + 64u : (uint32_t)COMPACT_AT;
            {
                // wave w looks after rows w, w+8, ...: one parallel look at the counters, then only the rows that are due
                const uint32_t myc = lane < TM / kSplitWaves ? s.cnt[wave + kSplitWaves * lane] : 0u;
                uint64_t due = __ballot(myc >= trig && myc > a.kk);
                while (due != 0) {
                    const int r = (int)wave + (int)kSplitWaves * (int)__builtin_ctzll(due);
                    due &= due - 1;
                    compact_row_split(s, myBuf + (size_t)r * CAP, r, a.kk, (int)lane);
                }
            }
        }
#undef fetch
#undef park
#undef fetch_norms
#undef park_norms
        if (pend && pend_slot < a.col_cap) a.col_list[(size_t)pend_row * a.col_cap + pend_slot] = pend_key;
        __threadfence_block();
        __syncthreads();
        for (uint32_t r = wave; r < (uint32_t)TM; r += kSplitWaves) {
            if (row0 + r >= a.M) continue;
            uint64_t* rowbuf = myBuf + (size_t)r * CAP;
            if (s.cnt[r] > a.kk) compact_row_split(s, rowbuf, (int)r, a.kk, (int)lane);
            __threadfence_block();
            const uint32_t n = s.cnt[r];
            uint64_t* out = a.cand_out + (size_t)(row0 + r) * a.kk;
            for (uint32_t g = lane; g < a.kk; g += 64) out[g] = g < n ? rowbuf[g] : kInvalidKey;
        }
    }
}

int launch_sym_split(const TileArgs& a, const uint16_t* rows, uint32_t grid, hipStream_t stream) {
    static_assert(sizeof(SplitLds) <= 160 * 1024, "one workgroup per CU");
    GRAB_REQUIRE(a.nsplit == 1 && a.M == a.N && a.dim <= 128 && a.row_tiles == a.col_tiles, "internal: shape of the bf16 symmetric pass");
    GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(sym_split_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(SplitLds)));
    hipLaunchKernelGGL(sym_split_kernel, dim3(grid), dim3(64 * kSplitWaves), sizeof(SplitLds), stream, a, rows);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
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

// largest value of a non-negative float array (as its bit pattern, which orders like the value)
__global__ void __launch_bounds__(256) max_float_kernel(const float* __restrict__ x, uint64_t n, uint32_t* __restrict__ out) {
    float v = 0.0f;  // a thread walks its share of the array: one atomic per wave of a small grid, not one per 64 values
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) v = fmaxf(v, x[i]);
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    if ((threadIdx.x & 63) == 0) atomicMax(out, __float_as_uint(v));
}

// one wave per row: canonical re-score, sort by (distance,id), emit
template <int METRIC, int NPL>
__global__ void __launch_bounds__(256) refine_kernel(const RefineArgs a) {
    __shared__ uint64_t keys[4][64 * NPL];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t slot = blockIdx.x * 4 + wave;
    if (slot >= a.M) return;  // wave-uniform
    const uint32_t row = a.rows ? a.rows[slot] : slot;
    uint64_t* mykeys = keys[wave];
    const uint64_t* cand = a.cand + (size_t)row * a.nc;
    for (uint32_t g = lane; g < 64u * NPL; g += 64) mykeys[g] = g < a.nc ? cand[g] : kInvalidKey;
    // Every column that is not a candidate has a GEMM-form distance of at least `outside`: the largest key of a full
    // list (a list that is not full holds every admissible column of its slice)
    float outside = __builtin_inff();
    if (a.doubt != nullptr) {
        for (uint32_t sp = lane; sp * a.kk < a.nc; sp += 64) {
            const uint64_t last = cand[(size_t)sp * a.kk + a.kk - 1];
            if (last != kInvalidKey) outside = fminf(outside, ord_float((uint32_t)(last >> 32)));
        }
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) outside = fminf(outside, __shfl_xor(outside, m, 64));
        if (a.outside_in != nullptr) outside = fminf(outside, a.outside_in[row]);
    }
    __builtin_amdgcn_wave_barrier();
    // How far the GEMM-form value of a pair can lie from its true distance (see the check below)
    auto form_error = [&]() -> double {
        const double u = 5.9604644775390625e-08, na = a.normA[row], nb = *a.max_normB, c = 1.25 * a.dim + 16.0;
        // bf16 keeps 8 bits: a value and its two halves differ by at most 2^-16 of it, and the three things a
        // split-bf16 product lacks (lo.lo and the two remainders against the other vector) are at most
        // 2^-16 |a||b| <= 2^-17 (|a|^2 + |b|^2) each - 3 * 2^-16 = 768 * 2^-24 of the norms in the distance.  Its fp32
        // sums run over split_terms products: at most split_terms * 2^-24 |a||b| each way when every addition rounds
        // to nearest, twice that should the matrix pipe chop - 2 * split_terms * 2^-24 of the norms in the distance.
        // A row's candidates are from one pass or the other: the larger error
        const double cs = c + 32.0 + 2.0 * (double)a.split_terms + 768.0;
        if (METRIC != kMetricL2) {
            double err = 2.0 * c * u * sqrt(na * nb);
            if (a.split_normA != nullptr) err = fmax(err, 2.0 * cs * u * sqrt((double)a.split_normA[row] * (double)*a.split_max_normB));
            return err;
        }
        double err = c * u * (na + nb);
        if (a.split_normA != nullptr) err = fmax(err, cs * u * ((double)a.split_normA[row] + (double)*a.split_max_normB));
        return err;
    };
    // An ascending list need not be scored to its end: the first need + 1 candidates have true distances of at most
    // A + err (A = the GEMM-form value of the last of them), so a candidate whose GEMM-form value exceeds A + 2 err -
    // and a little more, for what the re-scoring itself may be off on either side - is farther than all of them under
    // the re-scored order as well and cannot be among the row's neighbours.  It is dropped unscored (some 130 of 289
    // candidates are scored at k = 128).
    uint32_t n_score = a.nc;
    if (a.sorted && a.doubt != nullptr) {
        const uint32_t need = a.drop_self ? a.k : a.k - 1u;
        const uint64_t an = need < a.nc ? mykeys[need] : kInvalidKey;
        if (an != kInvalidKey) {
            const double A = (double)ord_float((uint32_t)(an >> 32)), err = form_error();
            const double slack = METRIC == kMetricL2 ? 4.0 * (a.dim / 8 + 8) * 5.9604644775390625e-08 * (fabs(A) + 2.0 * err) : 2.0 * err;
            const float cutoff = (float)(A + 2.0 * err + slack) + fabsf((float)A) * 2.4e-7f;  // the conversion rounds: two ulps up
            uint32_t kept = 0;
            for (uint32_t g0 = 0; g0 < a.nc; g0 += 64) {
                const uint32_t g = g0 + lane;
                const uint64_t key = g < a.nc ? mykeys[g] : kInvalidKey;
                kept += (uint32_t)__popcll(__ballot(key != kInvalidKey && ord_float((uint32_t)(key >> 32)) <= cutoff));
            }
            n_score = max(kept, need + 1u);  // ascending: the kept ones are the first `kept`
            for (uint32_t g = n_score + lane; g < 64u * NPL; g += 64) mykeys[g] = kInvalidKey;
            __builtin_amdgcn_wave_barrier();
        }
    }
    const float* q = a.A + (size_t)row * a.dim;
    const int grp = lane >> 3, j = lane & 7;
    for (uint32_t c0 = 0; c0 < n_score; c0 += 8) {
        const uint32_t c = c0 + grp;
        const uint64_t kc = c < n_score ? mykeys[c] : kInvalidKey;  // uniform per group of 8 lanes
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
    if (a.doubt != nullptr && outside < __builtin_inff()) {
        // The candidates were chosen by |a|^2+|b|^2-2ab (or -ab) in fp32, which differs from the true value by at most
        // err = (1.25 dim + 16) 2^-24 (|a|^2 + max|b|^2) (inner product: ... sqrt(|a|^2 max|b|^2)); the re-scored
        // distance differs from it by at most (dim/8 + 8) 2^-24 of itself (inner product: by err again).  The result
        // is proven when the last distance it needs - the k-th, or the (k+1)-th when the row's own id is dropped - lies
        // below everything a column outside the lists can have.  Otherwise the row is listed for the exact pass.
        const uint32_t need = a.drop_self ? a.k : a.k - 1u;
        const uint64_t kn = need < 64u * NPL ? mykeys[need] : kInvalidKey;
        bool proven = false;
        if (kn != kInvalidKey) {
            const double u = 5.9604644775390625e-08;
            const double last = (double)ord_float((uint32_t)(kn >> 32)), out = (double)outside, err = form_error();
            if (METRIC == kMetricL2) {
                const double low = out - err;
                proven = last < low - (a.dim / 8 + 8) * u * fabs(low);
            } else {
                proven = last < out - err;
            }
        }
        if (!proven && lane == 0) a.doubt[1 + atomicAdd(a.doubt, 1u)] = row;
    }
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

// ---- the row set against itself: helpers of the symmetric pass ----------------------------------------------
constexpr uint32_t kSymMinRows = 16384;     // below this the plain pass is quick,
constexpr uint32_t kSymMinRowsSplit = 4096; // ... unless the symmetric pass can run on bf16 instructions (10,000 rows x 128: 1.6 ms against 3.6)
constexpr uint32_t kSymSample = 49152;      // columns of the bounding pass (an evenly spaced sample of the rows), at most
constexpr uint32_t kSymRank = 28;           // a row's bound is its distance to the kSymRank-th nearest sample column, at least
constexpr uint32_t kSymMaxKeep = 320;       // longest candidate list for which a row's column-walk list holds twice as many
constexpr uint32_t kSymColCap = 1024;       // keys a row can receive from column walks
constexpr size_t kSymMaxListBytes = (size_t)64 << 30;

// row i * n / count of `src` becomes row i of `dst`, with its squared norm; 8 lanes per row
// (src_norms: the rows are not plain fp32 rows - bf16 halves - and their norms are taken from this array instead)
__global__ void __launch_bounds__(256) spaced_rows_kernel(const float* __restrict__ src, uint64_t n, uint32_t count, uint32_t dim,
                                                          float* __restrict__ dst, float* __restrict__ norms,
                                                          const float* __restrict__ src_norms = nullptr) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= count) return;
    const uint64_t from = (uint64_t)g * n / count;
    const float4* r4 = reinterpret_cast<const float4*>(src + (size_t)from * dim);
    float4* d4 = reinterpret_cast<float4*>(dst + (size_t)g * dim);
    float s = 0.0f;
    for (uint32_t c = j; c < (dim >> 2); c += 8) {
        const float4 v = r4[c];
        d4[c] = v;
        s = __builtin_fmaf(v.x, v.x, s);
        s = __builtin_fmaf(v.y, v.y, s);
        s = __builtin_fmaf(v.z, v.z, s);
        s = __builtin_fmaf(v.w, v.w, s);
    }
    s = group8_sum(s);
    if (j == 0) norms[g] = src_norms ? src_norms[from] : s;
}

// ---- rows as bf16 halves, for the SPLIT instances of tile_topk_kernel ----
// round to nearest, ties to even; the inputs are finite
__device__ __forceinline__ uint32_t to_bf16_bits(float x) {
    const uint32_t u = __float_as_uint(x);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// mean[k] = average of coordinate k over `count` evenly spaced rows; one workgroup per coordinate
__global__ void __launch_bounds__(256) spaced_mean_kernel(const float* __restrict__ data, uint64_t n, uint32_t count, uint32_t dim,
                                                          float* __restrict__ mean) {
    __shared__ float part[256];
    const uint32_t k = blockIdx.x;
    float s = 0.0f;
    for (uint32_t i = threadIdx.x; i < count; i += 256) s += data[(size_t)((uint64_t)i * n / count) * dim + k];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) mean[k] = part[0] / (float)count;
}

// out[row] = the row (less `mean`, where one is given: no squared distance notices, and bf16's eight bits then go to
// what differs between rows) as bf16 halves, chunk of 32 dimensions by chunk: 32 high halves (bf16 of x), then 32 low
// halves (bf16 of x - high, a difference that fp32 holds exactly).  A row takes dim * 4 bytes like the fp32 row.
// norm[row] = squared norm of the fp32 row as split (centred or not).  8 lanes per row; dim a multiple of 32.
__global__ void __launch_bounds__(256) split_rows_chunked_kernel(const float* __restrict__ data, uint64_t n, uint32_t dim,
                                                                 const float* __restrict__ mean, uint16_t* __restrict__ out,
                                                                 float* __restrict__ norm) {
    const uint64_t g = ((uint64_t)blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= n) return;
    const float4* r4 = reinterpret_cast<const float4*>(data + (size_t)g * dim);
    const float4* m4 = reinterpret_cast<const float4*>(mean);
    uint16_t* o = out + (size_t)g * dim * 2;
    float s = 0.0f;
    for (uint32_t c = j; c < (dim >> 2); c += 8) {
        float4 v = r4[c];
        if (mean != nullptr) {
            const float4 m = m4[c];
            v = make_float4(v.x - m.x, v.y - m.y, v.z - m.z, v.w - m.w);
        }
        const float x[4] = {v.x, v.y, v.z, v.w};
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            s = __builtin_fmaf(x[e], x[e], s);
            hi[e] = to_bf16_bits(x[e]);
            lo[e] = to_bf16_bits(x[e] - __uint_as_float(hi[e] << 16));
        }
        const uint32_t k = 4u * c, at = (k >> 5) * 64u + (k & 31u);  // chunk k / 32, place k % 32
        *reinterpret_cast<uint2*>(o + at) = make_uint2(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16));
        *reinterpret_cast<uint2*>(o + at + 32) = make_uint2(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16));
    }
    s = group8_sum(s);
    if (j == 0 && norm != nullptr) norm[g] = s;
}

// bound[row] = the largest distance among the row's `rank` nearest sample columns (+inf if it has fewer)
__global__ void __launch_bounds__(256) column_bound_kernel(const uint64_t* __restrict__ cand, uint32_t rank, uint32_t n,
                                                           float* __restrict__ bound) {
    const uint32_t row = blockIdx.x * 256 + threadIdx.x;
    if (row >= n) return;
    uint64_t worst = 0;
    for (uint32_t i = 0; i < rank; ++i) worst = max(worst, cand[(size_t)row * rank + i]);
    bound[row] = worst == kInvalidKey ? __builtin_inff() : ord_float((uint32_t)(worst >> 32));
}

// One wave per row: the row's own list (the kk best among the columns from its diagonal tile on) and the keys that
// column walks left for it (columns before that tile) become the kk best of all columns.  That is certain when at
// least kk keys at or below the row's bound are at hand: every key at or below the bound is, on either side.  Rows
// for which it is not (too few such keys, or more than the lists hold) are listed and redone by the plain pass.
__global__ void __launch_bounds__(256) merge_symmetric_kernel(uint64_t* __restrict__ cand, const uint64_t* __restrict__ col_list,
                                                              const uint32_t* __restrict__ col_count, uint32_t col_cap,
                                                              const float* __restrict__ bound, uint32_t kk, uint32_t n,
                                                              uint32_t* __restrict__ redo, uint32_t* __restrict__ redo_count) {
    __shared__ uint64_t keys_all[4][1024];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= n) return;
    uint64_t* keys = keys_all[wave];
    uint64_t* own = cand + (size_t)row * kk;
    const uint32_t nb = col_count[row];
    const float b = bound[row];
    // the row's own keys at or below the bound, packed
    uint32_t na = 0;
    for (uint32_t g0 = 0; g0 < kk; g0 += 64) {
        const uint32_t g = g0 + lane;
        const uint64_t key = g < kk ? own[g] : kInvalidKey;
        const bool in = key != kInvalidKey && ord_float((uint32_t)(key >> 32)) <= b;
        const uint64_t bal = __ballot(in);
        if (in) keys[na + __popcll(bal & ((1ull << lane) - 1ull))] = key;  // na + 64 <= kk + 63 < 1024
        na += (uint32_t)__popcll(bal);
    }
    const bool fits = nb <= col_cap && na + nb <= 1024;
    if (!fits || na + nb < kk) {
        if (lane == 0) redo[atomicAdd(redo_count, 1u)] = row;
        return;
    }
    for (uint32_t g = lane; g < nb; g += 64) keys[na + g] = col_list[(size_t)row * col_cap + g];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const uint32_t total = na + nb;
    if (total <= 512) {  // the usual case (about twice kk keys lie within the bound): half the sorting network
        uint64_t k[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) k[i] = (uint32_t)(lane * 8 + i) < total ? keys[lane * 8 + i] : kInvalidKey;
        wave_bitonic_sort<8>(k);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if ((uint32_t)(lane * 8 + i) < kk) own[lane * 8 + i] = k[i];
        return;
    }
    uint64_t k[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) k[i] = (uint32_t)(lane * 16 + i) < total ? keys[lane * 16 + i] : kInvalidKey;
    wave_bitonic_sort<16>(k);
#pragma unroll
    for (int i = 0; i < 16; ++i)
        if ((uint32_t)(lane * 16 + i) < kk) own[lane * 16 + i] = k[i];
}

// A redone row's partial lists (`parts` of kk keys each) are merged `per` at a time (per * kk <= 1024 keys, one sort
// by a wave): work item (row f, group g) leaves the kk best of parts g*per .. g*per+per-1 in out[(f * groups + g) * kk],
// or, when one group is all there is, in the row's place of the candidate array.
__global__ void __launch_bounds__(256) merge_redone_kernel(const uint64_t* __restrict__ part, uint32_t parts, uint32_t per, uint32_t kk,
                                                           const uint32_t* __restrict__ redo, uint32_t count, uint64_t* __restrict__ out,
                                                           uint64_t* __restrict__ cand) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t groups = (parts + per - 1) / per;
    const uint32_t item = blockIdx.x * 4 + wave;
    if (item >= count * groups) return;
    const uint32_t f = item / groups, g = item - f * groups;
    const uint32_t nc = (min((g + 1) * per, parts) - g * per) * kk;
    const uint64_t* src = part + ((size_t)f * parts + (size_t)g * per) * kk;
    uint64_t k[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) k[i] = (uint32_t)(lane * 16 + i) < nc ? src[lane * 16 + i] : kInvalidKey;
    wave_bitonic_sort<16>(k);
    uint64_t* own = groups == 1 ? cand + (size_t)redo[f] * kk : out + ((size_t)f * groups + g) * kk;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        if ((uint32_t)(lane * 16 + i) < kk) own[lane * 16 + i] = k[i];
}

template <int METRIC, int FILTER, bool STORE = false, bool SPLIT = false>
int launch_tile_one(const TileArgs& a, uint32_t grid, hipStream_t stream) {
    auto kern = tile_topk_kernel<METRIC, FILTER, STORE, SPLIT>;
    static_assert(sizeof(TileLds) <= 80 * 1024, "two workgroups per CU must fit 160 KB of LDS");
    static_assert(4 * 64 * TSTRIDE * sizeof(float) <= 2 * sizeof(float) * 2 * TM * LDS_STRIDE, "epilogue block must fit the tile buffers");
    GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(TileLds)));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), sizeof(TileLds), stream, a);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

// the same launches on rows split into bf16 halves (dim a multiple of 32)
template <int METRIC>
int launch_tile_split(const TileArgs& a, int filter, uint32_t grid, hipStream_t stream) {
    GRAB_REQUIRE(a.dim % KC == 0, "internal: rows split into bf16 halves come in whole chunks of %d dimensions", KC);
    switch (filter) {
        case kFilterNone: return launch_tile_one<METRIC, kFilterNone, false, true>(a, grid, stream);
        case kFilterRange: return launch_tile_one<METRIC, kFilterRange, false, true>(a, grid, stream);
        case kFilterMask: return launch_tile_one<METRIC, kFilterMask, false, true>(a, grid, stream);
        case kFilterColRange: return launch_tile_one<METRIC, kFilterColRange, false, true>(a, grid, stream);
        case kFilterSymmetric: return launch_tile_one<METRIC, kFilterSymmetric, false, true>(a, grid, stream);
        default: set_error("bad filter kind %d", filter); return GRAB_ERR_INVALID;
    }
}

template <int METRIC>
int launch_tile(const TileArgs& a, int filter, uint32_t grid, hipStream_t stream, bool split = false) {
    if (split) return launch_tile_split<METRIC>(a, filter, grid, stream);
    switch (filter) {
        case kFilterNone: return launch_tile_one<METRIC, kFilterNone>(a, grid, stream);
        case kFilterRange: return launch_tile_one<METRIC, kFilterRange>(a, grid, stream);
        case kFilterMask: return launch_tile_one<METRIC, kFilterMask>(a, grid, stream);
        case kFilterColRange: return launch_tile_one<METRIC, kFilterColRange>(a, grid, stream);
        case kFilterSymmetric: return launch_tile_one<METRIC, kFilterSymmetric>(a, grid, stream);
        default: set_error("bad filter kind %d", filter); return GRAB_ERR_INVALID;
    }
}

// The exact pass for rows whose candidates prove nothing (distances far below the rounding error of the GEMM form:
// a large common offset, many near-duplicates): one workgroup a row, every admissible column scored in the canonical
// order, eight lanes a column, the smallest keys kept through a threshold list in LDS.  Writes the row's kExactKeep
// smallest exact keys into its candidate slots.  Slow (the whole base per row) and exact for any input.
constexpr uint32_t kExactKeep = 520, kExactBuf = 1024, kExactStep = 256;  // k + 1 <= 513 keys are ever needed
struct ExactArgs {
    const float* A;
    const float* B;
    const uint32_t* rows;
    uint32_t count, dim, nc;
    uint64_t N;
    int filter;
    const uint64_t* ts;
    const uint64_t* win_start_arr;
    const uint64_t* win_end_arr;
    uint64_t win_start, win_end;
    int per_query_window;
    const uint8_t* labels;
    const uint64_t* masks;
    const uint32_t* row_lo;  // kFilterColRange: the row's admissible columns [lo, hi)
    const uint32_t* row_hi;
    uint64_t* cand;  // [M][nc]
};
template <int METRIC>
__global__ void __launch_bounds__(256) exact_rows_kernel(const ExactArgs a) {
    __shared__ uint64_t buf[kExactBuf];
    __shared__ uint32_t cnt;
    __shared__ uint64_t thr;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, grp = threadIdx.x >> 3, j = threadIdx.x & 7;
    for (uint32_t f = blockIdx.x; f < a.count; f += gridDim.x) {
        const uint32_t row = a.rows[f];
        const float* q = a.A + (size_t)row * a.dim;
        uint64_t w0 = a.win_start, w1 = a.win_end, mask = 0;
        if (a.filter == kFilterRange && a.per_query_window) {
            w0 = a.win_start_arr[row];
            w1 = a.win_end_arr[row];
        }
        if (a.filter == kFilterMask) mask = a.masks[row];
        uint64_t c_first = 0, c_last = a.N;
        if (a.filter == kFilterColRange) {
            c_first = a.row_lo[row];
            c_last = min((uint64_t)a.row_hi[row], a.N);
            if (c_last < c_first) c_last = c_first;
        }
        if (threadIdx.x == 0) {
            cnt = 0;
            thr = kInvalidKey;
        }
        __syncthreads();
        auto compact = [&]() {  // wave 0 sorts the list and keeps the kExactKeep smallest keys
            if (wave == 0) {
                const uint32_t n = cnt;
                uint64_t k[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) k[i] = (uint32_t)(lane * 16 + i) < n ? buf[lane * 16 + i] : kInvalidKey;
                wave_bitonic_sort<16>(k);
#pragma unroll
                for (int i = 0; i < 16; ++i) buf[lane * 16 + i] = k[i];
                __builtin_amdgcn_wave_barrier();
                if (lane == 0) {
                    if (n >= kExactKeep) {
                        cnt = kExactKeep;
                        thr = buf[kExactKeep - 1];
                    }
                }
            }
            __syncthreads();
        };
        for (uint64_t c0 = c_first; c0 < c_last; c0 += kExactStep) {
            const uint64_t bound = thr;
#pragma unroll 1
            for (uint32_t t = 0; t < kExactStep / 32; ++t) {
                const uint64_t col = c0 + 32u * t + (uint32_t)grp;
                bool ok = col < c_last;
                if (ok && a.filter == kFilterRange) {
                    const uint64_t ts = a.ts[col];
                    ok = ts >= w0 && ts < w1;
                } else if (ok && a.filter == kFilterMask) {
                    ok = (mask >> (a.labels[col] & 63)) & 1ull;
                }
                if (ok) {  // uniform over the eight lanes of the column
                    const float d = group8_distance<METRIC>(q, a.B + (size_t)col * a.dim, a.dim, j);
                    const uint64_t key = make_sel_key(d, (uint32_t)col);
                    if (j == 0 && key < bound) buf[atomicAdd(&cnt, 1u)] = key;  // at most kExactKeep + kExactStep <= kExactBuf entries
                }
            }
            __syncthreads();
            const uint32_t listed = cnt;
            __syncthreads();  // everyone has read the count before anyone appends again
            if (listed > kExactBuf - kExactStep) compact();
        }
        compact();
        const uint32_t n = min(cnt, kExactKeep);
        uint64_t* out = a.cand + (size_t)row * a.nc;
        for (uint32_t g = threadIdx.x; g < a.nc; g += 256) out[g] = g < n ? buf[g] : kInvalidKey;
        __syncthreads();
    }
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

namespace {
std::atomic<int> g_knn_bf16{1};                 // process-wide: may the symmetric pass run on bf16 instructions (grab_knn_allow_bf16)
thread_local double g_last_flop = 0.0;          // matrix work of this thread's last exact_topk call: fp32 instructions,
thread_local double g_last_flop_bf16 = 0.0;     // and bf16 instructions (three per product of the split rows, 128 dimensions)
thread_local uint64_t g_last_redone_rows = 0;   // rows its symmetric pass handed to the plain pass
thread_local uint64_t g_last_exact_rows = 0;    // rows that its candidates did not prove and the exact pass redid
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
    const bool same = (p.A == p.B && p.M == p.N);
    // A row set against itself (the kNN graph): only the tiles on and above the diagonal are computed.  A tile
    // above it is read twice - along its rows for the rows of A, as ever, and along its columns for the dataset rows
    // behind them, whose tile below the diagonal is never computed.  The rows behind the columns belong to other
    // work items, so their keys go to per-row lists in device memory, and only keys within a per-row bound go
    // there: the bound comes from a first pass against a sample of the rows and is chosen so that about twice the
    // needed number of keys lie within it.  merge_symmetric_kernel checks row by row that enough did; the few
    // rows where not are redone by the plain pass.  Same candidates as the plain pass, half the matrix work.
    const bool split_ok = g_knn_bf16.load(std::memory_order_relaxed) != 0 && p.metric == kMetricL2 && p.dim <= 128;
    bool sym = same && p.filter_kind == kFilterNone && p.N >= (split_ok ? kSymMinRowsSplit : kSymMinRows) && kk <= kSymMaxKeep &&
               (size_t)p.N * kSymColCap * sizeof(uint64_t) <= kSymMaxListBytes;
    DeviceScratch col_list;
    if (sym && col_list.alloc((size_t)p.N * kSymColCap * sizeof(uint64_t)) != hipSuccess) {
        (void)hipGetLastError();  // no room for the lists: the plain pass needs none
        sym = false;
    }
    uint32_t nsplit = 1;
    if (row_tiles < target && !sym) nsplit = std::min<uint32_t>((target + row_tiles - 1) / row_tiles, std::min<uint32_t>(col_tiles, 1024 / kk));
    nsplit = std::max(nsplit, 1u);
    uint32_t tiles_per_split = (col_tiles + nsplit - 1) / nsplit;
    nsplit = (col_tiles + tiles_per_split - 1) / tiles_per_split;
    const uint32_t nwork = row_tiles * nsplit;
    const uint32_t grid = std::min(nwork, target);
    const double tile_flop = 2.0 * TM * TN * p.dim;
    g_last_redone_rows = 0;
    g_last_exact_rows = 0;
    g_last_flop_bf16 = 0.0;
    g_last_flop = tile_flop * (sym ? 0.5 * row_tiles * (row_tiles + 1.0) : (double)row_tiles * col_tiles);

    DeviceScratch buf, cand, normA, normB, doubt;
    // the symmetric pass may redo rows with a launch of up to `target` workgroups, whatever the main grid
    GRAB_HIP(buf.alloc((size_t)(sym ? target : grid) * TM * CAP * sizeof(uint64_t)));
    GRAB_HIP(cand.alloc((size_t)p.M * nsplit * kk * sizeof(uint64_t)));
    {   // the squared norms: terms of the L2 form, and for both metrics the scale of the rounding error that the
        // check after the re-scoring allows for.  doubt: [0] rows that fail it, [1..M] which, [M+1] max |b|^2
        GRAB_HIP(normB.alloc((size_t)p.N * 4));
        hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((p.N * 8 + 255) / 256)), dim3(256), 0, stream, p.B,
                           (uint32_t)p.N, p.dim, normB.as<float>());
        if (!same) {
            GRAB_HIP(normA.alloc((size_t)p.M * 4));
            hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((p.M * 8 + 255) / 256)), dim3(256), 0, stream, p.A,
                               (uint32_t)p.M, p.dim, normA.as<float>());
        }
        GRAB_HIP(doubt.alloc(((size_t)p.M + 3) * 4));  // [M+2]: max |b|^2 of the centred rows, where the split-bf16 pass runs
        GRAB_HIP(hipMemsetAsync(doubt.ptr, 0, 4, stream));
        GRAB_HIP(hipMemsetAsync(doubt.as<uint32_t>() + p.M + 1, 0, 8, stream));
        hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<size_t>((p.N + 255) / 256, 512)), dim3(256), 0, stream, normB.as<float>(), (uint64_t)p.N,
                           doubt.as<uint32_t>() + p.M + 1);
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
    t.row_lo = p.row_lo;
    t.row_hi = p.row_hi;
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

    DeviceScratch sample_rows, sample_norms, sample_cand, col_bound, col_count, redo, redo_part, bound_ws;
    uint32_t n_sample = 0, rank = 0;
    // The bounds only steer the symmetric pass (a row whose bound admits too few keys is redone), so where the bf16
    // estimate applies - squared L2, rows of up to 128 dimensions, a rank its classes of columns can stand in for -
    // it replaces the fp32 pass against the sample
    bool bf16_bound = false;
    if (sym) {
        n_sample = (uint32_t)std::min<size_t>(kSymSample, p.N / 16);  // the rank below stays within what the bf16 estimate stands in for
        rank = std::max<uint32_t>(kSymRank, (uint32_t)((2ull * kk * n_sample + p.N - 1) / p.N));
        GRAB_REQUIRE(rank <= 768, "internal: bounding rank %u", rank);
        bf16_bound = split_ok && rank <= bf16_bound_classes() / 2;
        if (bf16_bound) {
            GRAB_HIP(bound_ws.alloc(bf16_bound_workspace_bytes(p.N, n_sample)));
        } else {
            GRAB_HIP(sample_rows.alloc((size_t)n_sample * p.dim * 4));
            GRAB_HIP(sample_norms.alloc((size_t)n_sample * 4));
            GRAB_HIP(sample_cand.alloc((size_t)p.N * rank * sizeof(uint64_t)));
        }
        GRAB_HIP(col_bound.alloc((size_t)p.N * 4));
        GRAB_HIP(col_count.alloc((size_t)p.N * 4 + 4));  // last word: number of rows to redo
        GRAB_HIP(redo.alloc((size_t)p.N * 4));
        GRAB_HIP(hipMemsetAsync(col_count.ptr, 0, (size_t)p.N * 4 + 4, stream));
        if (!bf16_bound) {
            hipLaunchKernelGGL(spaced_rows_kernel, dim3((n_sample * 8 + 255) / 256), dim3(256), 0, stream, p.B, (uint64_t)p.N, n_sample, p.dim,
                               sample_rows.as<float>(), sample_norms.as<float>());
            GRAB_HIP(hipGetLastError());
        }
    }

    // Where the pass above does not apply (inner product, rows beyond 128 dimensions, two different row sets) the
    // contraction still leaves the fp32 pipe when there is enough of it to pay for the copies: the same kernels on
    // rows split into bf16 halves - the symmetric pass with its bounding pass and the rows it redoes, or the plain one.
    const bool split_tiles = !bf16_bound && g_knn_bf16.load(std::memory_order_relaxed) != 0 && p.dim % KC == 0 &&
                             (sym || (p.M >= 1024 && p.N >= 4096));
    DeviceScratch split_buf, split_norm_buf, split_mean, split_buf_a, split_norm_buf_a;
    const float* split_cnorm = nullptr;    // norms of the rows of B as split: centred for squared L2
    const float* split_cnorm_a = nullptr;  // ... of the rows of A
    if (split_tiles) {
        GRAB_HIP(split_buf.alloc((size_t)p.N * p.dim * 4));
        GRAB_HIP(split_norm_buf.alloc((size_t)p.N * 4));
        const float* mean = nullptr;
        if (p.metric == kMetricL2) {
            GRAB_HIP(split_mean.alloc((size_t)p.dim * 4));
            hipLaunchKernelGGL(spaced_mean_kernel, dim3(p.dim), dim3(256), 0, stream, p.B, (uint64_t)p.N, (uint32_t)std::min<size_t>(p.N, 8192),
                               p.dim, split_mean.as<float>());
            mean = split_mean.as<float>();
        }
        hipLaunchKernelGGL(split_rows_chunked_kernel, dim3((uint32_t)(((size_t)p.N * 8 + 255) / 256)), dim3(256), 0, stream, p.B,
                           (uint64_t)p.N, p.dim, mean, split_buf.as<uint16_t>(), split_norm_buf.as<float>());
        GRAB_HIP(hipGetLastError());
        split_cnorm = split_cnorm_a = split_norm_buf.as<float>();
        t.A = t.B = split_buf.as<float>();
        if (!same) {  // the other row set, about the same mean
            GRAB_HIP(split_buf_a.alloc((size_t)p.M * p.dim * 4));
            GRAB_HIP(split_norm_buf_a.alloc((size_t)p.M * 4));
            hipLaunchKernelGGL(split_rows_chunked_kernel, dim3((uint32_t)(((size_t)p.M * 8 + 255) / 256)), dim3(256), 0, stream, p.A,
                               (uint64_t)p.M, p.dim, mean, split_buf_a.as<uint16_t>(), split_norm_buf_a.as<float>());
            GRAB_HIP(hipGetLastError());
            split_cnorm_a = split_norm_buf_a.as<float>();
            t.A = split_buf_a.as<float>();
        }
        t.normA = split_cnorm_a;
        t.normB = split_cnorm;
        hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<size_t>((p.N + 255) / 256, 512)), dim3(256), 0, stream, split_cnorm, (uint64_t)p.N,
                           doubt.as<uint32_t>() + p.M + 2);
        if (sym)
            hipLaunchKernelGGL(spaced_rows_kernel, dim3((n_sample * 8 + 255) / 256), dim3(256), 0, stream, split_buf.as<float>(), (uint64_t)p.N,
                               n_sample, p.dim, sample_rows.as<float>(), sample_norms.as<float>(), split_cnorm);
        GRAB_HIP(hipGetLastError());
        if (!sym) {
            g_last_flop_bf16 = 3.0 * g_last_flop;
            g_last_flop = 0.0;
        }
    }

    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (kernel_ms) {
        GRAB_HIP(hipEventCreate(&e0));
        GRAB_HIP(hipEventCreate(&e1));
        GRAB_HIP(hipEventRecord(e0, stream));
    }
    int rc = GRAB_OK;
    const uint16_t* split_rows = nullptr;
    const float* split_norms = nullptr;
    if (sym) {
        if (bf16_bound) {
            rc = bf16_bounds_async(p.B, (uint32_t)p.N, p.dim, n_sample, rank, bound_ws.ptr, col_bound.as<float>(), stream, &split_rows, &split_norms);
        } else {
            TileArgs b = t;  // the bounding pass: every row against the sample
            b.B = sample_rows.as<float>();
            b.normB = sample_norms.as<float>();
            b.N = n_sample;
            b.kk = rank;
            b.col_tiles = (n_sample + TN - 1) / TN;
            b.tiles_per_split = b.col_tiles;
            b.cand_out = sample_cand.as<uint64_t>();
            if (split_tiles) {  // three bf16 instructions a product; nothing of this pass runs on fp32 instructions
                g_last_flop = 0.0;
                g_last_flop_bf16 = 3.0 * tile_flop * (0.5 * row_tiles * (row_tiles + 1.0) + (double)row_tiles * b.col_tiles);
            } else {
                g_last_flop += tile_flop * row_tiles * b.col_tiles;
            }
            rc = p.metric == kMetricIP ? launch_tile<kMetricIP>(b, kFilterNone, grid, stream, split_tiles)
                                       : launch_tile<kMetricL2>(b, kFilterNone, grid, stream, split_tiles);
            if (rc == GRAB_OK)
                hipLaunchKernelGGL(column_bound_kernel, dim3((t.M + 255) / 256), dim3(256), 0, stream, sample_cand.as<uint64_t>(), rank, t.M,
                                   col_bound.as<float>());
        }
        if (rc == GRAB_OK) {
            t.col_bound = col_bound.as<float>();
            t.col_list = col_list.as<uint64_t>();
            t.col_count = col_count.as<uint32_t>();
            t.col_cap = kSymColCap;
            if (bf16_bound) {
                // where the bounds came from the bf16 pipe (squared L2, up to 128 dimensions) the pass runs there too,
                // on the split rows the bounding pass left behind: three instructions a product, each at 16x the rate
                TileArgs ts = t;
                ts.normA = ts.normB = split_norms;
                g_last_flop = 0.0;
                const double tile_flop_bf16 = 2.0 * TM * TN * 128;
                g_last_flop_bf16 = 3.0 * tile_flop_bf16 * 0.5 * row_tiles * (row_tiles + 1.0) + tile_flop_bf16 * row_tiles * ((n_sample + TN - 1) / TN);
                hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<size_t>((p.N + 255) / 256, 512)), dim3(256), 0, stream, split_norms, (uint64_t)p.N,
                                   doubt.as<uint32_t>() + p.M + 2);
                rc = launch_sym_split(ts, split_rows, std::min<uint32_t>(row_tiles, (uint32_t)num_cu), stream);
            } else {
                rc = p.metric == kMetricIP ? launch_tile<kMetricIP>(t, kFilterSymmetric, grid, stream, split_tiles)
                                           : launch_tile<kMetricL2>(t, kFilterSymmetric, grid, stream, split_tiles);
            }
        }
    } else {
        rc = p.metric == kMetricIP ? launch_tile<kMetricIP>(t, p.filter_kind, grid, stream, split_tiles)
                                   : launch_tile<kMetricL2>(t, p.filter_kind, grid, stream, split_tiles);
    }
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

    if (sym) {
        uint32_t* redo_count = col_count.as<uint32_t>() + p.N;
        hipLaunchKernelGGL(merge_symmetric_kernel, dim3((t.M + 3) / 4), dim3(256), 0, stream, cand.as<uint64_t>(), col_list.as<uint64_t>(),
                           col_count.as<uint32_t>(), kSymColCap, col_bound.as<float>(), kk, t.M, redo.as<uint32_t>(), redo_count);
        GRAB_HIP(hipGetLastError());
        uint32_t n_redo = 0;
        GRAB_HIP(hipMemcpyAsync(&n_redo, redo_count, 4, hipMemcpyDeviceToHost, stream));
        GRAB_HIP(hipStreamSynchronize(stream));
        if (n_redo > 0) {  // the plain pass over the listed rows, in as many column slices as one sort can merge
            TileArgs f = t;
            f.M = n_redo;
            f.row_perm = redo.as<uint32_t>();
            f.row_tiles = (n_redo + TM - 1) / TM;
            // few rows: the columns are cut into as many slices as fill the machine, and the slices' lists are merged
            // in rounds of as many as one sort holds
            f.nsplit = std::max(1u, std::min((target + f.row_tiles - 1) / f.row_tiles, col_tiles));
            f.tiles_per_split = (col_tiles + f.nsplit - 1) / f.nsplit;
            f.nsplit = (col_tiles + f.tiles_per_split - 1) / f.tiles_per_split;
            f.cand_by_grid_row = 1;
            g_last_redone_rows = n_redo;
            if (split_tiles) g_last_flop_bf16 += 3.0 * tile_flop * f.row_tiles * col_tiles;
            else g_last_flop += tile_flop * f.row_tiles * col_tiles;
            const uint32_t per = std::max(2u, 1024u / kk);
            const uint32_t first_groups = (f.nsplit + per - 1) / per;
            GRAB_HIP(redo_part.alloc(((size_t)n_redo * f.nsplit + (size_t)n_redo * first_groups) * kk * sizeof(uint64_t)));
            f.cand_out = redo_part.as<uint64_t>();
            const uint32_t fgrid = std::min(f.row_tiles * f.nsplit, target);
            GRAB_TRY(p.metric == kMetricIP ? launch_tile<kMetricIP>(f, kFilterNone, fgrid, stream, split_tiles)
                                           : launch_tile<kMetricL2>(f, kFilterNone, fgrid, stream, split_tiles));
            uint64_t* from = redo_part.as<uint64_t>();
            uint64_t* to = from + (size_t)n_redo * f.nsplit * kk;  // a round's output is at most as long as this; the rounds go to and fro
            for (uint32_t parts = f.nsplit;;) {
                const uint32_t groups = (parts + per - 1) / per;
                hipLaunchKernelGGL(merge_redone_kernel, dim3((uint32_t)(((size_t)n_redo * groups + 3) / 4)), dim3(256), 0, stream, from, parts, per, kk,
                                   redo.as<uint32_t>(), n_redo, to, cand.as<uint64_t>());
                GRAB_HIP(hipGetLastError());
                if (groups == 1) break;
                std::swap(from, to);
                parts = groups;
            }
        }
    }

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
    r.kk = kk;
    r.normA = same ? normB.as<float>() : normA.as<float>();
    r.max_normB = reinterpret_cast<const float*>(doubt.as<uint32_t>() + p.M + 1);
    r.doubt = doubt.as<uint32_t>();
    r.sorted = sym ? 1 : 0;  // merge_symmetric_kernel and merge_redone_kernel leave a row's candidates in ascending order
    if (split_rows != nullptr) {
        r.split_normA = split_norms;
        r.split_max_normB = reinterpret_cast<const float*>(doubt.as<uint32_t>() + p.M + 2);
        r.split_terms = 3.0f * 128.0f + 6.0f;
    } else if (split_tiles) {
        r.split_normA = split_cnorm_a;
        r.split_max_normB = reinterpret_cast<const float*>(doubt.as<uint32_t>() + p.M + 2);
        r.split_terms = 3.0f * (float)p.dim;
    }
    GRAB_REQUIRE(r.nc <= 1024, "internal: too many candidates per row");
    GRAB_TRY(p.metric == kMetricIP ? launch_refine<kMetricIP>(r, stream) : launch_refine<kMetricL2>(r, stream));
    uint32_t n_doubt = 0;
    GRAB_HIP(hipMemcpyAsync(&n_doubt, doubt.ptr, 4, hipMemcpyDeviceToHost, stream));
    GRAB_HIP(hipStreamSynchronize(stream));
    g_last_exact_rows = n_doubt;
    if (n_doubt > 0) {
        // rows whose candidates prove nothing: every admissible column scored exactly, then the same emit step
        ExactArgs x{};
        x.A = p.A;
        x.B = p.B;
        x.rows = doubt.as<uint32_t>() + 1;
        x.count = n_doubt;
        x.dim = p.dim;
        x.nc = r.nc;
        x.N = p.N;
        x.filter = p.filter_kind;
        x.ts = p.ts;
        x.win_start_arr = p.win_start_arr;
        x.win_end_arr = p.win_end_arr;
        x.win_start = p.win_start;
        x.win_end = p.win_end;
        x.per_query_window = p.per_query_window;
        x.labels = p.labels;
        x.masks = p.masks;
        x.row_lo = p.row_lo;
        x.row_hi = p.row_hi;
        x.cand = cand.as<uint64_t>();
        const uint32_t xgrid = std::min<uint32_t>(n_doubt, (uint32_t)num_cu * 8);
        if (p.metric == kMetricIP) hipLaunchKernelGGL(exact_rows_kernel<kMetricIP>, dim3(xgrid), dim3(256), 0, stream, x);
        else hipLaunchKernelGGL(exact_rows_kernel<kMetricL2>, dim3(xgrid), dim3(256), 0, stream, x);
        GRAB_HIP(hipGetLastError());
        r.rows = x.rows;
        r.M = n_doubt;
        r.doubt = nullptr;
        GRAB_TRY(p.metric == kMetricIP ? launch_refine<kMetricIP>(r, stream) : launch_refine<kMetricL2>(r, stream));
        GRAB_HIP(hipStreamSynchronize(stream));
    }
    return GRAB_OK;
}

// ---------------------------------------------------------------------------------------------
// Entry-point layer: an evenly spaced sample of the base, in timestamp order.  For a batch of
// queries the nearest admissible sample rows are found with the contraction kernel above and
// handed to the beam search as seeds.  The reference's closest counterpart is the "virtual
// index" of TimeStampIndex (src/timeStampIndex.cu:141-238: k-means centroids with entry
// points that seed the per-bucket searches); its CagraIndex::query_range seeds with a random
// sample of the window instead (src/cagraIndex.cu:270-295), which cannot reach a cluster of
// the data that holds no seed.
// ---------------------------------------------------------------------------------------------
namespace {

__global__ void __launch_bounds__(256) gather_sample_kernel(const float* __restrict__ data, uint32_t dim, uint64_t n,
                                                            const uint32_t* __restrict__ ids_by_ts,
                                                            const uint64_t* __restrict__ ts, const uint8_t* __restrict__ labels,
                                                            uint32_t S, float* __restrict__ sample, uint32_t* __restrict__ sample_ids,
                                                            uint64_t* __restrict__ sample_ts, uint8_t* __restrict__ sample_labels) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= S) return;
    const uint64_t pos = (uint64_t)g * n / S;
    const uint32_t id = ids_by_ts ? ids_by_ts[pos] : (uint32_t)pos;
    const float4* src = reinterpret_cast<const float4*>(data + (size_t)id * dim);
    float4* dst = reinterpret_cast<float4*>(sample + (size_t)g * dim);
    for (uint32_t c = j; c < (dim >> 2); c += 8) dst[c] = src[c];
    if (j == 0) {
        sample_ids[g] = id;
        if (sample_ts) sample_ts[g] = ts[id];
        if (sample_labels) sample_labels[g] = labels[id];
    }
}

__device__ __forceinline__ uint32_t lower_bound_ts(const uint64_t* a, uint32_t n, uint64_t v) {
    uint32_t lo = 0, hi = n;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (a[mid] < v) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// per query: the run of sample rows inside its window, and a sort key (run start, query)
__global__ void __launch_bounds__(256) window_to_columns_kernel(const uint64_t* __restrict__ sample_ts, uint32_t S,
                                                                const uint64_t* __restrict__ ws_arr, const uint64_t* __restrict__ we_arr,
                                                                uint64_t ws0, uint64_t we0, int per_query, uint32_t nq,
                                                                uint32_t padded, uint32_t* __restrict__ lo, uint32_t* __restrict__ hi,
                                                                uint64_t* __restrict__ keys) {
    __shared__ uint64_t piv[kPivots];
    const uint64_t step = load_pivots(sample_ts, S, piv);
    __syncthreads();
    const uint32_t q = blockIdx.x * 256 + threadIdx.x;
    if (q >= padded) return;
    if (q >= nq) {
        keys[q] = kInvalidKey;
        return;
    }
    const uint32_t l = (uint32_t)lower_bound_pivots(sample_ts, S, piv, step, per_query ? ws_arr[q] : ws0);
    uint32_t h = (uint32_t)lower_bound_pivots(sample_ts, S, piv, step, per_query ? we_arr[q] : we0);
    if (h < l) h = l;
    lo[q] = l;
    hi[q] = h;
    keys[q] = ((uint64_t)l << 32) | q;
}

// queries in their own order: for a layer whose every query admits every column, where the order decides nothing
__global__ void __launch_bounds__(256) identity_order_kernel(uint32_t* __restrict__ perm, uint32_t nq) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < nq) perm[i] = i;
}

__global__ void __launch_bounds__(256) keys_to_perm_kernel(const uint64_t* __restrict__ keys, uint32_t nq, uint32_t* __restrict__ perm) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < nq) perm[i] = (uint32_t)(keys[i] & 0xFFFFFFFFull);
}

// One workgroup orders up to 16384 queries by the start of their column run (counting sort
// over 2048 bins; the order inside a bin is arbitrary, which only decides which tile a query
// shares with which neighbours) and lays out the work of the dense-store contraction: per
// tile of 128 ordered queries the column tiles that some query of the tile admits, cut into
// items of `per` column tiles so that `grid` workgroups finish together.
__global__ void __launch_bounds__(1024) bucket_order_kernel(const uint32_t* __restrict__ lo, const uint32_t* __restrict__ hi,
                                                            uint32_t M, uint32_t S, uint32_t grid, uint32_t* __restrict__ perm,
                                                            uint32_t* __restrict__ sched) {
    constexpr uint32_t NB = 2048;
    __shared__ uint32_t bins[NB];
    __shared__ uint32_t tlo[128], thi[128], items[129];
    __shared__ uint32_t wsum[16];
    __shared__ uint32_t total;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t row_tiles = (M + TM - 1) / TM;
    bins[tid] = 0;
    bins[tid + 1024] = 0;
    if (tid < 128) {
        tlo[tid] = 0xFFFFFFFFu;
        thi[tid] = 0;
    }
    if (tid == 0) total = 0;
    __syncthreads();
    auto bin_of = [&](uint32_t l) { return (uint32_t)(((uint64_t)l * NB) / ((uint64_t)S + 1)); };
    // a thread owns the queries tid, tid + 1024, ... (at most 16): their runs are read once, all loads in flight
    constexpr int PER = 16;
    uint32_t mylo[PER], myhi[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const uint32_t q = tid + 1024u * j;
        mylo[j] = q < M ? lo[q] : 0u;
        myhi[j] = q < M ? hi[q] : 0u;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
        if (tid + 1024u * j < M) atomicAdd(&bins[bin_of(mylo[j])], 1u);
    __syncthreads();
    {  // exclusive scan of the bins, two per thread
        const uint32_t v0 = bins[2 * tid], v1 = bins[2 * tid + 1];
        uint32_t incl = v0 + v1;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = __shfl_up(incl, d, 64);
            if ((int)lane >= d) incl += o;
        }
        if (lane == 63) wsum[wave] = incl;
        __syncthreads();
        uint32_t base = 0;
        for (uint32_t w = 0; w < wave; ++w) base += wsum[w];
        const uint32_t excl = base + incl - (v0 + v1);
        bins[2 * tid] = excl;
        bins[2 * tid + 1] = excl + v0;
    }
    __syncthreads();
    // place every query and fold its run into the union of its tile of 128
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const uint32_t q = tid + 1024u * j;
        if (q < M) {
            const uint32_t pos = atomicAdd(&bins[bin_of(mylo[j])], 1u);
            perm[pos] = q;
            if (mylo[j] < myhi[j]) {
                atomicMin(&tlo[pos / TM], mylo[j]);
                atomicMax(&thi[pos / TM], myhi[j]);
            }
        }
    }
    __syncthreads();
    uint32_t c_lo = 0, c_hi = 0;
    if (tid < row_tiles) {
        c_lo = tlo[tid] < thi[tid] ? tlo[tid] / TN : 0;
        c_hi = tlo[tid] < thi[tid] ? (thi[tid] + TN - 1) / TN : 0;
        atomicAdd(&total, c_hi - c_lo);
    }
    __syncthreads();
    // wave w prices items of w+1 column tiles: rounds of `grid` concurrent items, each costing its
    // tiles plus a fixed start-up of about a third of a tile; the cheapest size wins
    __shared__ uint32_t cnts[128], cost[16];
    if (tid < 128) cnts[tid] = tid < row_tiles ? c_hi - c_lo : 0;
    __syncthreads();
    {
        const uint32_t base = max(1u, total / (grid * 8u));  // long sweeps: about 8 items per workgroup
        const uint32_t cand = base + wave;
        uint32_t n = (cnts[lane] + cand - 1) / cand + (cnts[lane + 64] + cand - 1) / cand;
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) n += __shfl_xor(n, m, 64);
        if (lane == 0) cost[wave] = ((n + grid - 1) / grid) * (3 * cand + 1);
    }
    __syncthreads();
    uint32_t per = max(1u, total / (grid * 8u));
    {
        uint32_t best = cost[0], arg = 0;
        for (uint32_t w = 1; w < 16; ++w)
            if (cost[w] < best) {
                best = cost[w];
                arg = w;
            }
        per += arg;
    }
    if (tid < row_tiles) {
        items[tid] = (c_hi - c_lo + per - 1) / per;
        sched[kSchedLo + tid] = c_lo;
        sched[kSchedHi + tid] = c_hi;
    }
    __syncthreads();
    if (tid <= row_tiles) {  // exclusive prefix of the item counts, one entry per thread
        uint32_t acc = 0;
        for (uint32_t t = 0; t < tid; ++t) acc += items[t];
        sched[kSchedOff + tid] = acc;
        if (tid == row_tiles) {
            sched[kSchedPer] = per;
            sched[kSchedItems] = acc;
        }
    }
}

// dst row i = src row perm[i] and its squared norm, 8 lanes per row (the summation order of row_norms_kernel)
__global__ void __launch_bounds__(256) gather_rows_norms_kernel(const float* __restrict__ src, const uint32_t* __restrict__ perm,
                                                                uint32_t M, uint32_t dim, float* __restrict__ dst,
                                                                float* __restrict__ norms) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= M) return;
    const float4* r4 = reinterpret_cast<const float4*>(src + (size_t)perm[g] * dim);
    float4* d4 = reinterpret_cast<float4*>(dst + (size_t)g * dim);
    float s = 0.0f;
    for (uint32_t c = j; c < (dim >> 2); c += 8) {
        const float4 v = r4[c];
        d4[c] = v;
        s = __builtin_fmaf(v.x, v.x, s);
        s = __builtin_fmaf(v.y, v.y, s);
        s = __builtin_fmaf(v.z, v.z, s);
        s = __builtin_fmaf(v.w, v.w, s);
    }
    s = group8_sum(s);
    if (j == 0 && norms != nullptr) norms[g] = s;
}

// one wave per query: best n_seeds of the nsplit partial lists, mapped to row ids of the base
template <int NPL>
__global__ void __launch_bounds__(256) finalize_seeds_kernel(const uint64_t* __restrict__ cand, uint32_t nc, uint32_t nq,
                                                             const uint32_t* __restrict__ sample_ids, uint32_t n_seeds,
                                                             uint32_t* __restrict__ out) {
    __shared__ uint64_t keys[4][64 * NPL];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t q = blockIdx.x * 4 + wave;
    if (q >= nq) return;
    uint64_t k[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const uint32_t g = lane * NPL + i;
        k[i] = g < nc ? cand[(size_t)q * nc + g] : kInvalidKey;
    }
    wave_bitonic_sort<NPL>(k);
#pragma unroll
    for (int i = 0; i < NPL; ++i) keys[wave][lane * NPL + i] = k[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (uint32_t o = lane; o < n_seeds; o += 64) {
        const uint64_t kk = o < 64u * NPL ? keys[wave][o] : kInvalidKey;
        out[(size_t)q * n_seeds + o] = kk == kInvalidKey ? kInvalidId : sample_ids[(uint32_t)(kk & 0xFFFFFFFFull)];
    }
}

// One wave per query walks the query's run of columns in the dense distance matrix and keeps the
// n_seeds (<= 64) smallest (distance,column) keys, one per lane, sorted across lanes.  A key that
// beats the current worst is inserted by shifting the tail of the list one lane up (DPP and
// v_readlane only); after the first few hundred columns almost every step fails the float
// pre-test and costs a compare per column.
__global__ void __launch_bounds__(256) stream_select_kernel(const float* __restrict__ dense, uint64_t pitch,
                                                            const uint32_t* __restrict__ perm, const uint32_t* __restrict__ lo,
                                                            const uint32_t* __restrict__ hi, uint32_t nq,
                                                            const uint32_t* __restrict__ sample_ids, uint32_t n_seeds,
                                                            uint32_t* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= nq) return;
    const uint32_t q = perm ? perm[row] : row;
    const uint32_t c_lo = lo[q], c_hi = hi[q];
    const float* drow = dense + (size_t)row * pitch;
    uint64_t mykey = kInvalidKey, thr = kInvalidKey;
    float thr_d = __builtin_inff();
    auto offer = [&](uint64_t key) {  // every lane calls this with its own key
        uint64_t b = __ballot(key < thr);
        while (b != 0) {
            const int bit = (int)__builtin_ctzll(b);
            b &= b - 1;
            const uint64_t x = readlane_u64(key, bit);
            if (x < thr) {  // wave-uniform
                const uint32_t p = (uint32_t)__popcll(__ballot(mykey < x));
                const uint64_t up = shfl_up_u64(mykey);
                if ((uint32_t)lane == p) mykey = x;
                else if ((uint32_t)lane > p && (uint32_t)lane < n_seeds) mykey = up;
                thr = readlane_u64(mykey, (int)n_seeds - 1);
                thr_d = thr == kInvalidKey ? __builtin_inff() : ord_float((uint32_t)(thr >> 32));
            }
        }
    };
    // 512 columns per step: two runs of four consecutive columns per lane; the next step's loads
    // are issued before this step's values are looked at
    constexpr uint32_t STEP = 512;
    const uint32_t c_begin = c_lo & ~(STEP - 1);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    auto load4 = [&](uint32_t c) { return c < c_hi ? *reinterpret_cast<const float4*>(drow + c) : zero; };
    float4 cur0 = zero, cur1 = zero;
    if (c_begin < c_hi) {
        cur0 = load4(c_begin + 4 * lane);
        cur1 = load4(c_begin + 256 + 4 * lane);
    }
    for (uint32_t c0 = c_begin; c0 < c_hi; c0 += STEP) {
        float4 nxt0 = zero, nxt1 = zero;
        if (c0 + STEP < c_hi) {
            nxt0 = load4(c0 + STEP + 4 * lane);
            nxt1 = load4(c0 + STEP + 256 + 4 * lane);
        }
        const float dv[8] = {cur0.x, cur0.y, cur0.z, cur0.w, cur1.x, cur1.y, cur1.z, cur1.w};
        const bool interior = c0 >= c_lo && c0 + STEP <= c_hi;  // wave-uniform
        bool any = false;
        if (interior) {
#pragma unroll
            for (int e = 0; e < 8; ++e) any = any || dv[e] <= thr_d;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t c = c0 + (e >> 2) * 256 + 4 * lane + (e & 3);
                any = any || (c >= c_lo && c < c_hi && dv[e] <= thr_d);
            }
        }
        if (__ballot(any) != 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t c = c0 + (e >> 2) * 256 + 4 * lane + (e & 3);
                const bool in = c >= c_lo && c < c_hi && dv[e] <= thr_d;
                offer(in ? make_sel_key(dv[e], c) : kInvalidKey);
            }
        }
        cur0 = nxt0;
        cur1 = nxt1;
    }
    if ((uint32_t)lane < n_seeds)
        out[(size_t)q * n_seeds + lane] = mykey == kInvalidKey ? kInvalidId : sample_ids[(uint32_t)(mykey & 0xFFFFFFFFull)];
}

// The same walk for the scan of id intervals: one wave per tile-grid row of a dense matrix whose rows start at the first
// column tile of their row tile (sched holds it).  The kk (<= 64) smallest (distance, column) keys of the row's columns
// [lo, hi) go to keys[query][kk] in ascending order; rows that admit no column are padding.
__global__ void __launch_bounds__(256) stream_select_keys_kernel(const float* __restrict__ dense, uint64_t pitch,
                                                                 const uint32_t* __restrict__ row_query, const uint32_t* __restrict__ row_lo,
                                                                 const uint32_t* __restrict__ row_hi, const uint32_t* __restrict__ sched,
                                                                 uint32_t nrows, uint32_t kk, uint64_t* __restrict__ out_keys) {
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= nrows) return;
    const uint32_t c_lo = row_lo[row], c_hi = row_hi[row];
    if (c_lo >= c_hi) return;
    const uint32_t base = sched[kSchedLo + row / TM] * TN;  // <= c_lo: the row tile's sweep starts at or before every interval of its rows
    const float* drow = dense + (size_t)row * pitch;
    uint64_t mykey = kInvalidKey, thr = kInvalidKey;
    float thr_d = __builtin_inff();
    auto offer = [&](uint64_t key) {  // every lane calls this with its own key
        uint64_t b = __ballot(key < thr);
        while (b != 0) {
            const int bit = (int)__builtin_ctzll(b);
            b &= b - 1;
            const uint64_t x = readlane_u64(key, bit);
            if (x < thr) {  // wave-uniform
                const uint32_t p = (uint32_t)__popcll(__ballot(mykey < x));
                const uint64_t up = shfl_up_u64(mykey);
                if ((uint32_t)lane == p) mykey = x;
                else if ((uint32_t)lane > p && (uint32_t)lane < kk) mykey = up;
                thr = readlane_u64(mykey, (int)kk - 1);
                thr_d = thr == kInvalidKey ? __builtin_inff() : ord_float((uint32_t)(thr >> 32));
            }
        }
    };
    // The first 512 columns of the interval at once: eight keys a lane, one sort, the kk smallest a lane each.  (Taken
    // one by one through `offer` they would nearly all be inserted - the list is empty at first - and an insertion is
    // a dozen wave-wide steps; after 512 columns one in eight still passes, after 5000 one in eighty.)
    uint32_t c_from = c_lo;
    if (c_hi - c_lo >= 512u) {
        uint64_t r[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t c = c_lo + 64u * i + (uint32_t)lane;
            r[i] = make_sel_key(drow[c - base], c);
        }
        dev::wave_bitonic_sort<8>(r);  // ascending, element lane * 8 + i in r[i]
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint64_t v = shfl_u64(r[i], lane >> 3);
            if ((lane & 7) == i) mykey = v;
        }
        if ((uint32_t)lane >= kk) mykey = kInvalidKey;
        thr = readlane_u64(mykey, (int)kk - 1);
        thr_d = ord_float((uint32_t)(thr >> 32));
        c_from = c_lo + 512u;
    }
    // 512 columns per step, two runs of four consecutive columns per lane, the next step's loads issued before this
    // step's values are looked at; steps are aligned to the row's first stored column
    constexpr uint32_t STEP = 512;
    const uint32_t c_begin = base + ((c_from - base) & ~(STEP - 1));
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    auto load4 = [&](uint32_t c) { return c < c_hi ? *reinterpret_cast<const float4*>(drow + (c - base)) : zero; };
    float4 cur0 = load4(c_begin + 4 * lane), cur1 = load4(c_begin + 256 + 4 * lane);
    for (uint32_t c0 = c_begin; c0 < c_hi; c0 += STEP) {
        float4 nxt0 = zero, nxt1 = zero;
        if (c0 + STEP < c_hi) {
            nxt0 = load4(c0 + STEP + 4 * lane);
            nxt1 = load4(c0 + STEP + 256 + 4 * lane);
        }
        const float dv[8] = {cur0.x, cur0.y, cur0.z, cur0.w, cur1.x, cur1.y, cur1.z, cur1.w};
        const bool interior = c0 >= c_from && c0 + STEP <= c_hi;  // wave-uniform
        bool any = false;
        if (interior) {
#pragma unroll
            for (int e = 0; e < 8; ++e) any = any || dv[e] <= thr_d;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t c = c0 + (e >> 2) * 256 + 4 * lane + (e & 3);
                any = any || (c >= c_from && c < c_hi && dv[e] <= thr_d);
            }
        }
        if (__ballot(any) != 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t c = c0 + (e >> 2) * 256 + 4 * lane + (e & 3);
                const bool in = c >= c_from && c < c_hi && dv[e] <= thr_d;
                offer(in ? make_sel_key(dv[e], c) : kInvalidKey);
            }
        }
        cur0 = nxt0;
        cur1 = nxt1;
    }
    if ((uint32_t)lane < kk) out_keys[(size_t)row_query[row] * kk + lane] = mykey;
}

// n (<= 48) smallest values of each row of a dense matrix with at most 1024 columns, one wave per row.
// Every lane reads 16 columns and keeps the smallest; the n-th smallest of the 64 lane minima bounds the
// n-th smallest value of the row from above, so only the columns at or below it (a few dozen) are listed
// and sorted.
__global__ void __launch_bounds__(256) select_short_rows_kernel(const float* __restrict__ dense, uint64_t pitch,
                                                                const uint32_t* __restrict__ perm, uint32_t ncols, uint32_t nq,
                                                                const uint32_t* __restrict__ sample_ids, uint32_t n_out,
                                                                uint32_t* __restrict__ out) {
    __shared__ uint64_t listed[4][1024];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= nq) return;
    const uint32_t q = perm ? perm[row] : row;
    const float* drow = dense + (size_t)row * pitch;
    const float inf = __builtin_inff();
    float v[16];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t c = e * 256 + 4 * lane;
        float4 x = make_float4(inf, inf, inf, inf);
        if (c < pitch) x = *reinterpret_cast<const float4*>(drow + c);
        v[4 * e + 0] = c + 0 < ncols ? x.x : inf;
        v[4 * e + 1] = c + 1 < ncols ? x.y : inf;
        v[4 * e + 2] = c + 2 < ncols ? x.z : inf;
        v[4 * e + 3] = c + 3 < ncols ? x.w : inf;
    }
    float m = v[0];
#pragma unroll
    for (int e = 1; e < 16; ++e) m = fminf(m, v[e]);
    uint64_t mk[1] = {((uint64_t)ord_bits(m) << 32) | (uint32_t)lane};
    wave_bitonic_sort<1>(mk);
    const float bound = ord_float((uint32_t)(readlane_u64(mk[0], (int)n_out - 1) >> 32));
    uint64_t* mine = listed[wave];
    const uint64_t below = (1ull << lane) - 1ull;
    uint32_t count = 0;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const bool in = v[e] <= bound && v[e] < inf;
        const uint64_t b = __ballot(in);
        if (in) mine[count + __popcll(b & below)] = make_sel_key(v[e], (uint32_t)((e >> 2) * 256 + 4 * lane + (e & 3)));
        count += (uint32_t)__popcll(b);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (count <= 64) {
        uint64_t k[1] = {(uint32_t)lane < count ? mine[lane] : kInvalidKey};
        wave_bitonic_sort<1>(k);
        if ((uint32_t)lane < n_out) out[(size_t)q * n_out + lane] = k[0] == kInvalidKey ? kInvalidId : sample_ids[(uint32_t)(k[0] & 0xFFFFFFFFull)];
    } else if (count <= 128) {
        uint64_t k[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) k[i] = (uint32_t)(lane * 2 + i) < count ? mine[lane * 2 + i] : kInvalidKey;
        wave_bitonic_sort<2>(k);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t r = lane * 2 + i;
            if (r < n_out) out[(size_t)q * n_out + r] = k[i] == kInvalidKey ? kInvalidId : sample_ids[(uint32_t)(k[i] & 0xFFFFFFFFull)];
        }
    } else {  // many equal values: sort everything that was listed
        uint64_t k[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) k[i] = (uint32_t)(lane * 16 + i) < count ? mine[lane * 16 + i] : kInvalidKey;
        wave_bitonic_sort<16>(k);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t r = lane * 16 + i;
            if (r < n_out) out[(size_t)q * n_out + r] = k[i] == kInvalidKey ? kInvalidId : sample_ids[(uint32_t)(k[i] & 0xFFFFFFFFull)];
        }
    }
}

// Coarse-to-fine seed selection.  The sample rows are grouped by nearest centroid; inside a group they keep
// their timestamp order, so the part of a group inside a query's window is one run of consecutive rows.
// A wave takes one query; lane p takes the group of the query's p-th nearest centroid (`probe`, nearest
// first) and cuts the run out with two binary searches.  The groups are taken nearest first until min_rows
// rows are reached (the group that crosses the mark is taken whole); the rows of all taken runs go into one
// list, eight lanes score a row, and the n_seeds (<= 64) smallest (distance, slot) keys stay sorted across
// the lanes.
constexpr uint32_t kProbeSlots = 512;
constexpr uint32_t kGroupStretches = 64;

// lower bound of v in an ascending array by a group of 16 consecutive lanes: every step looks at the last
// elements of 16 equal stretches at once, so a million entries take six dependent loads instead of twenty.
// All four groups of the wave must call this together (one ballot per step).
// The search runs over [lo, hi); the answer may be hi.  Groups with busy == false only keep the others company.
// (Indices are 32-bit: the arrays searched here have fewer than 2^31 entries.)
__device__ __forceinline__ uint32_t lower_bound_by16(const uint64_t* __restrict__ a, uint32_t lo, uint32_t hi, uint64_t v, bool busy,
                                                     int lane) {
    const uint32_t g = (uint32_t)lane & 15u;
    const int shift = lane & 48;
    while (__ballot(busy && lo < hi) != 0) {
        const bool act = busy && lo < hi;
        const uint32_t len = act ? hi - lo : 1u, step = (len + 15u) >> 4;
        const uint32_t end = min((g + 1u) * step, len);  // stretch g ends before `end`
        const bool less = act && a[lo + end - 1u] < v;
        const uint32_t k = (uint32_t)__popcll((__ballot(less) >> shift) & 0xFFFFull);  // stretches wholly below v
        if (act) {
            if (k == 16u) {
                lo = hi;
            } else {
                hi = lo + min((k + 1u) * step, len) - 1u;  // that element is >= v
                lo = lo + k * step;
            }
        }
    }
    return lo;
}

// LIST: the in-window rows of the groups are not scored; their base ids are written as they come (nearest group
// first, timestamp order inside a group), at most n_seeds of them - the search that takes them as seeds scores them anyway.
template <int CPL, int METRIC, bool LIST>
__global__ void __launch_bounds__(256) probe_groups_kernel(const float* __restrict__ queries, uint32_t nq, uint32_t dim,
                                                           const uint32_t* __restrict__ probe, uint32_t nprobe,
                                                           const uint64_t* __restrict__ sample_ts, const uint32_t* __restrict__ sample_ids,
                                                           uint32_t S, const uint64_t* __restrict__ ws_arr, const uint64_t* __restrict__ we_arr,
                                                           uint64_t ws0, uint64_t we0, int per_query,
                                                           const uint64_t* __restrict__ base_ts, uint64_t n_base,
                                                           uint64_t* __restrict__ id_lo, uint64_t* __restrict__ id_hi,
                                                           const uint32_t* __restrict__ group_tbl, const uint32_t* __restrict__ group_pos,
                                                           const float* __restrict__ group_rows,
                                                           uint32_t n_seeds, uint32_t min_rows, uint32_t* __restrict__ out,
                                                           const uint32_t* __restrict__ group_ids) {
    __shared__ __align__(8) uint32_t slots_all[4][kProbeSlots];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= nq) return;
    const uint32_t q = row;
    uint32_t* slots = slots_all[wave];
    // lane p: the query's p-th nearest centroid
    const uint32_t my_group = (uint32_t)lane < nprobe ? probe[(size_t)q * nprobe + lane] : kInvalidId;
    const int grp = lane >> 3, j = lane & 7;
    const float* qrow = queries + (size_t)q * dim;
    float4 qreg[CPL ? CPL : 1];
    if (CPL > 0 && !LIST) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) qreg[c] = reinterpret_cast<const float4*>(qrow)[c * 8 + j];
    }
    // the window as a run of sample rows and, when asked for, as an id interval of the base: four searches,
    // one per group of 16 lanes
    uint32_t w_lo = 0, w_hi = S;
    {
        const uint64_t w0 = per_query ? ws_arr[q] : ws0, w1 = per_query ? we_arr[q] : we0;
        const int part = lane >> 4;  // 0: sample lo, 1: sample hi, 2: base lo, 3: base hi
        const uint64_t mine = (part & 1) ? w1 : w0;
        const uint32_t r = lower_bound_by16(sample_ts, 0, S, mine, part < 2 && sample_ts != nullptr, lane);
        uint32_t s_lo = 0, s_hi = S;  // before the clamp: each is the lower bound of its own window end
        if (sample_ts != nullptr) {
            s_lo = __shfl(r, 0, 64);
            s_hi = __shfl(r, 16, 64);
            w_lo = s_lo;
            w_hi = s_hi < s_lo ? s_lo : s_hi;
        }
        if (base_ts != nullptr) {
            // base timestamps never decrease with the row id, and the sample rows are base rows in that order:
            // the bound lies between the base rows of the two sample rows around the bound found above
            uint32_t from = 0, to = (uint32_t)n_base;
            if (sample_ts != nullptr) {
                const uint32_t b = part == 2 ? s_lo : s_hi;
                if (b > 0) from = sample_ids[b - 1] + 1u;
                if (b < S) to = sample_ids[b];
            }
            const uint32_t r2 = lower_bound_by16(base_ts, from, to, mine, part >= 2, lane);
            const uint64_t bl = __shfl(r2, 32, 64);
            uint64_t bh = __shfl(r2, 48, 64);
            if (bh < bl) bh = bl;
            if (lane == 0) {
                id_lo[q] = bl;
                id_hi[q] = bh;
            }
        }
    }
    // lane p: the run of group probe[p] inside the window
    uint32_t first = 0, len = 0;
    {
        // group_tbl[c][b] = first member of group c at or after sample row b * width (b = 0..64): the search for
        // a bound only has to look at the members of one stretch of the table
        const uint32_t c = my_group;
        if (c != kInvalidId) {
            const uint32_t width = (S + kGroupStretches - 1) / kGroupStretches;
            const uint32_t* tbl = group_tbl + (size_t)c * (kGroupStretches + 1);
            const uint32_t s_lo = min(w_lo / width, kGroupStretches - 1), s_hi = min(w_hi / width, kGroupStretches - 1);
            uint32_t l0 = tbl[s_lo], h0 = tbl[s_lo + 1], l1 = tbl[s_hi], h1 = tbl[s_hi + 1];
            while (l0 < h0) {
                const uint32_t mid = (l0 + h0) >> 1;
                if (group_pos[mid] < w_lo) l0 = mid + 1; else h0 = mid;
            }
            while (l1 < h1) {
                const uint32_t mid = (l1 + h1) >> 1;
                if (group_pos[mid] < w_hi) l1 = mid + 1; else h1 = mid;
            }
            first = l0;
            len = l1 > l0 ? l1 - l0 : 0;
        }
    }
    auto scan = [&](uint32_t x) {  // inclusive prefix sum over the lanes
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t y = __shfl_up(x, d, 64);
            if (lane >= d) x += y;
        }
        return x;
    };
    {
        const uint32_t before = scan(len) - len;
        if (before >= min_rows) len = 0;  // the walk ended before this group
    }
    if (LIST) {
        // lane p owns the run of the p-th nearest group: the runs are laid end to end and cut at n_seeds
        const uint32_t incl = scan(len), excl = incl - len;
        for (uint32_t i = 0; i < len && excl + i < n_seeds; ++i) out[(size_t)q * n_seeds + excl + i] = group_ids[first + i];
        const uint32_t total = (uint32_t)__shfl(incl, 63, 64);
        if ((uint32_t)lane < n_seeds && (uint32_t)lane >= total) out[(size_t)q * n_seeds + lane] = kInvalidId;
        return;
    }
    uint64_t mykey = kInvalidKey;
    uint32_t rem = len;
    for (;;) {  // kProbeSlots rows at a time
        const uint32_t incl = scan(rem), excl = incl - rem;
        const uint32_t take = excl >= kProbeSlots ? 0u : min(rem, kProbeSlots - excl);
        const uint32_t total = min((uint32_t)__shfl(incl, 63, 64), kProbeSlots);
        if (total == 0) break;
        for (uint32_t i = 0; i < take; ++i) slots[excl + i] = first + (len - rem) + i;
        rem -= take;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        auto offer = [&](uint64_t key) {  // lanes with j == 0 bring a key each
            const uint64_t thr = readlane_u64(mykey, (int)n_seeds - 1);
            uint64_t b = __ballot(j == 0 && key < thr);
            while (b != 0) {  // wave-uniform
                const int bit = (int)__builtin_ctzll(b);
                b &= b - 1;
                const uint64_t x = readlane_u64(key, bit);
                const uint32_t p = (uint32_t)__popcll(__ballot(mykey < x));
                if (p >= n_seeds) continue;
                const uint64_t up = shfl_up_u64(mykey);
                if ((uint32_t)lane == p) mykey = x;
                else if ((uint32_t)lane > p) mykey = up;
            }
        };
        for (uint32_t t0 = 0; t0 < total; t0 += 16) {  // two rows per group of eight lanes in flight
            const uint32_t ta = t0 + grp, tb = ta + 8;
            uint64_t key0 = kInvalidKey, key1 = kInvalidKey;
            if (ta < total) {
                const bool two = tb < total;
                const uint32_t r0 = slots[ta], r1 = two ? slots[tb] : r0;
                float d0 = 0.0f, d1 = 0.0f;
                if (CPL > 0) {
                    const float4* a4 = reinterpret_cast<const float4*>(group_rows + (size_t)r0 * dim);
                    const float4* b4 = reinterpret_cast<const float4*>(group_rows + (size_t)r1 * dim);
                    float4 x[CPL ? CPL : 1], y[CPL ? CPL : 1];
#pragma unroll
                    for (int c = 0; c < CPL; ++c) x[c] = a4[c * 8 + j];
#pragma unroll
                    for (int c = 0; c < CPL; ++c) y[c] = b4[c * 8 + j];
#pragma unroll
                    for (int c = 0; c < CPL; ++c) d0 = fold4<METRIC>(d0, qreg[c], x[c]);
#pragma unroll
                    for (int c = 0; c < CPL; ++c) d1 = fold4<METRIC>(d1, qreg[c], y[c]);
                    d0 = group8_sum(d0);
                    d1 = group8_sum(d1);
                    if (METRIC == kMetricIP) {
                        d0 = -d0;
                        d1 = -d1;
                    }
                } else {
                    d0 = group8_distance<METRIC>(qrow, group_rows + (size_t)r0 * dim, dim, j);
                    d1 = group8_distance<METRIC>(qrow, group_rows + (size_t)r1 * dim, dim, j);
                }
                // ties go by the row's place in the sample, as in the exact selection
                key0 = make_sel_key(d0, group_pos[r0]);
                if (two) key1 = make_sel_key(d1, group_pos[r1]);
            }
            offer(key0);
            if (t0 + 8 < total) offer(key1);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    if ((uint32_t)lane < n_seeds)
        out[(size_t)q * n_seeds + lane] = mykey == kInvalidKey ? kInvalidId : sample_ids[(uint32_t)(mykey & 0xFFFFFFFFull)];
}

}  // namespace
}  // namespace grab

namespace grab {

// range filter with a short seed list: dense distances for the columns a tile of queries can use,
// then one streaming pass per query
static int entry_select_range_dense(grab_entry_layer* L, const float* d_queries, uint32_t M, int metric,
                                    const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                                    uint64_t win_end, int per_query_window, uint32_t n_seeds, uint32_t* d_out_seeds,
                                    float* kernel_ms, hipStream_t st) {
    const uint32_t S = L->S;
    const uint32_t row_tiles = (M + TM - 1) / TM, col_tiles = (S + TN - 1) / TN;
    const uint64_t pitch = (uint64_t)col_tiles * TN;
    const uint32_t grid = (uint32_t)L->num_cu * 2;
    GRAB_REQUIRE(row_tiles <= 128, "at most 16384 queries per pass");
    GRAB_TRY(L->dense.ensure((size_t)M * pitch * sizeof(float)));
    GRAB_TRY(L->lo.ensure((size_t)M * 4));
    GRAB_TRY(L->hi.ensure((size_t)M * 4));
    GRAB_TRY(L->keys.ensure((size_t)M * 8));
    GRAB_TRY(L->perm.ensure((size_t)M * 4));
    GRAB_TRY(L->sched.ensure((size_t)kSchedWords * 4));
    GRAB_TRY(L->qsorted.ensure((size_t)M * L->dim * 4));
    // the window of a query is a run of consecutive sample rows; queries are ordered by the start
    // of their run so that a tile of 128 queries only visits the columns it can use
    if (!(L->fixed_window && L->ordered_for == M)) {
        hipLaunchKernelGGL(window_to_columns_kernel, dim3((M + 255) / 256), dim3(256), 0, st, L->ts.as<uint64_t>(), S, d_win_start,
                           d_win_end, win_start, win_end, per_query_window, M, M, L->lo.as<uint32_t>(), L->hi.as<uint32_t>(),
                           L->keys.as<uint64_t>());
        hipLaunchKernelGGL(bucket_order_kernel, dim3(1), dim3(1024), 0, st, L->lo.as<uint32_t>(), L->hi.as<uint32_t>(), M, S, grid,
                           L->perm.as<uint32_t>(), L->sched.as<uint32_t>());
        if (L->fixed_window)
            hipLaunchKernelGGL(identity_order_kernel, dim3((M + 255) / 256), dim3(256), 0, st, L->perm.as<uint32_t>(), M);
        L->ordered_for = L->fixed_window ? M : 0;
    }
    const uint32_t* perm = L->perm.as<uint32_t>();
    if (metric == kMetricL2) GRAB_TRY(L->qnorm.ensure((size_t)M * 4));
    if (L->fixed_window) {
        // the queries are read where they are; only their norms are needed
        if (metric == kMetricL2)
            hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)(((size_t)M * 8 + 255) / 256)), dim3(256), 0, st, d_queries, M, L->dim,
                               L->qnorm.as<float>());
    } else {
        // the contraction reads the queries in tile order
        hipLaunchKernelGGL(gather_rows_norms_kernel, dim3((M * 8 + 255) / 256), dim3(256), 0, st, d_queries, perm, M, L->dim,
                           L->qsorted.as<float>(), metric == kMetricL2 ? L->qnorm.as<float>() : nullptr);
    }
    GRAB_HIP(hipGetLastError());
    TileArgs t{};
    t.A = L->fixed_window ? d_queries : L->qsorted.as<float>();
    t.B = L->sample.as<float>();
    t.normA = L->qnorm.as<float>();
    t.normB = L->norm.as<float>();
    t.row_perm = nullptr;
    t.dense = L->dense.as<float>();
    t.dense_pitch = pitch;
    t.sched = L->sched.as<uint32_t>();
    t.M = M;
    t.N = S;
    t.dim = L->dim;
    t.kk = n_seeds;
    t.nsplit = 1;
    t.col_tiles = col_tiles;
    t.tiles_per_split = col_tiles;
    t.row_tiles = row_tiles;
    hipEvent_t e0 = nullptr, e1 = nullptr, e2 = nullptr;
    if (kernel_ms) {
        GRAB_HIP(hipEventCreate(&e0));
        GRAB_HIP(hipEventCreate(&e1));
        GRAB_HIP(hipEventCreate(&e2));
        GRAB_HIP(hipEventRecord(e0, st));
    }
    int rc = metric == kMetricIP ? launch_tile_one<kMetricIP, kFilterColRange, true>(t, grid, st)
                                 : launch_tile_one<kMetricL2, kFilterColRange, true>(t, grid, st);
    if (kernel_ms && rc == GRAB_OK && hipEventRecord(e2, st) != hipSuccess) {
        set_error("entry layer: event record failed");
        rc = GRAB_ERR_HIP;
    }
    if (rc == GRAB_OK && d_out_seeds != nullptr) {  // without an output the caller selects from L->dense itself
        if (L->fixed_window && pitch <= 1024 && n_seeds <= 48)
            hipLaunchKernelGGL(select_short_rows_kernel, dim3((M + 3) / 4), dim3(256), 0, st, L->dense.as<float>(), pitch, perm, S, M,
                               L->ids.as<uint32_t>(), n_seeds, d_out_seeds);
        else
            hipLaunchKernelGGL(stream_select_kernel, dim3((M + 3) / 4), dim3(256), 0, st, L->dense.as<float>(), pitch, perm,
                               L->lo.as<uint32_t>(), L->hi.as<uint32_t>(), M, L->ids.as<uint32_t>(), n_seeds, d_out_seeds);
        if (hipGetLastError() != hipSuccess) {
            set_error("entry layer: select kernel launch failed");
            rc = GRAB_ERR_HIP;
        }
    }
    if (kernel_ms && rc == GRAB_OK) {
        float ms = 0.0f, ms_sel = 0.0f;
        hipError_t e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e2);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms_sel, e2, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the entry-layer kernels", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
        *kernel_ms += ms;
        L->last_select_ms += ms_sel;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (e2) (void)hipEventDestroy(e2);
    return rc;
}

int entry_layer_select_async(grab_entry_layer* L, const float* d_queries, size_t nq, int metric, int filter_kind,
                             const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start, uint64_t win_end,
                             int per_query_window, const uint64_t* d_masks, uint32_t n_seeds, uint32_t* d_out_seeds,
                             float* kernel_ms, hipStream_t st) {
    GRAB_REQUIRE(L && d_queries && d_out_seeds, "null pointer");
    GRAB_REQUIRE(n_seeds >= 1 && n_seeds <= 256, "n_seeds must be in [1,256]");
    GRAB_REQUIRE(nq < (1ull << 31), "too many queries");
    if (filter_kind == kFilterRange) {
        GRAB_REQUIRE(L->has_ts, "the entry layer was made without timestamps");
        GRAB_REQUIRE(!per_query_window || (d_win_start && d_win_end), "per-query windows missing");
    } else if (filter_kind == kFilterMask) {
        GRAB_REQUIRE(L->has_labels && d_masks, "the entry layer was made without labels, or masks are missing");
    } else {
        GRAB_REQUIRE(filter_kind == kFilterNone, "bad filter kind");
    }
    if (nq == 0) return GRAB_OK;
    if (kernel_ms) *kernel_ms = 0.0f;
    L->last_select_ms = 0.0f;
    if (filter_kind == kFilterRange && n_seeds <= 64) {
        // bounded scratch: at most 16384 queries per pass
        for (size_t off = 0; off < nq; off += 16384) {
            const uint32_t cur = (uint32_t)std::min<size_t>(16384, nq - off);
            GRAB_TRY(entry_select_range_dense(L, d_queries + off * L->dim, cur, metric, per_query_window ? d_win_start + off : nullptr,
                                              per_query_window ? d_win_end + off : nullptr, win_start, win_end, per_query_window,
                                              n_seeds, d_out_seeds + off * n_seeds, kernel_ms, st));
        }
        return GRAB_OK;
    }
    const uint32_t M = (uint32_t)nq, S = L->S;
    const uint32_t row_tiles = (M + TM - 1) / TM, col_tiles = (S + TN - 1) / TN;
    const uint32_t kk = n_seeds;
    const uint32_t target = (uint32_t)L->num_cu * 2;
    // every work item ends with a selection pass over its 128 rows, so the columns of a row tile are
    // cut into few parts: about one work item per CU
    uint32_t nsplit = std::max(1u, std::min({((uint32_t)L->num_cu + row_tiles - 1) / row_tiles, 1024u / kk, col_tiles, 8u}));
    const uint32_t tiles_per_split = (col_tiles + nsplit - 1) / nsplit;
    if (filter_kind != kFilterRange) nsplit = (col_tiles + tiles_per_split - 1) / tiles_per_split;
    const uint32_t nwork = row_tiles * nsplit, grid = std::min(nwork, target);
    const uint32_t padded = grab_next_power_of_2(std::max(M, 2u));

    GRAB_TRY(L->cand.ensure((size_t)M * nsplit * kk * sizeof(uint64_t)));
    GRAB_TRY(L->tilebuf.ensure((size_t)grid * TM * CAP * sizeof(uint64_t)));
    if (metric == kMetricL2) {
        GRAB_TRY(L->qnorm.ensure((size_t)M * 4));
        hipLaunchKernelGGL(row_norms_kernel, dim3((M * 8 + 255) / 256), dim3(256), 0, st, d_queries, M, L->dim, L->qnorm.as<float>());
    }
    TileArgs t{};
    t.A = d_queries;
    t.B = L->sample.as<float>();
    t.normA = L->qnorm.as<float>();
    t.normB = L->norm.as<float>();
    t.labels = L->labels.as<uint8_t>();
    t.masks = d_masks;
    t.buf = L->tilebuf.as<uint64_t>();
    t.cand_out = L->cand.as<uint64_t>();
    t.M = M;
    t.N = S;
    t.dim = L->dim;
    t.kk = kk;
    t.nsplit = nsplit;
    t.col_tiles = col_tiles;
    t.tiles_per_split = tiles_per_split;
    t.row_tiles = row_tiles;
    int tile_filter = filter_kind;
    if (filter_kind == kFilterRange) {  // long seed lists: threshold selection inside the contraction
        GRAB_TRY(L->lo.ensure((size_t)M * 4));
        GRAB_TRY(L->hi.ensure((size_t)M * 4));
        GRAB_TRY(L->keys.ensure((size_t)padded * 8));
        GRAB_TRY(L->perm.ensure((size_t)M * 4));
        hipLaunchKernelGGL(window_to_columns_kernel, dim3((padded + 255) / 256), dim3(256), 0, st, L->ts.as<uint64_t>(), S,
                           d_win_start, d_win_end, win_start, win_end, per_query_window, M, padded, L->lo.as<uint32_t>(),
                           L->hi.as<uint32_t>(), L->keys.as<uint64_t>());
        if (per_query_window) {
            GRAB_TRY(sort_u64_async(L->keys.as<uint64_t>(), padded, st));
            hipLaunchKernelGGL(keys_to_perm_kernel, dim3((M + 255) / 256), dim3(256), 0, st, L->keys.as<uint64_t>(), M, L->perm.as<uint32_t>());
            t.row_perm = L->perm.as<uint32_t>();
        }
        t.row_lo = L->lo.as<uint32_t>();
        t.row_hi = L->hi.as<uint32_t>();
        tile_filter = kFilterColRange;
    }
    GRAB_HIP(hipGetLastError());

    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (kernel_ms) {
        GRAB_HIP(hipEventCreate(&e0));
        GRAB_HIP(hipEventCreate(&e1));
        GRAB_HIP(hipEventRecord(e0, st));
    }
    int rc = metric == kMetricIP ? launch_tile<kMetricIP>(t, tile_filter, grid, st) : launch_tile<kMetricL2>(t, tile_filter, grid, st);
    if (kernel_ms && rc == GRAB_OK) {
        hipError_t e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(kernel_ms, e0, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the entry-layer kernel", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    GRAB_TRY(rc);
    const uint32_t nc = nsplit * kk, fgrid = (M + 3) / 4;
    if (nc <= 256)
        hipLaunchKernelGGL(finalize_seeds_kernel<4>, dim3(fgrid), dim3(256), 0, st, L->cand.as<uint64_t>(), nc, M, L->ids.as<uint32_t>(), n_seeds, d_out_seeds);
    else
        hipLaunchKernelGGL(finalize_seeds_kernel<16>, dim3(fgrid), dim3(256), 0, st, L->cand.as<uint64_t>(), nc, M, L->ids.as<uint32_t>(), n_seeds, d_out_seeds);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

// nearest centroids per query (the coarse layer's own dense contraction + selection), then the walk over
// their groups
int entry_layer_select_grouped_async(grab_entry_layer* L, const float* d_queries, size_t nq, int metric,
                                     const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                                     uint64_t win_end, int per_query_window, const uint64_t* d_base_ts, size_t num_base,
                                     uint64_t* d_id_lo, uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows, uint32_t n_seeds,
                                     uint32_t* d_out_seeds, float* kernel_ms, hipStream_t st, bool list_only, uint32_t* d_probe) {
    GRAB_REQUIRE(L && d_queries && d_out_seeds, "null pointer");
    GRAB_REQUIRE(d_base_ts == nullptr || (d_id_lo && d_id_hi && num_base > 0 && num_base < (1ull << 31)),
                 "id interval outputs missing, or a base of 2^31 rows or more");
    GRAB_REQUIRE(L->coarse != nullptr, "the entry layer has no groups (grab_entry_layer_build_groups)");
    GRAB_REQUIRE(n_seeds >= 1 && n_seeds <= 64, "n_seeds must be in [1,64]");
    GRAB_REQUIRE(nprobe >= 1 && nprobe <= 64, "nprobe must be in [1,64]");
    GRAB_REQUIRE(nq < (1ull << 31), "too many queries");
    GRAB_REQUIRE(!per_query_window || (d_win_start && d_win_end), "per-query windows missing");
    if (nq == 0) return GRAB_OK;
    if (kernel_ms) *kernel_ms = 0.0f;
    L->last_select_ms = 0.0f;
    L->coarse->last_select_ms = 0.0f;
    const uint32_t M = (uint32_t)nq;
    if (d_probe == nullptr) {
        GRAB_TRY(L->probe.ensure((size_t)M * nprobe * 4));
        d_probe = L->probe.as<uint32_t>();
    }
    if (L->num_groups <= 1024) {
        // the nearest centroids, nearest first, straight from the accumulators of the contraction (entry_probe.hip)
        GRAB_TRY(entry_layer_probe_async(L, d_queries, nq, metric, nprobe, d_probe, kernel_ms, st));
    } else {
        // more centroids than that kernel ranks: dense distances to the centroids, then a selection kernel.  Every
        // centroid carries timestamp 0: the window [0,1) covers them all.
        for (size_t off = 0; off < nq; off += 16384) {
            const uint32_t cur = (uint32_t)std::min<size_t>(16384, nq - off);
            GRAB_TRY(entry_select_range_dense(L->coarse, d_queries + off * L->dim, cur, metric, nullptr, nullptr, 0, 1, 0, nprobe,
                                              d_probe + off * nprobe, kernel_ms, st));
        }
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (kernel_ms) {
        GRAB_HIP(hipEventCreate(&e0));
        GRAB_HIP(hipEventCreate(&e1));
        GRAB_HIP(hipEventRecord(e0, st));
    }
    // listing only, base in timestamp order, its timestamps at hand, at most 16 groups: sixteen lanes a query do
    const bool list16 = list_only && nprobe <= 16 && L->base_in_ts_order && d_base_ts != nullptr && num_base == L->num_base &&
                        L->num_base >= 2;
    if (list16) {
        const int rc16 = entry_layer_list16_async(L, d_probe, nq, d_win_start, d_win_end, win_start, win_end, per_query_window, d_base_ts, d_id_lo,
                                                  d_id_hi, nprobe, min_rows, n_seeds, d_out_seeds, st);
        if (rc16 != GRAB_OK) {
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
            return rc16;
        }
    } else {
#define GRAB_PROBE(CPL, MET) do { if (list_only) GRAB_PROBE_(CPL, MET, true); else GRAB_PROBE_(CPL, MET, false); } while (0)
#define GRAB_PROBE_(CPL, MET, LST)                                                                                              \
    hipLaunchKernelGGL((probe_groups_kernel<CPL, MET, LST>), dim3((M + 3) / 4), dim3(256), 0, st, d_queries, M, L->dim,         \
                       d_probe, nprobe, L->has_ts ? L->ts.as<uint64_t>() : nullptr, L->ids.as<uint32_t>(),                  \
                       L->S, d_win_start,                                                                                    \
                       d_win_end, win_start, win_end, per_query_window, d_base_ts, (uint64_t)num_base, d_id_lo, d_id_hi,     \
                       L->group_tbl.as<uint32_t>(), L->group_pos.as<uint32_t>(), L->group_rows.as<float>(),                 \
                       n_seeds, min_rows, d_out_seeds, L->group_ids.as<uint32_t>())
    if (L->dim == 128) {
        if (metric == kMetricIP) GRAB_PROBE(4, kMetricIP); else GRAB_PROBE(4, kMetricL2);
    } else {
        if (metric == kMetricIP) GRAB_PROBE(0, kMetricIP); else GRAB_PROBE(0, kMetricL2);
    }
#undef GRAB_PROBE
#undef GRAB_PROBE_
    }
    int rc = GRAB_OK;
    if (hipGetLastError() != hipSuccess) {
        set_error("entry layer: group walk launch failed");
        rc = GRAB_ERR_HIP;
    }
    if (kernel_ms && rc == GRAB_OK) {
        float ms = 0.0f;
        hipError_t e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the group walk", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
        L->last_select_ms = L->coarse->last_select_ms + ms;  // centroid selection + group walk
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return rc;
}

}  // namespace grab

// ---- exact top-k over sets of buckets, for bases stored bucket by bucket --------------------------------------
namespace grab {
namespace {

// row f of dst = row src_row[f] of src (zeros where src_row[f] is 0xFFFFFFFF); 8 lanes per row
__global__ void __launch_bounds__(256) gather_query_rows_kernel(const float* __restrict__ src, const uint32_t* __restrict__ src_row,
                                                                uint32_t count, uint32_t dim, float* __restrict__ dst) {
    const uint32_t g = (blockIdx.x * 256 + threadIdx.x) >> 3;
    const int j = threadIdx.x & 7;
    if (g >= count) return;
    const uint32_t r = src_row[g];
    float4* d4 = reinterpret_cast<float4*>(dst + (size_t)g * dim);
    const float4* s4 = reinterpret_cast<const float4*>(src + (size_t)(r == 0xFFFFFFFFu ? 0 : r) * dim);
    for (uint32_t c = j; c < (dim >> 2); c += 8) d4[c] = r == 0xFFFFFFFFu ? make_float4(0.f, 0.f, 0.f, 0.f) : s4[c];
}

// One wave per query: the k best of the query's partial lists (k sorted results each, -1 where a list ran short),
// by (distance, id).  The lists are taken as many at a time as fit one 1024-key sort beside the best so far.
__global__ void __launch_bounds__(256) merge_partial_lists_kernel(const int64_t* __restrict__ part_ids, const float* __restrict__ part_dist,
                                                                  const uint32_t* __restrict__ list_off, const uint32_t* __restrict__ lists,
                                                                  uint32_t nq, uint32_t k, int64_t* __restrict__ out_ids,
                                                                  float* __restrict__ out_dist) {
    __shared__ uint64_t keys_all[4][1024];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t q = blockIdx.x * 4 + wave;
    if (q >= nq) return;
    uint64_t* keys = keys_all[wave];
    const uint32_t first = list_off[q], last = list_off[q + 1];
    const uint32_t per = (1024u - k) / k;  // lists per round
    for (uint32_t g = lane; g < k; g += 64) keys[g] = kInvalidKey;
    for (uint32_t l0 = first; l0 < last || l0 == first; l0 += per) {
        const uint32_t nl = l0 < last ? min(per, last - l0) : 0u;
        for (uint32_t g = lane; g < 1024u - k; g += 64) {
            uint64_t key = kInvalidKey;
            if (g < nl * k) {
                const size_t at = (size_t)lists[l0 + g / k] * k + g % k;
                const int64_t id = part_ids[at];
                if (id >= 0) key = make_sel_key(part_dist[at], (uint32_t)id);
            }
            keys[k + g] = key;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        uint64_t r[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) r[i] = keys[lane * 16 + i];
        wave_bitonic_sort<16>(r);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 16; ++i)
            if ((uint32_t)(lane * 16 + i) < k) keys[lane * 16 + i] = r[i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (nl == 0) break;
    }
    for (uint32_t g = lane; g < k; g += 64) {
        const uint64_t key = keys[g];
        const bool valid = key != kInvalidKey;
        out_ids[(size_t)q * k + g] = valid ? (int64_t)(key & 0xFFFFFFFFull) : -1;
        out_dist[(size_t)q * k + g] = valid ? ord_float((uint32_t)(key >> 32)) : kDistMax;
    }
}

// One wave per query: the query's candidate lists - `splits` lists of kk GEMM-form keys for each of its tile-grid rows,
// each the kk smallest of its slice of columns - become one ascending list of the kk smallest.  outside[q] = the
// smallest last key of a full list: every column that is in no list lies at or beyond it (what the merge itself
// drops shows in the merged list's own last key).
__global__ void __launch_bounds__(256) premerge_lists_kernel(const uint64_t* __restrict__ cand, uint32_t splits, uint32_t kk,
                                                             const uint32_t* __restrict__ list_off, const uint32_t* __restrict__ lists,
                                                             uint32_t nq, uint64_t* __restrict__ merged, float* __restrict__ outside) {
    __shared__ uint64_t keys_all[4][1024];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t q = blockIdx.x * 4 + wave;
    if (q >= nq) return;
    uint64_t* keys = keys_all[wave];
    const uint32_t first = list_off[q], total = (list_off[q + 1] - first) * splits;
    const uint32_t per = (1024u - kk) / kk;  // lists per round (kk <= 512)
    auto list_base = [&](uint32_t li) { return cand + ((size_t)lists[first + li / splits] * splits + li % splits) * kk; };
    for (uint32_t g = lane; g < kk; g += 64) keys[g] = kInvalidKey;
    float out = __builtin_inff();
    for (uint32_t l0 = 0; l0 < total; l0 += per) {
        const uint32_t nl = min(per, total - l0);
        for (uint32_t g = lane; g < 1024u - kk; g += 64) keys[kk + g] = g < nl * kk ? list_base(l0 + g / kk)[g % kk] : kInvalidKey;
        if ((uint32_t)lane < nl) {
            const uint64_t last = list_base(l0 + lane)[kk - 1];
            if (last != kInvalidKey) out = fminf(out, ord_float((uint32_t)(last >> 32)));
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        uint64_t r[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) r[i] = keys[lane * 16 + i];
        wave_bitonic_sort<16>(r);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < 16; ++i)
            if ((uint32_t)(lane * 16 + i) < kk) keys[lane * 16 + i] = r[i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) out = fminf(out, __shfl_xor(out, m, 64));
    for (uint32_t g = lane; g < kk; g += 64) merged[(size_t)q * kk + g] = keys[g];
    if (lane == 0) outside[q] = out;
}

// results of a subset of the queries back to their places
__global__ void __launch_bounds__(256) scatter_results_kernel(const int64_t* __restrict__ ids, const float* __restrict__ dist,
                                                              const uint32_t* __restrict__ rows, uint32_t count, uint32_t k,
                                                              int64_t* __restrict__ out_ids, float* __restrict__ out_dist) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count * k) return;
    const size_t at = (size_t)rows[i / k] * k + i % k;
    out_ids[at] = ids[i];
    out_dist[at] = dist[i];
}

constexpr uint32_t kScanPiece = 128 * TN;  // columns of one piece of a bucket: a work item sweeps at most this many

// What both ways of the bucket scan work on: every (query, bucket of the query) pair is a tile-grid row with the
// bucket's rows as its admissible columns; a long bucket is cut into pieces, a row per piece.  The rows of a piece
// follow each other, padded to whole row tiles (with rows that admit no column): a tile visits its piece's columns only.
struct ScanRows {
    struct Piece {
        uint32_t lo, hi;
    };
    std::vector<Piece> pieces;
    std::vector<uint32_t> piece_row0;                  // first row of each piece
    std::vector<uint32_t> row_query, row_lo, row_hi;   // per tile-grid row
    std::vector<uint32_t> list_off, lists;             // per query: its tile-grid rows
    uint32_t rows = 0;
    double tiles = 0.0;                                // (row tile, column tile) pairs that the sweep visits
    bool one_row_per_query = false;                    // id intervals: row tiles in the order of the intervals' starts
    std::vector<uint32_t> tile_lo, tile_hi;            // ... and per row tile the column tiles [lo, hi) that its rows admit
};

void scan_rows(const uint64_t* h_bucket_offsets, uint32_t num_buckets, const uint64_t* h_masks, size_t num_queries, ScanRows* out) {
    ScanRows& r = *out;
    std::vector<uint32_t> first_piece(num_buckets + 1, 0);
    for (uint32_t b = 0; b < num_buckets; ++b) {
        first_piece[b] = (uint32_t)r.pieces.size();
        for (uint64_t s0 = h_bucket_offsets[b]; s0 < h_bucket_offsets[b + 1]; s0 += kScanPiece)
            r.pieces.push_back({(uint32_t)s0, (uint32_t)std::min<uint64_t>(s0 + kScanPiece, h_bucket_offsets[b + 1])});
    }
    first_piece[num_buckets] = (uint32_t)r.pieces.size();
    std::vector<uint32_t> piece_count(r.pieces.size() + 1, 0);
    r.list_off.assign(num_queries + 1, 0);
    for (size_t q = 0; q < num_queries; ++q) {
        uint32_t n = 0;
        for (uint32_t b = 0; b < num_buckets; ++b) {
            if (!((h_masks[q] >> b) & 1ull)) continue;
            for (uint32_t pc = first_piece[b]; pc < first_piece[b + 1]; ++pc) piece_count[pc + 1]++;
            n += first_piece[b + 1] - first_piece[b];
        }
        r.list_off[q + 1] = r.list_off[q] + n;
    }
    r.piece_row0.assign(r.pieces.size() + 1, 0);
    for (size_t pc = 0; pc < r.pieces.size(); ++pc) r.piece_row0[pc + 1] = r.piece_row0[pc] + (piece_count[pc + 1] + TM - 1) / TM * TM;
    r.rows = r.piece_row0[r.pieces.size()];
    r.row_query.assign(r.rows, 0u);  // padding rows stand for query 0 and admit no column
    r.row_lo.assign(r.rows, 0);
    r.row_hi.assign(r.rows, 0);
    r.lists.resize(r.list_off[num_queries]);
    std::vector<uint32_t> fill(r.piece_row0.begin(), r.piece_row0.end() - 1), at(r.list_off.begin(), r.list_off.end() - 1);
    for (size_t q = 0; q < num_queries; ++q)
        for (uint32_t b = 0; b < num_buckets; ++b) {
            if (!((h_masks[q] >> b) & 1ull)) continue;
            for (uint32_t pc = first_piece[b]; pc < first_piece[b + 1]; ++pc) {
                const uint32_t row = fill[pc]++;
                r.row_query[row] = (uint32_t)q;
                r.row_lo[row] = r.pieces[pc].lo;
                r.row_hi[row] = r.pieces[pc].hi;
                r.lists[at[q]++] = row;
            }
        }
    for (size_t pc = 0; pc < r.pieces.size(); ++pc)
        r.tiles += (double)((r.piece_row0[pc + 1] - r.piece_row0[pc]) / TM) * ((r.pieces[pc].hi + TN - 1) / TN - r.pieces[pc].lo / TN);
}

// Id intervals instead of buckets: a query is one tile-grid row whose admissible columns are its interval.  The queries
// go into the row tiles in the order of their intervals' starts, so that a tile - which sweeps the union of its rows'
// intervals - visits few columns that none of its rows admits.  `which`: the queries meant (numbered 0.. in the result), or
// null for all.  A query with an empty interval gets no row.
void window_rows(const uint64_t* h_lo, const uint64_t* h_hi, const uint32_t* which, size_t count, size_t num_dataset, ScanRows* out) {
    ScanRows& r = *out;
    struct Item {
        uint32_t lo, hi, q;
    };
    std::vector<Item> items;
    items.reserve(count);
    for (size_t i = 0; i < count; ++i) {
        const size_t src = which ? which[i] : i;
        const uint64_t lo = std::min<uint64_t>(h_lo[src], num_dataset), hi = std::min<uint64_t>(h_hi[src], num_dataset);
        if (lo < hi) items.push_back({(uint32_t)lo, (uint32_t)hi, (uint32_t)i});
    }
    {   // by (start, end, query): a counting pass over 4096 stretches of the starts, then the few items of a stretch
        constexpr uint32_t kBins = 4096;
        std::vector<uint32_t> first(kBins + 1, 0);
        auto bin = [&](const Item& it) { return (uint32_t)(((uint64_t)it.lo * kBins) / (num_dataset + 1)); };
        for (const Item& it : items) first[bin(it) + 1]++;
        for (uint32_t b = 0; b < kBins; ++b) first[b + 1] += first[b];
        std::vector<Item> placed(items.size());
        std::vector<uint32_t> at(first.begin(), first.end() - 1);
        for (const Item& it : items) placed[at[bin(it)]++] = it;
        for (uint32_t b = 0; b < kBins; ++b)
            if (first[b + 1] - first[b] > 1)
                std::sort(placed.begin() + first[b], placed.begin() + first[b + 1],
                          [](const Item& a, const Item& b) { return a.lo != b.lo ? a.lo < b.lo : (a.hi != b.hi ? a.hi < b.hi : a.q < b.q); });
        items.swap(placed);
    }
    r.rows = (uint32_t)((items.size() + TM - 1) / TM * TM);
    r.row_query.assign(r.rows, 0u);  // padding rows stand for query 0 and admit no column
    r.row_lo.assign(r.rows, 0);
    r.row_hi.assign(r.rows, 0);
    r.list_off.assign(count + 1, 0);
    for (const Item& it : items) r.list_off[it.q + 1] = 1;
    for (size_t q = 0; q < count; ++q) r.list_off[q + 1] += r.list_off[q];
    r.lists.assign(items.size(), 0u);
    for (size_t row = 0; row < items.size(); ++row) {
        r.row_query[row] = items[row].q;
        r.row_lo[row] = items[row].lo;
        r.row_hi[row] = items[row].hi;
        r.lists[r.list_off[items[row].q]] = (uint32_t)row;
    }
    for (size_t row0 = 0; row0 < items.size(); row0 += TM) {
        uint32_t lo = 0xFFFFFFFFu, hi = 0;
        for (size_t row = row0; row < std::min(items.size(), row0 + TM); ++row) {
            lo = std::min(lo, items[row].lo);
            hi = std::max(hi, items[row].hi);
        }
        r.tiles += (double)((hi + TN - 1) / TN - lo / TN);
        r.tile_lo.push_back(lo / TN);
        r.tile_hi.push_back((hi + TN - 1) / TN);
    }
    r.one_row_per_query = true;
}

// The plain way: every tile-grid row is a problem of its own for exact_topk (the query's row gathered once per
// tile-grid row, candidates re-scored and checked per row), and a query's partial results are merged at the end.
// Takes what the quick way below cannot prove.
int bucket_scan_by_rows(const float* d_dataset, size_t num_dataset, uint32_t dim, const ScanRows& r, const float* d_queries,
                        size_t num_queries, uint32_t k, int metric, int64_t* d_out_indices, float* d_out_dists, hipStream_t st) {
    DeviceScratch d_rq, d_lo, d_hi, d_rows, d_pid, d_pdist, d_loff, d_lists;
    const uint32_t rows = r.rows;
    GRAB_HIP(d_rq.alloc((size_t)rows * 4));
    GRAB_HIP(d_lo.alloc((size_t)rows * 4));
    GRAB_HIP(d_hi.alloc((size_t)rows * 4));
    GRAB_HIP(d_rows.alloc((size_t)rows * dim * 4));
    GRAB_HIP(d_pid.alloc((size_t)rows * k * 8));
    GRAB_HIP(d_pdist.alloc((size_t)rows * k * 4));
    GRAB_HIP(d_loff.alloc(r.list_off.size() * 4));
    GRAB_HIP(d_lists.alloc(std::max<size_t>(r.lists.size(), 1) * 4));
    GRAB_HIP(hipMemcpyAsync(d_rq.ptr, r.row_query.data(), (size_t)rows * 4, hipMemcpyHostToDevice, st));
    GRAB_HIP(hipMemcpyAsync(d_lo.ptr, r.row_lo.data(), (size_t)rows * 4, hipMemcpyHostToDevice, st));
    GRAB_HIP(hipMemcpyAsync(d_hi.ptr, r.row_hi.data(), (size_t)rows * 4, hipMemcpyHostToDevice, st));
    GRAB_HIP(hipMemcpyAsync(d_loff.ptr, r.list_off.data(), r.list_off.size() * 4, hipMemcpyHostToDevice, st));
    if (!r.lists.empty()) GRAB_HIP(hipMemcpyAsync(d_lists.ptr, r.lists.data(), r.lists.size() * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(gather_query_rows_kernel, dim3((uint32_t)(((size_t)rows * 8 + 255) / 256)), dim3(256), 0, st, d_queries,
                       d_rq.as<uint32_t>(), rows, dim, d_rows.as<float>());
    GRAB_HIP(hipGetLastError());
    TopkProblem p{};
    p.A = d_rows.as<float>();
    p.B = d_dataset;
    p.M = rows;
    p.N = num_dataset;
    p.dim = dim;
    p.k = k;
    p.metric = metric;
    p.filter_kind = kFilterColRange;
    p.row_lo = d_lo.as<uint32_t>();
    p.row_hi = d_hi.as<uint32_t>();
    p.out_i64 = d_pid.as<int64_t>();
    p.out_dist = d_pdist.as<float>();
    GRAB_TRY(exact_topk(p, st, nullptr));
    hipLaunchKernelGGL(merge_partial_lists_kernel, dim3((uint32_t)((num_queries + 3) / 4)), dim3(256), 0, st, d_pid.as<int64_t>(),
                       d_pdist.as<float>(), d_loff.as<uint32_t>(), d_lists.as<uint32_t>(), (uint32_t)num_queries, k, d_out_indices,
                       d_out_dists);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));  // the partial lists are freed on return
    return GRAB_OK;
}


// the base rows as bf16 halves, centred on a mean of spaced rows for squared L2 (mean_out receives it), and their norms
int split_base_rows(const float* d_dataset, size_t num_dataset, uint32_t dim, int metric, DeviceScratch* mean_out, uint16_t* d_split,
                    float* d_norm, hipStream_t st) {
    const float* mu = nullptr;
    if (metric == kMetricL2) {
        GRAB_HIP(mean_out->alloc((size_t)dim * 4));
        hipLaunchKernelGGL(spaced_mean_kernel, dim3(dim), dim3(256), 0, st, d_dataset, (uint64_t)num_dataset,
                           (uint32_t)std::min<size_t>(num_dataset, 8192), dim, mean_out->as<float>());
        mu = mean_out->as<float>();
    }
    hipLaunchKernelGGL(split_rows_chunked_kernel, dim3((uint32_t)((num_dataset * 8 + 255) / 256)), dim3(256), 0, st, d_dataset,
                       (uint64_t)num_dataset, dim, mu, d_split, d_norm);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

// What a scan needs of the base rows and can keep between calls: the rows as bf16 halves (centred on `mean` for squared
// L2) or as they are, their squared norms (of the centred rows where centred) and the largest of these.
struct ScanBase {
    bool split = false;
    const uint16_t* rows_split = nullptr;
    const float* norm = nullptr;
    const float* mean = nullptr;      // null: not centred
    const float* max_norm = nullptr;  // one float
};

// The work list of the dense-store contraction for row tiles whose column tiles [lo, hi) are known on the host: items of
// `per` column tiles, priced like bucket_order_kernel prices them (rounds of `grid` concurrent items, each costing its
// tiles plus a start-up of about a third of a tile).
void dense_sched(const uint32_t* tile_lo, const uint32_t* tile_hi, uint32_t row_tiles, uint32_t grid, uint32_t* sched) {
    uint32_t total = 0;
    for (uint32_t t = 0; t < row_tiles; ++t) total += tile_hi[t] - tile_lo[t];
    const uint32_t base = std::max(1u, total / (grid * 8u));
    uint32_t per = base, best = 0xFFFFFFFFu;
    for (uint32_t w = 0; w < 16; ++w) {
        const uint32_t cand = base + w;
        uint32_t n = 0;
        for (uint32_t t = 0; t < row_tiles; ++t) n += (tile_hi[t] - tile_lo[t] + cand - 1) / cand;
        const uint32_t cost = ((n + grid - 1) / grid) * (3 * cand + 1);
        if (cost < best) {
            best = cost;
            per = cand;
        }
    }
    uint32_t acc = 0;
    for (uint32_t t = 0; t < row_tiles; ++t) {
        sched[kSchedOff + t] = acc;
        sched[kSchedLo + t] = tile_lo[t];
        sched[kSchedHi + t] = tile_hi[t];
        acc += (tile_hi[t] - tile_lo[t] + per - 1) / per;
    }
    sched[kSchedOff + row_tiles] = acc;
    sched[kSchedPer] = per;
    sched[kSchedItems] = acc;
}

// What the quick way needs beyond the rows: the rows of a subset of the queries (ascending query numbers), for the plain way.
using SubRows = std::function<void(const std::vector<uint32_t>& which, ScanRows* out)>;

// The quick way.  One contraction over all tile-grid rows, which read their query's row in place; where there are
// fewer row tiles than workgroups a tile's sweep over its columns is cut into `splits` work items.  The lists of a
// query's rows - GEMM-form keys - are merged into one before anything is re-scored: the exact re-scoring and its
// check run once per query, not once per tile-grid row.  Queries that the check cannot prove go the plain way.
int scan_topk(const float* d_dataset, size_t num_dataset, uint32_t dim, const ScanRows& rw, const SubRows& sub_rows,
              const float* d_queries, size_t num_queries, uint32_t k, int metric, int64_t* d_out_indices, float* d_out_dists,
              float* kernel_ms, hipStream_t st, const ScanBase* base = nullptr) {
    const uint32_t rows = rw.rows, nq = (uint32_t)num_queries;
    g_last_flop = g_last_flop_bf16 = 0.0;
    g_last_redone_rows = g_last_exact_rows = 0;
    if (rows == 0) {  // no query admits a row
        std::vector<int64_t> ids(num_queries * (size_t)k, -1);
        std::vector<float> dist(num_queries * (size_t)k, kDistMax);
        GRAB_HIP(hipMemcpyAsync(d_out_indices, ids.data(), ids.size() * 8, hipMemcpyHostToDevice, st));
        GRAB_HIP(hipMemcpyAsync(d_out_dists, dist.data(), dist.size() * 4, hipMemcpyHostToDevice, st));
        GRAB_HIP(hipStreamSynchronize(st));
        return GRAB_OK;
    }
    int dev = 0, num_cu = 0;
    GRAB_HIP(hipGetDevice(&dev));
    GRAB_HIP(hipDeviceGetAttribute(&num_cu, hipDeviceAttributeMultiprocessorCount, dev));
    const uint32_t kk = std::max<uint32_t>(2 * k + 32, 64);  // <= 288
    const uint32_t row_tiles = rows / TM, col_tiles = (uint32_t)((num_dataset + TN - 1) / TN), target = (uint32_t)num_cu * 2;
    // enough work items for every workgroup of the grid, and no more: an item ends with a selection over each of its
    // 128 rows, which costs as much as several tile steps (1M x 768, 10,000 queries: 2 splits 6.9 ms, 5 splits 8.2 ms)
    const uint32_t splits = std::max(1u, std::min({(target + row_tiles - 1) / row_tiles, 8u, 1024u / kk}));
    // a prepared base has paid for its split rows; otherwise splitting a million rows pays from a thousand query rows on
    const bool split = base ? base->split
                            : g_knn_bf16.load(std::memory_order_relaxed) != 0 && dim % KC == 0 && rows >= 1024 && num_dataset >= 4096;
    DeviceScratch d_tab, buf, cand, merged, outside, norm_a, norm_b, split_a, split_b, mean, doubt;
    const uint32_t grid = std::min(row_tiles * splits, target);
    // Id intervals with short candidate lists go the dense way: the contraction writes the distances of the columns
    // that a row tile sweeps, a streaming pass per query keeps the kk smallest of the query's interval.  (The
    // thresholds of the other way start open for every row and tighten over the first hundreds of admitted columns,
    // which is most of a narrow interval: its tiles spend their time appending and compacting.)  In passes of at most
    // 128 row tiles whose distances fit kDenseCap bytes.
    constexpr uint64_t kDenseCap = 4ull << 30;
    struct Pass {
        uint32_t t0, t1;
        uint64_t pitch;
    };
    std::vector<Pass> passes;
    bool dense_way = rw.one_row_per_query && kk <= 64;
    if (dense_way) {
        for (uint32_t t0 = 0; t0 < row_tiles && dense_way;) {
            uint32_t t1 = t0;
            uint64_t width = 0;
            while (t1 < row_tiles && t1 - t0 < 128) {
                const uint64_t w = std::max<uint64_t>(width, rw.tile_hi[t1] - rw.tile_lo[t1]);
                if ((uint64_t)(t1 + 1 - t0) * TM * w * TN * 4 > kDenseCap) break;
                width = w;
                ++t1;
            }
            if (t1 == t0) dense_way = false;  // one row tile's sweep alone is beyond the cap
            passes.push_back({t0, t1, width * TN});
            t0 = t1;
        }
    }
    if (!dense_way) {
        GRAB_HIP(buf.alloc((size_t)grid * TM * CAP * sizeof(uint64_t)));
        GRAB_HIP(cand.alloc((size_t)rows * splits * kk * sizeof(uint64_t)));
    }
    GRAB_HIP(merged.alloc((size_t)nq * kk * sizeof(uint64_t)));
    GRAB_HIP(outside.alloc((size_t)nq * 4));
    GRAB_HIP(norm_a.alloc((size_t)nq * 4));
    if (!base) GRAB_HIP(norm_b.alloc(num_dataset * 4));
    GRAB_HIP(doubt.alloc(((size_t)nq + 3) * 4));  // [0] rows not proven, [1..nq] which, [nq+1] max norm of the base rows
    // the host's tables in one upload: per tile-grid row its query and column range, per query its rows, per pass its work list
    std::vector<uint32_t> tab;
    tab.reserve((size_t)rows * 3 + rw.list_off.size() + rw.lists.size() + passes.size() * kSchedWords + 64);
    auto put = [&](const uint32_t* src, size_t count) {  // every table starts on a 64-byte boundary
        tab.resize((tab.size() + 15) / 16 * 16);
        const size_t at = tab.size();
        tab.insert(tab.end(), src, src + count);
        return at;
    };
    const size_t at_rq = put(rw.row_query.data(), rows), at_lo = put(rw.row_lo.data(), rows), at_hi = put(rw.row_hi.data(), rows);
    const size_t at_loff = put(rw.list_off.data(), rw.list_off.size()), at_lists = put(rw.lists.data(), rw.lists.size());
    size_t at_sched = 0;
    uint64_t dense_bytes = 0;
    if (dense_way) {
        std::vector<uint32_t> sched(passes.size() * (size_t)kSchedWords, 0u);
        for (size_t pi = 0; pi < passes.size(); ++pi) {
            const Pass& ps = passes[pi];
            dense_bytes = std::max<uint64_t>(dense_bytes, (uint64_t)(ps.t1 - ps.t0) * TM * ps.pitch * 4);
            dense_sched(rw.tile_lo.data() + ps.t0, rw.tile_hi.data() + ps.t0, ps.t1 - ps.t0, target, sched.data() + pi * kSchedWords);
        }
        at_sched = put(sched.data(), sched.size());
    }
    GRAB_HIP(d_tab.alloc(tab.size() * 4 + 64));
    GRAB_HIP(hipMemcpyAsync(d_tab.ptr, tab.data(), tab.size() * 4, hipMemcpyHostToDevice, st));
    const uint32_t* d_rq = d_tab.as<uint32_t>() + at_rq;
    const uint32_t* d_lo = d_tab.as<uint32_t>() + at_lo;
    const uint32_t* d_hi = d_tab.as<uint32_t>() + at_hi;
    const uint32_t* d_loff = d_tab.as<uint32_t>() + at_loff;
    const uint32_t* d_lists = d_tab.as<uint32_t>() + at_lists;
    const uint32_t* d_sched_all = d_tab.as<uint32_t>() + at_sched;
    GRAB_HIP(hipMemsetAsync(doubt.ptr, 0, 4, st));
    GRAB_HIP(hipMemsetAsync(doubt.as<uint32_t>() + nq + 1, 0, 8, st));
    TileArgs t{};
    t.A = d_queries;
    t.B = d_dataset;
    const float* d_norm_b = base ? base->norm : norm_b.as<float>();
    const float* d_max_norm_b = base ? base->max_norm : reinterpret_cast<const float*>(doubt.as<uint32_t>() + nq + 1);
    if (split) {
        // rows as bf16 halves (centred on the base's mean for squared L2); their norms serve the distance form and the
        // error bound of the check alike
        GRAB_HIP(split_a.alloc((size_t)nq * dim * 4));
        const float* mu = base ? base->mean : nullptr;
        if (!base) {
            GRAB_HIP(split_b.alloc(num_dataset * dim * 4));
            GRAB_TRY(split_base_rows(d_dataset, num_dataset, dim, metric, &mean, split_b.as<uint16_t>(), norm_b.as<float>(), st));
            mu = mean.as<float>();
        }
        hipLaunchKernelGGL(split_rows_chunked_kernel, dim3((uint32_t)(((size_t)nq * 8 + 255) / 256)), dim3(256), 0, st, d_queries,
                           (uint64_t)nq, dim, mu, split_a.as<uint16_t>(), norm_a.as<float>());
        t.A = split_a.as<float>();
        t.B = base ? reinterpret_cast<const float*>(base->rows_split) : split_b.as<float>();
    } else {
        if (!base)
            hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((num_dataset * 8 + 255) / 256)), dim3(256), 0, st, d_dataset,
                               (uint32_t)num_dataset, dim, norm_b.as<float>());
        hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)(((size_t)nq * 8 + 255) / 256)), dim3(256), 0, st, d_queries, nq, dim,
                           norm_a.as<float>());
    }
    if (!base)
        hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<size_t>((num_dataset + 255) / 256, 512)), dim3(256), 0, st,
                           norm_b.as<float>(), (uint64_t)num_dataset, doubt.as<uint32_t>() + nq + 1);
    GRAB_HIP(hipGetLastError());
    t.normA = norm_a.as<float>();
    t.normB = d_norm_b;
    t.row_perm = d_rq;
    t.row_lo = d_lo;
    t.row_hi = d_hi;
    t.range_by_grid_row = 1;
    t.cand_by_grid_row = 1;
    t.buf = buf.as<uint64_t>();
    t.cand_out = cand.as<uint64_t>();
    t.M = rows;
    t.N = (uint32_t)num_dataset;
    t.dim = dim;
    t.kk = kk;
    t.nsplit = splits;
    t.col_tiles = col_tiles;
    t.tiles_per_split = (col_tiles + splits - 1) / splits;
    t.row_tiles = row_tiles;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (kernel_ms) {
        GRAB_HIP(hipEventCreate(&e0));
        GRAB_HIP(hipEventCreate(&e1));
        GRAB_HIP(hipEventRecord(e0, st));
    }
    int rc = GRAB_OK;
    DeviceScratch dense;
    if (dense_way) {
        if (dense.alloc(dense_bytes) != hipSuccess) {
            set_error("scan: out of device memory for %llu bytes of distances", (unsigned long long)dense_bytes);
            rc = GRAB_ERR_HIP;
        }
        if (rc == GRAB_OK && hipMemsetAsync(merged.ptr, 0xFF, (size_t)nq * kk * sizeof(uint64_t), st) != hipSuccess)  // no row: an empty list
            rc = GRAB_ERR_HIP;
        for (size_t pi = 0; pi < passes.size() && rc == GRAB_OK; ++pi) {
            const Pass& ps = passes[pi];
            TileArgs tp = t;
            tp.row_perm = d_rq + (size_t)ps.t0 * TM;
            tp.row_lo = d_lo + (size_t)ps.t0 * TM;
            tp.row_hi = d_hi + (size_t)ps.t0 * TM;
            tp.M = (ps.t1 - ps.t0) * TM;
            tp.row_tiles = ps.t1 - ps.t0;
            tp.nsplit = 1;
            tp.dense = dense.as<float>();
            tp.dense_pitch = ps.pitch;
            tp.dense_rel = 1;
            tp.sched = d_sched_all + pi * kSchedWords;
            if (metric == kMetricIP) rc = split ? launch_tile_one<kMetricIP, kFilterColRange, true, true>(tp, target, st)
                                                : launch_tile_one<kMetricIP, kFilterColRange, true, false>(tp, target, st);
            else rc = split ? launch_tile_one<kMetricL2, kFilterColRange, true, true>(tp, target, st)
                            : launch_tile_one<kMetricL2, kFilterColRange, true, false>(tp, target, st);
            if (rc != GRAB_OK) break;
            hipLaunchKernelGGL(stream_select_keys_kernel, dim3((tp.M + 3) / 4), dim3(256), 0, st, dense.as<float>(), ps.pitch,
                               tp.row_perm, d_lo + (size_t)ps.t0 * TM, d_hi + (size_t)ps.t0 * TM, tp.sched,
                               tp.M, kk, merged.as<uint64_t>());
            if (hipGetLastError() != hipSuccess) {
                set_error("scan: select kernel launch failed");
                rc = GRAB_ERR_HIP;
            }
        }
    } else {
        rc = metric == kMetricIP ? launch_tile<kMetricIP>(t, kFilterColRange, grid, st, split)
                                 : launch_tile<kMetricL2>(t, kFilterColRange, grid, st, split);
    }
    if (kernel_ms && rc == GRAB_OK) {
        hipError_t e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(kernel_ms, e0, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the contraction kernel", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (rc != GRAB_OK) {
        (void)hipStreamSynchronize(st);  // the host tables and the scratch above go out of scope
        return rc;
    }
    const double flop = rw.tiles * 2.0 * TM * TN * dim;
    if (split) g_last_flop_bf16 = 3.0 * flop;  // three instructions a product
    else g_last_flop = flop;
    if (!dense_way)
        hipLaunchKernelGGL(premerge_lists_kernel, dim3((nq + 3) / 4), dim3(256), 0, st, cand.as<uint64_t>(), splits, kk, d_loff, d_lists, nq,
                           merged.as<uint64_t>(), outside.as<float>());
    RefineArgs r{};
    r.A = d_queries;
    r.B = d_dataset;
    r.cand = merged.as<uint64_t>();
    r.out_i64 = d_out_indices;
    r.out_dist = d_out_dists;
    r.M = nq;
    r.dim = dim;
    r.nc = kk;
    r.k = k;
    r.kk = kk;
    r.normA = norm_a.as<float>();
    r.max_normB = d_max_norm_b;
    r.sorted = 1;
    r.outside_in = dense_way ? nullptr : outside.as<float>();  // the dense way leaves one whole list per query: its last key is the bound
    r.doubt = doubt.as<uint32_t>();
    if (split) {
        r.split_normA = norm_a.as<float>();
        r.split_max_normB = r.max_normB;
        r.split_terms = 3.0f * (float)dim;
    }
    rc = metric == kMetricIP ? launch_refine<kMetricIP>(r, st) : launch_refine<kMetricL2>(r, st);
    uint32_t n_doubt = 0;
    if (rc == GRAB_OK && hipMemcpyAsync(&n_doubt, doubt.ptr, 4, hipMemcpyDeviceToHost, st) != hipSuccess) rc = GRAB_ERR_HIP;
    if (hipStreamSynchronize(st) != hipSuccess && rc == GRAB_OK) rc = GRAB_ERR_HIP;
    if (rc != GRAB_OK) {
        set_error("scan: re-scoring failed");
        return rc;
    }
    g_last_exact_rows = n_doubt;
    if (n_doubt == 0) return GRAB_OK;
    // queries whose merged list proves nothing (distances far below the rounding error of the GEMM form): the plain way
    std::vector<uint32_t> which(n_doubt);
    GRAB_HIP(hipMemcpy(which.data(), doubt.as<uint32_t>() + 1, (size_t)n_doubt * 4, hipMemcpyDeviceToHost));
    std::sort(which.begin(), which.end());
    ScanRows sub;
    sub_rows(which, &sub);
    DeviceScratch d_which, sub_q, sub_ids, sub_dist;
    GRAB_HIP(d_which.alloc((size_t)n_doubt * 4));
    GRAB_HIP(sub_q.alloc((size_t)n_doubt * dim * 4));
    GRAB_HIP(sub_ids.alloc((size_t)n_doubt * k * 8));
    GRAB_HIP(sub_dist.alloc((size_t)n_doubt * k * 4));
    GRAB_HIP(hipMemcpyAsync(d_which.ptr, which.data(), (size_t)n_doubt * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL(gather_query_rows_kernel, dim3((uint32_t)(((size_t)n_doubt * 8 + 255) / 256)), dim3(256), 0, st, d_queries,
                       d_which.as<uint32_t>(), n_doubt, dim, sub_q.as<float>());
    GRAB_HIP(hipGetLastError());
    const double flop_fp32 = g_last_flop, flop_bf16 = g_last_flop_bf16;
    GRAB_TRY(bucket_scan_by_rows(d_dataset, num_dataset, dim, sub, sub_q.as<float>(), n_doubt, k, metric, sub_ids.as<int64_t>(),
                                 sub_dist.as<float>(), st));
    g_last_flop = flop_fp32;  // the figures of the main pass
    g_last_flop_bf16 = flop_bf16;
    g_last_exact_rows = n_doubt;
    hipLaunchKernelGGL(scatter_results_kernel, dim3((n_doubt * k + 255) / 256), dim3(256), 0, st, sub_ids.as<int64_t>(), sub_dist.as<float>(),
                       d_which.as<uint32_t>(), n_doubt, k, d_out_indices, d_out_dists);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

}  // namespace
}  // namespace grab

using namespace grab;

extern "C" {

// k-means over the sample rows (grab_kmeans), then the rows of each group laid out together
int grab_entry_layer_build_groups(grab_entry_layer* L, uint32_t num_groups, uint32_t niter, uint64_t seed) {
    GRAB_REQUIRE(L != nullptr, "null entry layer");
    const uint32_t S = L->S, dim = L->dim;
    GRAB_REQUIRE(num_groups >= 1 && num_groups <= S, "num_groups must be in [1, %u]", S);
    std::vector<float> rows((size_t)S * dim), centroids((size_t)num_groups * dim);
    std::vector<int64_t> assign(S);
    GRAB_HIP(hipMemcpy(rows.data(), L->sample.ptr, rows.size() * 4, hipMemcpyDeviceToHost));
    GRAB_TRY(grab_kmeans(rows.data(), S, dim, num_groups, niter, seed, centroids.data(), assign.data()));
    std::vector<uint32_t> off(num_groups + 1, 0), pos(S);
    for (uint32_t i = 0; i < S; ++i) off[(size_t)assign[i] + 1]++;
    for (uint32_t g = 0; g < num_groups; ++g) off[g + 1] += off[g];
    {
        std::vector<uint32_t> fill(off.begin(), off.end() - 1);
        for (uint32_t i = 0; i < S; ++i) {  // ascending sample position inside a group
            pos[fill[(size_t)assign[i]]++] = i;
        }
    }
    std::vector<uint32_t> tbl((size_t)num_groups * (kGroupStretches + 1));
    {
        const uint32_t width = (S + kGroupStretches - 1) / kGroupStretches;
        for (uint32_t g = 0; g < num_groups; ++g) {
            uint32_t m = off[g];
            for (uint32_t b = 0; b <= kGroupStretches; ++b) {
                while (b < kGroupStretches && m < off[g + 1] && pos[m] < (uint64_t)b * width) ++m;
                tbl[(size_t)g * (kGroupStretches + 1) + b] = b < kGroupStretches ? m : off[g + 1];
            }
        }
    }
    GRAB_TRY(L->group_tbl.ensure(tbl.size() * 4));
    GRAB_TRY(L->group_pos.ensure((size_t)S * 4));
    GRAB_TRY(L->group_rows.ensure((size_t)S * dim * 4));
    GRAB_HIP(hipMemcpy(L->group_tbl.ptr, tbl.data(), tbl.size() * 4, hipMemcpyHostToDevice));
    GRAB_HIP(hipMemcpy(L->group_pos.ptr, pos.data(), (size_t)S * 4, hipMemcpyHostToDevice));
    {
        std::vector<uint32_t> ids(S), gid(S);
        GRAB_HIP(hipMemcpy(ids.data(), L->ids.ptr, (size_t)S * 4, hipMemcpyDeviceToHost));
        for (uint32_t r = 0; r < S; ++r) gid[r] = ids[pos[r]];
        GRAB_TRY(L->group_ids.ensure((size_t)S * 4));
        GRAB_HIP(hipMemcpy(L->group_ids.ptr, gid.data(), (size_t)S * 4, hipMemcpyHostToDevice));
        // the stretch table once more, over stretches of base ids (ids ascend with the sample position when the
        // base is in timestamp order): tbl_id[g][b] = first member of group g whose base id is at least b * stretch
        const uint64_t stretch = (L->num_base + kIdStretches - 1) / kIdStretches;
        std::vector<uint32_t> tid((size_t)num_groups * (kIdStretches + 1));
        for (uint32_t g = 0; g < num_groups; ++g) {
            uint32_t m = off[g];
            for (uint32_t b = 0; b <= kIdStretches; ++b) {
                while (b < kIdStretches && m < off[g + 1] && gid[m] < (uint64_t)b * stretch) ++m;
                tid[(size_t)g * (kIdStretches + 1) + b] = b < kIdStretches ? m : off[g + 1];
            }
        }
        GRAB_TRY(L->group_tbl_id.ensure(tid.size() * 4));
        GRAB_HIP(hipMemcpy(L->group_tbl_id.ptr, tid.data(), tid.size() * 4, hipMemcpyHostToDevice));
    }
    hipLaunchKernelGGL(gather_rows_norms_kernel, dim3((uint32_t)(((size_t)S * 8 + 255) / 256)), dim3(256), 0, 0, L->sample.as<float>(),
                       L->group_pos.as<uint32_t>(), S, dim, L->group_rows.as<float>(), static_cast<float*>(nullptr));
    GRAB_HIP(hipGetLastError());
    // the centroids as a layer of their own: all with timestamp 0
    DeviceScratch d_cent, d_zero;
    GRAB_HIP(d_cent.alloc(centroids.size() * 4));
    GRAB_HIP(d_zero.alloc((size_t)num_groups * 8));
    GRAB_HIP(hipMemcpy(d_cent.ptr, centroids.data(), centroids.size() * 4, hipMemcpyHostToDevice));
    GRAB_HIP(hipMemset(d_zero.ptr, 0, (size_t)num_groups * 8));
    grab_entry_layer_destroy(L->coarse);
    L->coarse = nullptr;
    L->num_groups = 0;
    GRAB_TRY(grab_entry_layer_create(d_cent.as<float>(), num_groups, dim, nullptr, d_zero.as<uint64_t>(), nullptr, num_groups,
                                     &L->coarse));
    GRAB_HIP(hipDeviceSynchronize());
    L->coarse->fixed_window = true;
    L->num_groups = num_groups;
    GRAB_TRY(entry_layer_pad_centroids(L));
    return GRAB_OK;
}

uint32_t grab_entry_layer_num_groups(const grab_entry_layer* L) { return L ? L->num_groups : 0; }

int grab_entry_layer_select_grouped(grab_entry_layer* layer, const float* d_queries, size_t num_queries, int metric,
                                    const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start, uint64_t win_end,
                                    int per_query_window, const uint64_t* d_base_ts, size_t num_base, uint64_t* d_id_lo,
                                    uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows, uint32_t n_seeds,
                                    uint32_t* d_out_seeds, float* kernel_ms, void* stream) {
    return entry_layer_select_grouped_async(layer, d_queries, num_queries, metric, d_win_start, d_win_end, win_start, win_end,
                                            per_query_window, d_base_ts, num_base, d_id_lo, d_id_hi, nprobe, min_rows, n_seeds,
                                            d_out_seeds, kernel_ms, static_cast<hipStream_t>(stream), false, nullptr);
}

int grab_entry_layer_list_grouped(grab_entry_layer* layer, const float* d_queries, size_t num_queries, int metric,
                                  const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start, uint64_t win_end,
                                  int per_query_window, const uint64_t* d_base_ts, size_t num_base, uint64_t* d_id_lo,
                                  uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows, uint32_t max_ids,
                                  uint32_t* d_out_ids, float* kernel_ms, void* stream) {
    return entry_layer_select_grouped_async(layer, d_queries, num_queries, metric, d_win_start, d_win_end, win_start, win_end,
                                            per_query_window, d_base_ts, num_base, d_id_lo, d_id_hi, nprobe, min_rows, max_ids,
                                            d_out_ids, kernel_ms, static_cast<hipStream_t>(stream), true, nullptr);
}

int grab_entry_layer_create(const float* d_dataset, size_t num_dataset, uint32_t dim, const uint32_t* d_ids_by_ts,
                            const uint64_t* d_ts, const uint8_t* d_labels, uint32_t num_samples, grab_entry_layer** out) {
    GRAB_REQUIRE(d_dataset && out, "null pointer");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(num_samples >= 1, "num_samples must be positive");
    auto* L = new grab_entry_layer();
    L->S = (uint32_t)std::min<size_t>(num_samples, num_dataset);
    L->dim = dim;
    L->has_ts = d_ts != nullptr;
    L->has_labels = d_labels != nullptr;
    int dev = 0;
    int rc = GRAB_OK;
    auto fail = [&](int code) {
        grab_entry_layer_destroy(L);
        return code;
    };
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&L->num_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        set_error("cannot query the device (is a GPU present?)");
        return fail(GRAB_ERR_HIP);
    }
    const uint32_t S = L->S;
    if ((rc = L->sample.ensure((size_t)S * dim * 4)) != GRAB_OK) return fail(rc);
    if ((rc = L->norm.ensure((size_t)S * 4)) != GRAB_OK) return fail(rc);
    if ((rc = L->ids.ensure((size_t)S * 4)) != GRAB_OK) return fail(rc);
    if (L->has_ts && (rc = L->ts.ensure((size_t)S * 8)) != GRAB_OK) return fail(rc);
    if (L->has_labels && (rc = L->labels.ensure((size_t)S)) != GRAB_OK) return fail(rc);
    hipLaunchKernelGGL(gather_sample_kernel, dim3((uint32_t)(((size_t)S * 8 + 255) / 256)), dim3(256), 0, 0, d_dataset, dim,
                       (uint64_t)num_dataset, d_ids_by_ts, d_ts, d_labels, S, L->sample.as<float>(), L->ids.as<uint32_t>(),
                       L->has_ts ? L->ts.as<uint64_t>() : nullptr, L->has_labels ? L->labels.as<uint8_t>() : nullptr);
    hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)(((size_t)S * 8 + 255) / 256)), dim3(256), 0, 0, L->sample.as<float>(), S, dim,
                       L->norm.as<float>());
    if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
        set_error("entry layer: sample gather failed");
        return fail(GRAB_ERR_HIP);
    }
    // row order is timestamp order: a window is an interval of row ids, found through pivot levels over the timestamps
    L->num_base = num_dataset;
    if (d_ids_by_ts == nullptr && d_ts != nullptr && (rc = entry_layer_build_pivots(L, d_ts, num_dataset)) != GRAB_OK) return fail(rc);
    *out = L;
    return GRAB_OK;
}

void grab_entry_layer_destroy(grab_entry_layer* L) {
    if (!L) return;
    for (grab::GrowBuf* b : {&L->sample, &L->norm, &L->ids, &L->ts, &L->labels, &L->qnorm, &L->lo, &L->hi, &L->keys, &L->perm,
                             &L->cand, &L->tilebuf, &L->dense, &L->sched, &L->qsorted, &L->group_tbl, &L->group_pos, &L->group_rows,
                             &L->group_ids, &L->group_tbl_id, &L->pivots, &L->cent_pad, &L->probe})
        b->release();
    grab_entry_layer_destroy(L->coarse);
    delete L;
}

uint32_t grab_entry_layer_size(const grab_entry_layer* L) { return L ? L->S : 0; }
float grab_entry_layer_last_select_ms(const grab_entry_layer* L) { return L ? L->last_select_ms : 0.0f; }

int grab_entry_layer_select(grab_entry_layer* layer, const float* d_queries, size_t num_queries, int metric, int filter_kind,
                            const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start, uint64_t win_end,
                            int per_query_window, const uint64_t* d_masks, uint32_t n_seeds, uint32_t* d_out_seeds,
                            float* kernel_ms, void* stream) {
    // stream-ordered: the seeds are consumed by a search on the same stream
    return entry_layer_select_async(layer, d_queries, num_queries, metric, filter_kind, d_win_start, d_win_end, win_start, win_end,
                                    per_query_window, d_masks, n_seeds, d_out_seeds, kernel_ms, static_cast<hipStream_t>(stream));
}

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

int grab_last_knn_stats(double* flop, uint64_t* rows_redone) {
    if (flop) *flop = g_last_flop;
    if (rows_redone) *rows_redone = g_last_redone_rows;
    return GRAB_OK;
}

uint64_t grab_last_knn_exact_rows(void) { return g_last_exact_rows; }

double grab_last_knn_bf16_flop(void) { return g_last_flop_bf16; }

int grab_knn_allow_bf16(int allow) { return g_knn_bf16.exchange(allow != 0 ? 1 : 0, std::memory_order_relaxed); }

int grab_bucket_scan_topk(const float* d_dataset, size_t num_dataset, uint32_t dim, const uint64_t* h_bucket_offsets,
                          uint32_t num_buckets, const float* d_queries, size_t num_queries, uint32_t k, int metric,
                          const uint64_t* h_masks, int64_t* d_out_indices, float* d_out_dists, float* kernel_ms, void* stream) {
    GRAB_REQUIRE(d_dataset && d_queries && h_bucket_offsets && h_masks && d_out_indices && d_out_dists, "null pointer");
    GRAB_REQUIRE(num_buckets >= 1 && num_buckets <= 64, "num_buckets must be in [1,64] (a query's buckets are a 64-bit set)");
    GRAB_REQUIRE(k >= 1 && k <= 128, "k must be in [1,128]");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(metric == kMetricL2 || metric == kMetricIP, "bad metric");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31) && num_queries < (1ull << 31), "bad problem size");
    for (uint32_t b = 0; b < num_buckets; ++b)
        GRAB_REQUIRE(h_bucket_offsets[b] <= h_bucket_offsets[b + 1], "bucket offsets must not decrease");
    GRAB_REQUIRE(h_bucket_offsets[num_buckets] <= num_dataset, "the last bucket ends beyond the dataset");
    if (kernel_ms) *kernel_ms = 0.0f;
    if (num_queries == 0) return GRAB_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    ScanRows rw;
    scan_rows(h_bucket_offsets, num_buckets, h_masks, num_queries, &rw);
    const SubRows sub_rows = [&](const std::vector<uint32_t>& which, ScanRows* out) {
        std::vector<uint64_t> sub_masks(which.size());
        for (size_t i = 0; i < which.size(); ++i) sub_masks[i] = h_masks[which[i]];
        scan_rows(h_bucket_offsets, num_buckets, sub_masks.data(), which.size(), out);
    };
    return scan_topk(d_dataset, num_dataset, dim, rw, sub_rows, d_queries, num_queries, k, metric, d_out_indices, d_out_dists, kernel_ms, st);
}

int grab_window_scan_topk(const float* d_dataset, size_t num_dataset, uint32_t dim, const float* d_queries, size_t num_queries,
                          uint32_t k, int metric, const uint64_t* h_id_lo, const uint64_t* h_id_hi, int64_t* d_out_indices,
                          float* d_out_dists, float* kernel_ms, void* stream) {
    GRAB_REQUIRE(d_dataset && d_queries && h_id_lo && h_id_hi && d_out_indices && d_out_dists, "null pointer");
    GRAB_REQUIRE(k >= 1 && k <= 128, "k must be in [1,128]");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(metric == kMetricL2 || metric == kMetricIP, "bad metric");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31) && num_queries < (1ull << 31), "bad problem size");
    if (kernel_ms) *kernel_ms = 0.0f;
    if (num_queries == 0) return GRAB_OK;
    ScanRows rw;
    window_rows(h_id_lo, h_id_hi, nullptr, num_queries, num_dataset, &rw);
    const SubRows sub_rows = [&](const std::vector<uint32_t>& which, ScanRows* out) {
        window_rows(h_id_lo, h_id_hi, which.data(), which.size(), num_dataset, out);
    };
    return scan_topk(d_dataset, num_dataset, dim, rw, sub_rows, d_queries, num_queries, k, metric, d_out_indices, d_out_dists, kernel_ms,
                     static_cast<hipStream_t>(stream));
}

// A base prepared for the two scans: what a call would otherwise make of the base rows every time, and a block of
// device memory that the calls' scratch is taken from.
struct grab_scan_base {
    const float* d_dataset = nullptr;
    size_t num_dataset = 0;
    uint32_t dim = 0;
    int metric = 0;
    DeviceScratch rows_split, norm, mean, max_norm;
    ScanBase view;
    void* block = nullptr;  // scratch of the calls; grown to what the last call asked for
    size_t block_bytes = 0;
};

int grab_scan_base_create(const float* d_dataset, size_t num_dataset, uint32_t dim, int metric, grab_scan_base** out) {
    GRAB_REQUIRE(d_dataset && out, "null pointer");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(metric == kMetricL2 || metric == kMetricIP, "bad metric");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31), "bad problem size");
    auto* b = new grab_scan_base();
    b->d_dataset = d_dataset;
    b->num_dataset = num_dataset;
    b->dim = dim;
    b->metric = metric;
    auto fail = [&](int rc) {
        grab_scan_base_destroy(b);
        return rc;
    };
    b->view.split = g_knn_bf16.load(std::memory_order_relaxed) != 0 && dim % KC == 0 && num_dataset >= 4096;
    if (b->norm.alloc(num_dataset * 4) != hipSuccess || b->max_norm.alloc(4) != hipSuccess ||
        (b->view.split && b->rows_split.alloc(num_dataset * dim * 4) != hipSuccess)) {
        (void)hipGetLastError();
        set_error("scan base: out of device memory");
        return fail(GRAB_ERR_HIP);
    }
    int rc = GRAB_OK;
    if (b->view.split) {
        rc = split_base_rows(d_dataset, num_dataset, dim, metric, &b->mean, b->rows_split.as<uint16_t>(), b->norm.as<float>(), nullptr);
    } else {
        hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((num_dataset * 8 + 255) / 256)), dim3(256), 0, nullptr, d_dataset,
                           (uint32_t)num_dataset, dim, b->norm.as<float>());
    }
    if (rc != GRAB_OK) return fail(rc);
    if (hipMemsetAsync(b->max_norm.ptr, 0, 4, nullptr) != hipSuccess) return fail(GRAB_ERR_HIP);
    hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<size_t>((num_dataset + 255) / 256, 512)), dim3(256), 0, nullptr,
                       b->norm.as<float>(), (uint64_t)num_dataset, b->max_norm.as<uint32_t>());
    if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
        set_error("scan base: preparing the rows failed");
        return fail(GRAB_ERR_HIP);
    }
    b->view.rows_split = b->rows_split.as<uint16_t>();
    b->view.norm = b->norm.as<float>();
    b->view.mean = b->mean.as<float>();
    b->view.max_norm = b->max_norm.as<float>();
    *out = b;
    return GRAB_OK;
}

void grab_scan_base_destroy(grab_scan_base* b) {
    if (!b) return;
    if (b->block) (void)hipFree(b->block);
    delete b;
}

namespace {
// a scan with the calls' scratch taken from the base's block; the block follows what the call asked for (up to 8 GiB:
// beyond that, and on the first call, scratch is allocated as ever)
int scan_on_base(grab_scan_base* b, const std::function<int()>& run) {
    ScratchArena arena{static_cast<char*>(b->block), b->block_bytes, 0, 0};
    ScratchArena*& slot = scratch_arena();
    ScratchArena* const before = slot;
    slot = &arena;
    const int rc = run();  // returns with the stream drained: nothing of the block is in use any more
    slot = before;
    const size_t want = std::min<size_t>(arena.wanted + arena.wanted / 8 + (1u << 20), 8ull << 30);
    if (arena.wanted > b->block_bytes && want > b->block_bytes) {
        if (b->block) (void)hipFree(b->block);
        b->block = nullptr;
        b->block_bytes = 0;
        if (hipMalloc(&b->block, want) == hipSuccess) b->block_bytes = want;
        else (void)hipGetLastError();  // no block: the next call allocates as this one did
    }
    return rc;
}
}  // namespace

int grab_scan_base_window_topk(grab_scan_base* b, const float* d_queries, size_t num_queries, uint32_t k, const uint64_t* h_id_lo,
                               const uint64_t* h_id_hi, int64_t* d_out_indices, float* d_out_dists, float* kernel_ms, void* stream) {
    GRAB_REQUIRE(b && d_queries && h_id_lo && h_id_hi && d_out_indices && d_out_dists, "null pointer");
    GRAB_REQUIRE(k >= 1 && k <= 128, "k must be in [1,128]");
    GRAB_REQUIRE(num_queries < (1ull << 31), "bad problem size");
    if (kernel_ms) *kernel_ms = 0.0f;
    if (num_queries == 0) return GRAB_OK;
    ScanRows rw;
    window_rows(h_id_lo, h_id_hi, nullptr, num_queries, b->num_dataset, &rw);
    const SubRows sub_rows = [&](const std::vector<uint32_t>& which, ScanRows* out) {
        window_rows(h_id_lo, h_id_hi, which.data(), which.size(), b->num_dataset, out);
    };
    return scan_on_base(b, [&]() {
        return scan_topk(b->d_dataset, b->num_dataset, b->dim, rw, sub_rows, d_queries, num_queries, k, b->metric, d_out_indices,
                         d_out_dists, kernel_ms, static_cast<hipStream_t>(stream), &b->view);
    });
}

int grab_scan_base_bucket_topk(grab_scan_base* b, const uint64_t* h_bucket_offsets, uint32_t num_buckets, const float* d_queries,
                               size_t num_queries, uint32_t k, const uint64_t* h_masks, int64_t* d_out_indices, float* d_out_dists,
                               float* kernel_ms, void* stream) {
    GRAB_REQUIRE(b && d_queries && h_bucket_offsets && h_masks && d_out_indices && d_out_dists, "null pointer");
    GRAB_REQUIRE(num_buckets >= 1 && num_buckets <= 64, "num_buckets must be in [1,64] (a query's buckets are a 64-bit set)");
    GRAB_REQUIRE(k >= 1 && k <= 128, "k must be in [1,128]");
    GRAB_REQUIRE(num_queries < (1ull << 31), "bad problem size");
    for (uint32_t i = 0; i < num_buckets; ++i)
        GRAB_REQUIRE(h_bucket_offsets[i] <= h_bucket_offsets[i + 1], "bucket offsets must not decrease");
    GRAB_REQUIRE(h_bucket_offsets[num_buckets] <= b->num_dataset, "the last bucket ends beyond the dataset");
    if (kernel_ms) *kernel_ms = 0.0f;
    if (num_queries == 0) return GRAB_OK;
    ScanRows rw;
    scan_rows(h_bucket_offsets, num_buckets, h_masks, num_queries, &rw);
    const SubRows sub_rows = [&](const std::vector<uint32_t>& which, ScanRows* out) {
        std::vector<uint64_t> sub_masks(which.size());
        for (size_t i = 0; i < which.size(); ++i) sub_masks[i] = h_masks[which[i]];
        scan_rows(h_bucket_offsets, num_buckets, sub_masks.data(), which.size(), out);
    };
    return scan_on_base(b, [&]() {
        return scan_topk(b->d_dataset, b->num_dataset, b->dim, rw, sub_rows, d_queries, num_queries, k, b->metric, d_out_indices,
                         d_out_dists, kernel_ms, static_cast<hipStream_t>(stream), &b->view);
    });
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
