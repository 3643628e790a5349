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
#include <type_traits>
#include <vector>

#include "common.hpp"
#include "device_sort.hpp"
#include "device_utils.hpp"
#include "topk_gemm.hpp"
#include "topk_internal.hpp"

namespace grab {
using namespace dev;
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __attribute__((ext_vector_type(8))) __bf16 v8bf16;



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

    __shared__ uint32_t next_item;
    for (uint32_t base = 0; base < nwork; base += gridDim.x) {
        // With a counter the items are handed out in their order to whichever workgroup is free (the two workgroups of
        // a CU do not run at the same pace: with equal shares the launch lasts as long as the slower ones).  Symmetric
        // pass: row tile rt sweeps the column tiles from rt on, so the items shrink with rt - the longest go first.
        uint32_t work = base + blockIdx.x;
        if (a.work_counter != nullptr) {
            __syncthreads();  // the item before is fully drained
            if (tid == 0) next_item = atomicAdd(a.work_counter, 1u);
            __syncthreads();
            work = next_item;
            if (work >= nwork) break;  // workgroup-uniform
            base = 0;  // the loop ends by the counter
        }
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
// Workgroup = 4 waves, one per SIMD, two workgroups a CU; wave w owns rows w*32..+31 of the row tile, and a step of
// the sweep takes 64 columns, half a column tile.  The rows' halves stay in registers for the whole sweep (64 VGPRs),
// the columns (64 x 544 bytes a step) are staged in LDS, the next ones in flight during this step.  Two workgroups of
// four waves and not one of eight: a step is matrix instructions, a barrier, the epilogue's vector work,
// and the waves of one workgroup go through these phases together - with two workgroups a SIMD's two waves belong to
// different ones and one's epilogue runs beside the other's matrix instructions.  The sweep runs from the last column
// tile down to the diagonal, so that workgroups that start together read the same columns at about the same time and
// share them in L2.  Row tiles are handed out through a counter, the longest sweeps first: the two workgroups of a CU
// do not run at the same pace (the waves that arrived first win the issue slots), so equal shares would leave the
// faster ones idle at the end.
constexpr uint32_t kSplitRow = 272;      // bf16 values of a split row: 128 high halves, 128 low halves, 8 of the norm as a column, 8 as a row
constexpr uint32_t kSplitPitch = 560;    // bytes of a column in LDS: 528 of data, 32 so that 16-byte reads of 8 consecutive columns cover all banks
constexpr uint32_t kSplitWaves = 4;
constexpr uint32_t kSplitCols = 64;      // columns of a step: half a column tile
constexpr uint32_t kSplitT = 68;         // row stride of a wave's transposed 32 x 64 block: 16-byte aligned rows, conflict-free b128 reads
constexpr uint32_t kSplitSlot = kSplitCols * kSplitPitch;  // a buffer of columns, which the epilogue's transposed blocks (smaller by 1 KB) take over
static_assert(16 * kSplitPitch >= 32 * kSplitT * 4, "a wave's transposed block fits the place of its 16 columns");
static_assert(kSplitWaves * 16 == kSplitCols && TM == kSplitWaves * 32, "a wave moves 16 of a step's columns and owns 32 rows");
static_assert(kSplitPadRows >= TN, "the rows of zeros behind the split rows cover the last column tile");

struct SplitLds {
    uint8_t b[2][kSplitSlot];
    uint64_t thr[TM];
    uint32_t cnt[TM];
    float cbound[kSplitWaves][64];  // -bound/2 of the wave's columns
    float cbmin[kSplitWaves][16];   // the smallest of them per group of four columns
};

// Sorting a row's buffer needs some 60 registers that the sweep, with the rows' halves in 128 of its 256, does not
// have: as a function of its own it saves and restores what it uses when it runs - once in hundreds of steps -
// instead of the sweep keeping part of the halves in scratch memory and fetching them in every step.
__device__ __attribute__((noinline)) void compact_row_split(SplitLds& s, uint64_t* rowbuf, int r, uint32_t kk, int lane) {
    compact_row(s, rowbuf, r, kk, lane);
}

__global__ void __launch_bounds__(64 * kSplitWaves, 2) sym_split_kernel(const TileArgs a, const uint16_t* __restrict__ rows) {
    extern __shared__ __align__(16) uint8_t tile_smem[];
    SplitLds& s = *reinterpret_cast<SplitLds*>(tile_smem);
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wr = wave, half = lane >> 5, l32 = lane & 31;
    uint64_t* myBuf = a.buf + (size_t)blockIdx.x * TM * CAP;
    const uint32_t nwork = a.row_tiles;

    __shared__ uint32_t next_item;
    for (;;) {
        // row tile rt sweeps the column tiles from rt on, so the items shrink with rt: handed out in that order, the
        // largest first, to whichever workgroup is free (the two workgroups of a CU do not run at the same pace)
        __syncthreads();  // the item before is fully drained
        if (tid == 0) next_item = atomicAdd(a.work_counter, 1u);
        __syncthreads();
        const uint32_t work = next_item;
        if (work >= nwork) break;  // workgroup-uniform
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

        // A step's 64 columns are 64 x 33 pieces of 16 bytes (32 of the halves, one of the norms).  Wave w moves columns
        // 16 w .. + 15, whose place in a buffer is where the wave's own transposed block lies in the epilogue: what a
        // wave overwrites there is its own, so no barrier stands between an epilogue and the next parking.  A lane
        // moves piece lane & 31 of columns 16 w + (lane >> 5) + 2 i, i = 0..7 - addresses that differ by constants -
        // and the first 16 lanes the norms of one column each.  No look at n: the rows are followed by rows of zeros
        // up to a whole tile, and what such a column yields is never kept.
        const uint32_t steps = 2u * (a.col_tiles - rt);
        const uint32_t g_lane = (16u * wave + half) * (kSplitRow * 2u) + 16u * l32, g_norm = (16u * wave + (lane & 15u)) * (kSplitRow * 2u) + 512u;
        const uint32_t l_lane = (16u * wave + half) * kSplitPitch + 16u * l32, l_norm = (16u * wave + (lane & 15u)) * kSplitPitch + 512u;
        const bool ninth = lane < 16u;
        uint4 p0, p1, p2, p3, p4, p5, p6, p7, p8 = make_uint4(0u, 0u, 0u, 0u);
        const uint8_t* rows_b = reinterpret_cast<const uint8_t*>(rows);
        // the pieces travel in two lots: five are fetched at the start of a step, four (the norms among them) at the
        // start of its epilogue; all are parked at the start of the next step, a step before they are read
        constexpr uint32_t kG = 4 * kSplitRow, kL = 2 * kSplitPitch;  // two columns on: bytes in memory, bytes in LDS
        auto ld = [&](const uint8_t* p) { return *reinterpret_cast<const uint4*>(p); };
        auto fetch_early = [&](uint32_t cols) {
            const uint8_t* src = rows_b + (size_t)cols * (kSplitRow * 2u) + g_lane;
            p0 = ld(src); p1 = ld(src + kG); p2 = ld(src + 2 * kG); p3 = ld(src + 3 * kG); p4 = ld(src + 4 * kG);
        };
        auto fetch_late = [&](uint32_t cols) {
            const uint8_t* src = rows_b + (size_t)cols * (kSplitRow * 2u);
            p5 = ld(src + g_lane + 5 * kG); p6 = ld(src + g_lane + 6 * kG); p7 = ld(src + g_lane + 7 * kG);
            if (ninth) p8 = ld(src + g_norm);
        };
        auto park_all = [&](uint32_t buf) {
            uint8_t* dst = &s.b[buf][l_lane];
            *reinterpret_cast<uint4*>(dst) = p0;
            *reinterpret_cast<uint4*>(dst + kL) = p1;
            *reinterpret_cast<uint4*>(dst + 2 * kL) = p2;
            *reinterpret_cast<uint4*>(dst + 3 * kL) = p3;
            *reinterpret_cast<uint4*>(dst + 4 * kL) = p4;
            *reinterpret_cast<uint4*>(dst + 5 * kL) = p5;
            *reinterpret_cast<uint4*>(dst + 6 * kL) = p6;
            *reinterpret_cast<uint4*>(dst + 7 * kL) = p7;
            if (ninth) *reinterpret_cast<uint4*>(&s.b[buf][l_norm]) = p8;
        };
        // a step takes half a column tile: the tiles from the last one down to the diagonal, each its low half first.
        // (Past the end of the sweep the last columns are fetched once more, into the buffer nobody reads.)
        auto tile_of = [&](uint32_t step) { return a.col_tiles - 1u - (min(step, steps - 1u) >> 1); };
        auto cols_of = [&](uint32_t step) { return tile_of(step) * TN + kSplitCols * (min(step, steps - 1u) & 1u); };
        fetch_early(cols_of(0));
        fetch_late(cols_of(0));
        park_all(0);
        fetch_early(cols_of(1));
        fetch_late(cols_of(1));
        // a key for a column's list waits one step for its place: the addition that reserves it is on its way during the
        // matrix instructions of the next step instead of being waited for (most lanes have at most one such key a step)
        bool pend = false;
        uint32_t pend_slot = 0, pend_row = 0;
        uint64_t pend_key = 0;
        __syncthreads();  // first tile and row table visible
        for (uint32_t step = 0; step < steps; ++step) {
            const uint32_t buf = step & 1u;
            const uint32_t ct = tile_of(step), col0 = ct * TN, wc = step & 1u;
            v16f acc[2];  // the wave's two blocks of 32 columns; the first k-step starts them from the constant 0 (no 32 register moves)
            const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            park_all(buf ^ 1u);
            fetch_early(cols_of(step + 2));
            // what the epilogue wants of the wave's columns, on its way during the matrix instructions
            const uint32_t mycol = col0 + wc * 64 + lane;
            const float cbv = a.col_bound[min(mycol, a.N - 1u)];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                v8bf16 bh[2], bl[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint8_t* colp = &s.b[buf][(j * 32 + l32) * kSplitPitch + 32u * ks + 16u * half];
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
                const v8bf16 bn = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(&s.b[buf][(j * 32 + l32) * kSplitPitch + 512u]));
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(anorm, bn, acc[j], 0, 0, 0);
            }
            __syncthreads();  // every wave is done reading these columns: their buffer becomes the transposed blocks
            fetch_late(cols_of(step + 2));

            // ---- epilogue, as in tile_topk_kernel: the wave's 32 x 64 block goes through LDS, and each lane walks half a row ----
            {
                float* T = reinterpret_cast<float*>(s.b[buf] + wave * (16u * kSplitPitch));  // where the wave's own columns lay
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) T[((v & 3) + 4 * half + 8 * (v >> 2)) * kSplitT + j * 32 + l32] = acc[j][v];
                const bool mirror = ct > rt;  // the diagonal tile holds both orders of its pairs itself
                // columns past the end can never pass, nor any column of the diagonal tile
                const float cbl = mirror && mycol < a.N ? -0.5f * cbv : __builtin_inff();
                s.cbound[wave][lane] = cbl;
                {   // the smallest bound of every four columns: neighbours within a quad of lanes
                    const int b0 = __float_as_int(cbl);
                    const float m1 = __builtin_fminf(cbl, __int_as_float(__builtin_amdgcn_update_dpp(b0, b0, 0xB1, 0xF, 0xF, false)));  // lanes 1 0 3 2
                    const int b1 = __float_as_int(m1);
                    const float m2 = __builtin_fminf(m1, __int_as_float(__builtin_amdgcn_update_dpp(b1, b1, 0x4E, 0xF, 0xF, false)));   // lanes 2 3 0 1
                    if ((lane & 3u) == 0u) s.cbmin[wave][lane >> 2] = m2;
                }
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
                // Four columns at a time: nothing passes either test unless the largest of the four reaches the smaller of
                // the row's threshold and the four columns' smallest bound - one comparison; the eight comparisons proper
                // (and the read of the four bounds), and the marks put together lane by lane, only where some lane of the
                // wave gets that far (1.3 of 8 groups in a step at 1M rows).  Eight comparisons into wave-wide masks joined
                // by the scalar unit took half as long again.
                uint32_t hits = 0, chits = 0;
                float lim[8];
                {
                    const float4* cm4 = reinterpret_cast<const float4*>(s.cbmin[wave] + 8u * half);
                    const float4 c0 = cm4[0], c1 = cm4[1];
                    lim[0] = __builtin_fminf(thr_g, c0.x); lim[1] = __builtin_fminf(thr_g, c0.y);
                    lim[2] = __builtin_fminf(thr_g, c0.z); lim[3] = __builtin_fminf(thr_g, c0.w);
                    lim[4] = __builtin_fminf(thr_g, c1.x); lim[5] = __builtin_fminf(thr_g, c1.y);
                    lim[6] = __builtin_fminf(thr_g, c1.z); lim[7] = __builtin_fminf(thr_g, c1.w);
                }
                float4 tv[8];  // all of them requested before the first is looked at
#pragma unroll
                for (uint32_t c4 = 0; c4 < 8; ++c4) tv[c4] = Trow4[c4];
#pragma unroll
                for (uint32_t c4 = 0; c4 < 8; ++c4) {
                    const float4 t = tv[c4];
                    if (__ballot(__builtin_fmaxf(__builtin_fmaxf(t.x, t.y), __builtin_fmaxf(t.z, t.w)) >= lim[c4]) != 0) {
                        const float4 cb = cb4[c4];
                        const bool o0 = t.x >= thr_g, o1 = t.y >= thr_g, o2 = t.z >= thr_g, o3 = t.w >= thr_g;
                        const bool m0 = t.x >= cb.x, m1 = t.y >= cb.y, m2 = t.z >= cb.z, m3 = t.w >= cb.w;
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
            // A row's buffer and counter are its wave's alone (the wave owns all 64 columns of a step), so the look at the
            // counters and the sorts need no barrier - and no wait for this wave's appends unless a buffer is due: such
            // a wait is also one for the pieces under way.
            const uint32_t trig = a.kk <= 64 ? 128u : a.kk <= 128 ? a.kk + 64u : (uint32_t)COMPACT_AT;
            {
                const uint32_t myc = lane < 32u ? s.cnt[wr * 32u + lane] : 0u;
                uint64_t due = __ballot(myc >= trig && myc > a.kk);
                if (due != 0) __threadfence_block();
                while (due != 0) {
                    const int r = (int)(wr * 32u) + (int)__builtin_ctzll(due);
                    due &= due - 1;
                    compact_row_split(s, myBuf + (size_t)r * CAP, r, a.kk, (int)lane);
                }
            }
        }
        if (pend && pend_slot < a.col_cap) a.col_list[(size_t)pend_row * a.col_cap + pend_slot] = pend_key;
        __threadfence_block();
        __syncthreads();
        for (uint32_t r = wr * 32u; r < wr * 32u + 32u; ++r) {  // the wave's own rows
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
    static_assert(sizeof(SplitLds) <= 80 * 1024, "two workgroups per CU");
    GRAB_REQUIRE(a.nsplit == 1 && a.M == a.N && a.dim <= 128 && a.row_tiles == a.col_tiles && a.work_counter, "internal: shape of the bf16 symmetric pass");
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
std::atomic<int> g_knn_bf16{1};  // process-wide: may candidates come from bf16 matrix instructions (grab_knn_allow_bf16)
}  // namespace

KnnStats& knn_stats() {
    static thread_local KnnStats s;
    return s;
}

bool knn_bf16_allowed() { return g_knn_bf16.load(std::memory_order_relaxed) != 0; }

int launch_tile_any(const TileArgs& a, int metric, int filter, uint32_t grid, hipStream_t stream, bool split) {
    return metric == kMetricIP ? launch_tile<kMetricIP>(a, filter, grid, stream, split) : launch_tile<kMetricL2>(a, filter, grid, stream, split);
}

int launch_tile_store(const TileArgs& a, int metric, uint32_t grid, hipStream_t stream, bool split) {
    if (metric == kMetricIP)
        return split ? launch_tile_one<kMetricIP, kFilterColRange, true, true>(a, grid, stream)
                     : launch_tile_one<kMetricIP, kFilterColRange, true, false>(a, grid, stream);
    return split ? launch_tile_one<kMetricL2, kFilterColRange, true, true>(a, grid, stream)
                 : launch_tile_one<kMetricL2, kFilterColRange, true, false>(a, grid, stream);
}

int launch_refine_any(const RefineArgs& a, int metric, hipStream_t stream) {
    return metric == kMetricIP ? launch_refine<kMetricIP>(a, stream) : launch_refine<kMetricL2>(a, stream);
}

void launch_row_norms(const float* x, size_t n, uint32_t dim, float* out, hipStream_t stream) {
    hipLaunchKernelGGL(row_norms_kernel, dim3((uint32_t)((n * 8 + 255) / 256)), dim3(256), 0, stream, x, (uint32_t)n, dim, out);
}

void launch_max_float(const float* x, uint64_t n, uint32_t* out, hipStream_t stream) {
    hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<uint64_t>((n + 255) / 256, 512)), dim3(256), 0, stream, x, n, out);
}

void launch_spaced_mean(const float* data, uint64_t n, uint32_t count, uint32_t dim, float* mean, hipStream_t stream) {
    hipLaunchKernelGGL(spaced_mean_kernel, dim3(dim), dim3(256), 0, stream, data, n, count, dim, mean);
}

void launch_split_rows_chunked(const float* data, uint64_t n, uint32_t dim, const float* mean, uint16_t* out, float* norm,
                               hipStream_t stream) {
    hipLaunchKernelGGL(split_rows_chunked_kernel, dim3((uint32_t)((n * 8 + 255) / 256)), dim3(256), 0, stream, data, n, dim, mean, out, norm);
}

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
    const bool split_ok = knn_bf16_allowed() && p.metric == kMetricL2 && p.dim <= 128;
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
    knn_stats().redone_rows = 0;
    knn_stats().exact_rows = 0;
    knn_stats().flop_bf16 = 0.0;
    knn_stats().flop = tile_flop * (sym ? 0.5 * row_tiles * (row_tiles + 1.0) : (double)row_tiles * col_tiles);

    DeviceScratch buf, cand, normA, normB, doubt;
    constexpr uint32_t kCounters = 16;
    uint32_t counters_used = 0;
    auto next_counter = [&]() -> uint32_t* {  // null once they are used up: that launch deals its items out in equal shares
        return counters_used < kCounters ? doubt.as<uint32_t>() + p.M + 3 + counters_used++ : nullptr;
    };
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
        // [M+2]: max |b|^2 of the centred rows, where the split-bf16 pass runs; then kCounters work counters, one a launch
        GRAB_HIP(doubt.alloc(((size_t)p.M + 3 + kCounters) * 4));
        GRAB_HIP(hipMemsetAsync(doubt.ptr, 0, 4, stream));
        GRAB_HIP(hipMemsetAsync(doubt.as<uint32_t>() + p.M + 1, 0, 8 + 4 * kCounters, stream));
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
    const bool split_tiles = !bf16_bound && knn_bf16_allowed() && p.dim % KC == 0 &&
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
            knn_stats().flop_bf16 = 3.0 * knn_stats().flop;
            knn_stats().flop = 0.0;
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
            b.work_counter = next_counter();
            if (split_tiles) {  // three bf16 instructions a product; nothing of this pass runs on fp32 instructions
                knn_stats().flop = 0.0;
                knn_stats().flop_bf16 = 3.0 * tile_flop * (0.5 * row_tiles * (row_tiles + 1.0) + (double)row_tiles * b.col_tiles);
            } else {
                knn_stats().flop += tile_flop * row_tiles * b.col_tiles;
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
            t.work_counter = next_counter();
            if (bf16_bound) {
                // where the bounds came from the bf16 pipe (squared L2, up to 128 dimensions) the pass runs there too,
                // on the split rows the bounding pass left behind: three instructions a product, each at 16x the rate
                TileArgs ts = t;
                ts.normA = ts.normB = split_norms;
                knn_stats().flop = 0.0;
                const double tile_flop_bf16 = 2.0 * TM * TN * 128;
                knn_stats().flop_bf16 = 3.0 * tile_flop_bf16 * 0.5 * row_tiles * (row_tiles + 1.0) + tile_flop_bf16 * row_tiles * ((n_sample + TN - 1) / TN);
                hipLaunchKernelGGL(max_float_kernel, dim3((uint32_t)std::min<size_t>((p.N + 255) / 256, 512)), dim3(256), 0, stream, split_norms, (uint64_t)p.N,
                                   doubt.as<uint32_t>() + p.M + 2);
                rc = launch_sym_split(ts, split_rows, std::min<uint32_t>(row_tiles, target), stream);
            } else {
                rc = p.metric == kMetricIP ? launch_tile<kMetricIP>(t, kFilterSymmetric, grid, stream, split_tiles)
                                           : launch_tile<kMetricL2>(t, kFilterSymmetric, grid, stream, split_tiles);
            }
        }
    } else {
        t.work_counter = next_counter();
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
            knn_stats().redone_rows = n_redo;
            if (split_tiles) knn_stats().flop_bf16 += 3.0 * tile_flop * f.row_tiles * col_tiles;
            else knn_stats().flop += tile_flop * f.row_tiles * col_tiles;
            const uint32_t per = std::max(2u, 1024u / kk);
            const uint32_t first_groups = (f.nsplit + per - 1) / per;
            GRAB_HIP(redo_part.alloc(((size_t)n_redo * f.nsplit + (size_t)n_redo * first_groups) * kk * sizeof(uint64_t)));
            f.cand_out = redo_part.as<uint64_t>();
            const uint32_t fgrid = std::min(f.row_tiles * f.nsplit, target);
            f.work_counter = next_counter();
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
    knn_stats().exact_rows = n_doubt;
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

int grab_last_knn_stats(double* flop, uint64_t* rows_redone) {
    if (flop) *flop = knn_stats().flop;
    if (rows_redone) *rows_redone = knn_stats().redone_rows;
    return GRAB_OK;
}

uint64_t grab_last_knn_exact_rows(void) { return knn_stats().exact_rows; }

double grab_last_knn_bf16_flop(void) { return knn_stats().flop_bf16; }

int grab_knn_allow_bf16(int allow) { return g_knn_bf16.exchange(allow != 0 ? 1 : 0, std::memory_order_relaxed); }

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
