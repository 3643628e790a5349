// Coarse level of the entry-point layer: which groups of sample rows a query should look at.
//
// centroid_probe_kernel ranks the k-means centroids of the layer for every query: the inner products of 16
// queries with all centroids on the matrix pipe, and the nprobe smallest (distance, centroid) keys of every
// query selected where the products are - in the accumulator registers - so that 64 bytes per query leave the
// kernel instead of a dense row of distances.  The products are formed from bf16 halves of the fp32 operands
// (x = hi + lo, hi = x rounded to bf16, lo = the rest rounded to bf16; q.c ~ q_hi.c_hi + q_lo.c_hi + q_hi.c_lo, sums
// in fp32): three v_mfma_f32_16x16x32_bf16 where eight v_mfma_f32_16x16x4f32 stood, a fifth of the matrix time, at
// a relative error of at most 3 * 2^-16 in a product - what is ranked are centroids thousands of such errors apart.  Same role in the reference: the nearest virtual centroids of
// timestamp::TimeStampIndex (src/timeStampIndex.cu:141-238, FAISS flat search over the k-means centroids).
//
// The pivot levels built here let a wave turn a timestamp window into an interval of base ids with one coalesced
// read per level (search_wave.hip does that at the start of a search that lists its own seeds).
#include <vector>

#include "device_utils.hpp"
#include "entry_layer.hpp"

namespace grab {

using namespace dev;

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((ext_vector_type(8))) __bf16 v8bf16;

constexpr int kProbeWaves = 8;     // waves of a workgroup: each owns an eighth of the centroids
constexpr int kProbeCap = 96;      // columns listed per query before the exact fallback takes over
constexpr int kProbeAStride = 136; // bf16 values per query row in LDS (272 bytes): 16-byte reads of 8 consecutive rows touch all banks once

// x = hi + lo + (an error below 2^-17 |x|), both halves bf16 (round to nearest even; finite input)
__device__ __forceinline__ uint32_t bf16_rne(float x) {
    const uint32_t u = __float_as_uint(x);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ void split_bf16(float x, uint32_t& hi, uint32_t& lo) {
    hi = bf16_rne(x);
    lo = bf16_rne(x - __uint_as_float(hi << 16));
}

// Workgroup = 8 waves, 16*R queries x all centroids; wave w owns the column subtiles w*NS .. w*NS+NS-1 (16 centroids
// each) for all R row subtiles (16 queries each), so a centroid fragment loaded once feeds R matrix instructions:
// the centroids are read once per workgroup, and with R = 3 a batch of 10,000 queries is 209 workgroups - one per
// CU, all in one round - that fetch 82 MB from L2 between them (16-query workgroups fetched 246 MB and waited for it).
// Lane (c = lane % 16, g = lane / 16) holds, for k-step t, the 8 values k = 32t + 8g .. + 7 of row c.  Queries and
// centroids use the same split of k, so every product q[k]*c[k] is formed exactly once; only the order of the sum
// differs from a left-to-right loop.  The queries' halves sit in LDS; the centroids' (stored in the order of the waves' loads, see
// split_rows_kernel) come straight from global memory, the next
// subtile's eight loads in flight during this subtile's matrix instructions.  Accumulator layout of the 16x16
// instructions: register i of lane (c, g) holds row 4g+i, column c.
template <int R, int NS, int METRIC>
__global__ void __launch_bounds__(64 * kProbeWaves, 1)
centroid_probe_kernel(const float* __restrict__ Q, uint32_t nq, uint32_t dim, const uint16_t* __restrict__ Cs, uint32_t dimp,
                      const float* __restrict__ cnorm, uint32_t G, uint32_t nprobe, uint32_t* __restrict__ out) {
    constexpr int ROWS = 16 * R;
    constexpr int RPW = ROWS / kProbeWaves;  // rows a wave selects for (2 * R)
    __shared__ __align__(16) uint16_t s_hi[ROWS][kProbeAStride], s_lo[ROWS][kProbeAStride];
    __shared__ float s_min[ROWS][64];
    __shared__ float s_bound[ROWS];
    __shared__ uint32_t s_cnt[ROWS];
    __shared__ uint64_t s_list[ROWS][kProbeCap];
    __shared__ uint64_t s_red[kProbeWaves][ROWS];
    __shared__ uint32_t s_over;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const uint32_t row0 = blockIdx.x * ROWS;
    const float inf = __builtin_inff();
    if (threadIdx.x == 0) s_over = 0;
    // Workgroups walk their waves' subtiles from different starting points, so that the device does not read the
    // same few KB of centroids everywhere at the same moment: accumulator s of wave w holds subtile w*NS + (s + rot) % NS
    const uint32_t rot = blockIdx.x % (uint32_t)NS;
    auto subtile_of = [&](int s) { const uint32_t r = (uint32_t)s + rot; return (uint32_t)(w * NS) + (r >= (uint32_t)NS ? r - NS : r); };
    auto col_of = [&](int s) { return subtile_of(s) * 16u + (uint32_t)c; };

    v4f acc[R][NS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[r][s] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t kc = 0; kc < dimp; kc += 128) {
        if (kc > 0) __syncthreads();  // the chunk before has been read by every wave
        // ROWS rows x 32 pieces of 4 values, a row's pieces by consecutive lanes; zeros beyond the row's end
        for (uint32_t piece = threadIdx.x; piece < (uint32_t)ROWS * 32u; piece += 64u * kProbeWaves) {
            const uint32_t r = piece >> 5, k = kc + 4u * (piece & 31u);
            float4 x = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (k < dim) x = *reinterpret_cast<const float4*>(Q + (size_t)min(row0 + r, nq - 1u) * dim + k);
            uint32_t h0, h1, h2, h3, l0, l1, l2, l3;
            split_bf16(x.x, h0, l0);
            split_bf16(x.y, h1, l1);
            split_bf16(x.z, h2, l2);
            split_bf16(x.w, h3, l3);
            *reinterpret_cast<uint2*>(&s_hi[r][4u * (piece & 31u)]) = make_uint2(h0 | (h1 << 16), h2 | (h3 << 16));
            *reinterpret_cast<uint2*>(&s_lo[r][4u * (piece & 31u)]) = make_uint2(l0 | (l1 << 16), l2 | (l3 << 16));
        }
        __syncthreads();
        auto load_b = [&](uint4 (&b4)[8], int s) {  // 0..3: the hi halves of the four k-steps, 4..7: the lo halves
            // fragment order in memory: a load of the wave is 1 KB in one piece (eight whole cache lines)
            const uint32_t u = min(subtile_of(s), (G - 1u) >> 4);
            const uint4* cb = reinterpret_cast<const uint4*>(Cs) + ((size_t)u * (dimp >> 7) + (kc >> 7)) * 512u + (uint32_t)lane;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                b4[t] = cb[(2 * t) * 64];
                b4[4 + t] = cb[(2 * t + 1) * 64];
            }
        };
        uint4 bcur[8], bnext[8];
        load_b(bcur, 0);
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            if (s + 1 < NS) load_b(bnext, s + 1);  // in flight while this subtile's matrix instructions run
            if (subtile_of(s) * 16u < G) {  // wave-uniform: subtiles wholly beyond the last centroid are skipped
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const v8bf16 bh = __builtin_bit_cast(v8bf16, bcur[t]), bl = __builtin_bit_cast(v8bf16, bcur[4 + t]);
                    v8bf16 ah[R], al[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        ah[r] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(&s_hi[16 * r + c][32 * t + 8 * g]));
                        al[r] = __builtin_bit_cast(v8bf16, *reinterpret_cast<const uint4*>(&s_lo[16 * r + c][32 * t + 8 * g]));
                    }
                    // the small terms first; consecutive instructions go to different accumulators, so none waits for
                    // the result of the one before
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r][s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[r], bh, acc[r][s], 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r][s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[r], bl, acc[r][s], 0, 0, 0);
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r][s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[r], bh, acc[r][s], 0, 0, 0);
                }
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) bcur[t] = bnext[t];
        }
    }

    // ---- selection: the nprobe smallest (value, column) keys of each of the ROWS rows ----
    // value = |c|^2 - 2 q.c (the query's own norm does not change the order) or -q.c
    float v[R][NS][4];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const uint32_t col = col_of(s);
        const bool valid = col < G;
        const float nb = (METRIC == kMetricL2 && valid) ? cnorm[col] : 0.0f;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) v[r][s][i] = valid ? (METRIC == kMetricL2 ? nb - 2.0f * acc[r][s][i] : -acc[r][s][i]) : inf;
    }
    // every pair of lanes of every wave keeps the smallest of its 2*NS columns per row: 64 minima a row.  The
    // nprobe-th smallest of them bounds the nprobe-th smallest value of the row from above.
    float lmin[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float m = v[r][0][i];
#pragma unroll
            for (int s = 1; s < NS; ++s) m = fminf(m, v[r][s][i]);
            lmin[r][i] = m;
            m = fminf(m, dpp_f32<0xB1>(m));  // the neighbour lane (quad_perm [1,0,3,2])
            if ((c & 1) == 0) s_min[16 * r + 4 * g + i][w * 8 + (c >> 1)] = m;
        }
    __syncthreads();
    {   // wave w: rows w*RPW .. w*RPW+RPW-1, lane = position.  The 64 minima of a row are sorted across the lanes (a
        // bitonic network on plain floats: only the value of the nprobe-th smallest is wanted, so ties need no order),
        // the rows side by side so that the cross-lane moves of one overlap the compares of another.  (A looser bound
        // from four sorts of 16 minima each, which needs no moves through LDS, lists a third more columns and the
        // kernel as a whole then takes longer: the lists are the expensive part, not this sort.)
        float x[RPW];
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) x[rr] = s_min[w * RPW + rr][lane];
#pragma unroll
        for (int k = 2; k <= 64; k <<= 1) {
#pragma unroll
            for (int j = k >> 1; j > 0; j >>= 1) {
                const bool keep_min = ((lane & k) == 0) == ((lane & j) == 0);
#pragma unroll
                for (int rr = 0; rr < RPW; ++rr) {
                    const float y = __shfl_xor(x[rr], j, 64);
                    x[rr] = keep_min ? fminf(x[rr], y) : fmaxf(x[rr], y);
                }
            }
        }
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            // kept finite, so that "at or below the bound" is false for the positions without a column (infinite values)
            const float b = fminf(__shfl(x[rr], (int)nprobe - 1, 64), 3.402823466e+38f);
            if (lane == 0) {
                s_bound[w * RPW + rr] = b;
                s_cnt[w * RPW + rr] = 0;
            }
        }
    }
    __syncthreads();
    // columns at or below the bound go to the row's list, in the order they arrive: the list is sorted afterwards, and
    // whether it overflowed depends on the count alone, so the result does not depend on timing.  A lane counts its
    // hits of a row, reserves that many places with one addition, and writes them; the twelve reservations of a lane
    // are in flight together.
    {
        uint32_t hits[R][4], at[R][4];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float bound = s_bound[16 * r + 4 * g + i];
                uint32_t h = 0;
#pragma unroll
                for (int s = 0; s < NS; ++s) h += v[r][s][i] <= bound ? 1u : 0u;
                hits[r][i] = h;
            }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) at[r][i] = hits[r][i] ? atomicAdd(&s_cnt[16 * r + 4 * g + i], hits[r][i]) : 0u;
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (hits[r][i] == 0) continue;
                const int row = 16 * r + 4 * g + i;
                const float bound = s_bound[row];
                uint32_t pos = at[r][i];
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    if (v[r][s][i] <= bound) {
                        if (pos < (uint32_t)kProbeCap) s_list[row][pos] = make_sel_key(v[r][s][i], col_of(s));
                        ++pos;
                    }
                }
            }
    }
    __syncthreads();
    if (threadIdx.x < (uint32_t)ROWS && s_cnt[threadIdx.x] > (uint32_t)kProbeCap) s_over = 1;  // same value from every writer
    __syncthreads();
    if (s_over == 0) {
        // wave w orders the lists of its RPW rows: all their entries side by side over the lanes, an entry's place the
        // number of keys of its row that are smaller (the keys are distinct)
        uint32_t n_of[RPW], start[RPW + 1];
        start[0] = 0;
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {
            n_of[rr] = s_cnt[w * RPW + rr];
            start[rr + 1] = start[rr] + n_of[rr];
        }
        for (uint32_t e = lane; e < start[RPW]; e += 64) {
            int rr = 0;
#pragma unroll
            for (int t = 1; t < RPW; ++t) rr += e >= start[t] ? 1 : 0;
            uint32_t n = n_of[0], first = 0;
#pragma unroll
            for (int t = 1; t < RPW; ++t) {
                n = rr == t ? n_of[t] : n;
                first = rr == t ? start[t] : first;
            }
            const int row = w * RPW + rr;
            const uint64_t* list = s_list[row];
            const uint64_t key = list[e - first];
            uint32_t rank = 0;
            for (uint32_t y = 0; y < n; y += 4) {  // four reads in flight
                uint64_t k4[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) k4[u] = list[min(y + u, n - 1u)];
#pragma unroll
                for (int u = 0; u < 4; ++u) rank += (y + u < n && k4[u] < key) ? 1u : 0u;
            }
            const uint32_t grow = row0 + (uint32_t)row;
            if (grow < nq && rank < nprobe) out[(size_t)grow * nprobe + rank] = (uint32_t)(key & 0xFFFFFFFFull);
        }
#pragma unroll
        for (int rr = 0; rr < RPW; ++rr) {  // fewer centroids than nprobe: padding
            const uint32_t grow = row0 + (uint32_t)(w * RPW + rr);
            for (uint32_t p = n_of[rr] + lane; grow < nq && p < nprobe; p += 64) out[(size_t)grow * nprobe + p] = kInvalidId;
        }
        return;
    }
    // A row listed more than the lists hold (many equal values, or fewer than nprobe positions with a column):
    // the keys are taken out one by one instead, smallest first, all rows together.  Exact for any input.
    uint64_t last[R][4];
#pragma unroll 1
    for (uint32_t it = 0; it < nprobe; ++it) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint64_t best = kInvalidKey;
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const uint64_t key = v[r][s][i] < inf ? make_sel_key(v[r][s][i], col_of(s)) : kInvalidKey;
                    if ((it == 0 || key > last[r][i]) && key < best) best = key;
                }
#pragma unroll
                for (int m = 1; m < 16; m <<= 1) {
                    const uint64_t o = shfl_xor_u64(best, m);
                    best = o < best ? o : best;
                }
                if (c == 0) s_red[w][16 * r + 4 * g + i] = best;
            }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int lrow = 16 * r + 4 * g + i;
                uint64_t nb = s_red[0][lrow];
#pragma unroll
                for (int ww = 1; ww < kProbeWaves; ++ww) {
                    const uint64_t o = s_red[ww][lrow];
                    nb = o < nb ? o : nb;
                }
                last[r][i] = nb;  // once a row is used up this is the invalid key, which no key exceeds
                const uint32_t row = row0 + (uint32_t)lrow;
                if (w == 0 && c == 0 && row < nq) out[(size_t)row * nprobe + it] = nb == kInvalidKey ? kInvalidId : (uint32_t)(nb & 0xFFFFFFFFull);
            }
        __syncthreads();
    }
}

// rows copied into rows of `dimp` floats, zeros behind the first `dim`
// The rows of src (dim floats each) as bf16 halves in the order in which centroid_probe_kernel's waves load them:
// for every 16 rows, every 128 dimensions, every k-step t of 32 and each half (hi, lo), the 64 lanes' 16 bytes side
// by side - lane c + 16 g holds dimensions 32 t + 8 g .. + 7 of row c.  Zeros beyond dim and beyond the last row.
__global__ void __launch_bounds__(256) split_rows_kernel(const float* __restrict__ src, uint32_t rows, uint32_t dim, uint32_t dimp,
                                                         uint16_t* __restrict__ dst) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const uint32_t rows_p = (rows + 15u) & ~15u;
    if (i >= (uint64_t)rows_p * dimp) return;
    const uint32_t r = (uint32_t)(i / dimp), k = (uint32_t)(i % dimp);
    uint32_t hi = 0, lo = 0;
    if (r < rows && k < dim) split_bf16(src[(size_t)r * dim + k], hi, lo);
    const uint32_t u = r >> 4, c = r & 15u, chunk = k >> 7, t = (k >> 5) & 3u, g = (k >> 3) & 3u, e = k & 7u;
    const size_t at = ((((size_t)u * (dimp >> 7) + chunk) * 4u + t) * 2u * 64u + (c + 16u * g)) * 8u + e;
    dst[at] = (uint16_t)hi;
    dst[at + 64u * 8u] = (uint16_t)lo;
}

// The walk over the groups for bases in timestamp order, sixteen lanes a query (four queries a wave; at most 16
// groups are probed).  Per query: the window becomes the interval of row ids [id_lo, id_hi) through the pivot levels
// - a level is 32 consecutive pivots, two per lane in one 16-byte read, for the start and the end of the window side
// by side, then 32 consecutive timestamps of the base itself; lane p cuts the members of the p-th nearest group that
// lie in the interval out of the group's ascending id list (the stretch table brackets each bound; a stretch
// nearly always holds at most four members, which one round of reads covers); the groups are taken nearest first
// until min_rows members are reached (the group that crosses the mark is taken whole) and their ids are laid end
// to end, at most max_ids of them, 0xFFFFFFFF behind.  Nothing is scored: the search scores its seeds anyway.
__global__ void __launch_bounds__(256) list_groups16_kernel(const uint32_t* __restrict__ groups, uint32_t nq, uint32_t nprobe,
                                                            const uint64_t* __restrict__ ws_arr, const uint64_t* __restrict__ we_arr,
                                                            uint64_t ws0, uint64_t we0, int per_query, const uint64_t* __restrict__ base_ts,
                                                            uint32_t n_base, const uint64_t* __restrict__ piv, EntryPivots pv,
                                                            const uint32_t* __restrict__ tbl_id, uint32_t stretch,
                                                            const uint32_t* __restrict__ ids, uint32_t min_rows, uint32_t max_ids,
                                                            uint32_t* __restrict__ out, uint64_t* __restrict__ id_lo_out,
                                                            uint64_t* __restrict__ id_hi_out) {
    const int lane = threadIdx.x & 63, p = lane & 15, sub = lane >> 4;
    const uint32_t q = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 4u + (uint32_t)sub;
    const bool live = q < nq;
    const uint32_t qq = live ? q : nq - 1u;  // lanes of a missing query keep the others company, they write nothing
    const uint32_t grp = (uint32_t)p < nprobe ? groups[(size_t)qq * nprobe + p] : kInvalidId;
    const uint64_t w0 = per_query ? ws_arr[qq] : ws0, w1 = per_query ? we_arr[qq] : we0;
    auto mine16 = [&](bool x) { return (uint32_t)__popc((uint32_t)(__ballot(x) >> (16 * sub)) & 0xFFFFu); };
    uint32_t blk0 = 0, blk1 = 0;  // block of the next level that holds the start / the end
#pragma unroll
    for (int lev = (int)kPivotMaxLevels - 1; lev >= 0; --lev) {
        if ((uint32_t)lev < pv.levels) {  // uniform
            // a level is stored in whole blocks of 32, padded with the largest timestamp: two pivots a lane, one 16-byte read
            const uint32_t cnt = pv.cnt[lev];
            const uint64_t* level = piv + pv.off[lev];
            // both reads are issued before either is waited for: the index is clamped and what lies beyond the level is
            // replaced afterwards (a read under a condition would be a branch and a wait of its own - the two window ends,
            // and further down the four base timestamps and the eight member ids, one after the other)
            const uint32_t i0 = blk0 * 32u + 2u * p, i1 = blk1 * 32u + 2u * p;
            ulonglong2 a = *reinterpret_cast<const ulonglong2*>(level + min(i0, cnt - 2u));
            ulonglong2 b = *reinterpret_cast<const ulonglong2*>(level + min(i1, cnt - 2u));
            if (i0 >= cnt) a = make_ulonglong2(~0ull, ~0ull);
            if (i1 >= cnt) b = make_ulonglong2(~0ull, ~0ull);
            blk0 = blk0 * 32u + mine16(a.x < w0) + mine16(a.y < w0);
            blk1 = blk1 * 32u + mine16(b.x < w1) + mine16(b.y < w1);
        }
    }
    {
        const uint32_t i0 = blk0 * 32u + 2u * p, i1 = blk1 * 32u + 2u * p;
        const uint64_t tx0 = base_ts[min(i0, n_base - 1u)], tx1 = base_ts[min(i0 + 1u, n_base - 1u)];
        const uint64_t ty0 = base_ts[min(i1, n_base - 1u)], ty1 = base_ts[min(i1 + 1u, n_base - 1u)];
        const bool x0 = (i0 < n_base) & (tx0 < w0), x1 = (i0 + 1u < n_base) & (tx1 < w0);
        const bool y0 = (i1 < n_base) & (ty0 < w1), y1 = (i1 + 1u < n_base) & (ty1 < w1);
        blk0 = min(blk0 * 32u + mine16(x0) + mine16(x1), n_base);
        blk1 = min(blk1 * 32u + mine16(y0) + mine16(y1), n_base);
    }
    const uint32_t id_lo = blk0, id_hi = max(blk1, blk0);
    if (live && p == 0 && id_lo_out != nullptr) {
        id_lo_out[q] = id_lo;
        id_hi_out[q] = id_hi;
    }
    uint32_t first = 0, len = 0;
    {
        const bool act = grp != kInvalidId;
        uint32_t l0 = 0, h0 = 0, l1 = 0, h1 = 0;
        if (act) {
            const uint32_t* tbl = tbl_id + (size_t)grp * (kIdStretches + 1);
            const uint32_t s_lo = min(id_lo / stretch, kIdStretches - 1u), s_hi = min(id_hi / stretch, kIdStretches - 1u);
            l0 = tbl[s_lo], h0 = tbl[s_lo + 1], l1 = tbl[s_hi], h1 = tbl[s_hi + 1];
        }
        if (__ballot(act && (h0 - l0 > 4u || h1 - l1 > 4u)) == 0) {
            uint32_t below0 = 0, below1 = 0;
            if (act) {
                uint32_t m0[4], m1[4];
                const uint32_t last0 = h0 > 0u ? h0 - 1u : 0u, last1 = h1 > 0u ? h1 - 1u : 0u;  // places that exist
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    m0[j] = ids[min(l0 + j, last0)];
                    m1[j] = ids[min(l1 + j, last1)];
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    below0 += (l0 + j < h0) & (m0[j] < id_lo) ? 1u : 0u;
                    below1 += (l1 + j < h1) & (m1[j] < id_hi) ? 1u : 0u;
                }
            }
            l0 += below0;
            l1 += below1;
        } else if (act) {
            while (l0 < h0) {
                const uint32_t mid = (l0 + h0) >> 1;
                if (ids[mid] < id_lo) l0 = mid + 1; else h0 = mid;
            }
            while (l1 < h1) {
                const uint32_t mid = (l1 + h1) >> 1;
                if (ids[mid] < id_hi) l1 = mid + 1; else h1 = mid;
            }
        }
        first = l0;
        len = l1 > l0 ? l1 - l0 : 0;
    }
    auto scan16 = [&](uint32_t x) {  // inclusive prefix sum over the 16 lanes of the query: DPP shifts inside a row
        int v = (int)x;
        v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1
        v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
        v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
        v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
        return (uint32_t)v;
    };
    if (scan16(len) - len >= min_rows) len = 0;  // the walk ended before this group
    const uint32_t incl = scan16(len), excl = incl - len;
    const uint32_t total = min((uint32_t)__shfl((int)incl, 16 * sub + 15, 64), max_ids);
    if (!live) return;
    uint32_t* orow = out + (size_t)q * max_ids;
    // sixteen ids in flight at a time: one at a time, every id of the longest run was a wait for memory of its own
    // (half of the kernel's duration)
    for (uint32_t i0 = 0; i0 < len && excl + i0 < max_ids; i0 += 16) {
        uint32_t v[16];
#pragma unroll
        for (uint32_t u = 0; u < 16; ++u) v[u] = ids[first + min(i0 + u, len - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < 16; ++u) asm volatile("" : "+v"(v[u]));  // all sixteen are read here: none is put off into the branch that stores it
#pragma unroll
        for (uint32_t u = 0; u < 16; ++u)
            if (i0 + u < len && excl + i0 + u < max_ids) orow[excl + i0 + u] = v[u];
    }
    for (uint32_t i = total + (uint32_t)p; i < max_ids; i += 16) orow[i] = kInvalidId;
}

// one level of pivots: the last entry of every block of kPivotFan entries of the level below
__global__ void __launch_bounds__(256) pivot_level_kernel(const uint64_t* __restrict__ src, uint32_t src_cnt, uint64_t* __restrict__ dst,
                                                          uint32_t dst_cnt, uint32_t dst_padded) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= dst_padded) return;
    const uint64_t last = min((uint64_t)(i + 1) * kPivotFan, (uint64_t)src_cnt) - 1;
    dst[i] = i < dst_cnt ? src[last] : ~0ull;
}

// flag = 1 when some timestamp is smaller than the one before it
__global__ void __launch_bounds__(256) ts_order_kernel(const uint64_t* __restrict__ ts, uint64_t n, uint32_t* __restrict__ flag) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i + 1 < n && ts[i + 1] < ts[i]) *flag = 1;  // same value from every writer
}

}  // namespace

int entry_layer_pad_centroids(grab_entry_layer* L) {
    const uint32_t G = L->num_groups, dim = L->dim, dimp = (dim + 127u) / 128u * 128u;
    const uint32_t Gp = (G + 15u) & ~15u;
    GRAB_TRY(L->cent_pad.ensure((size_t)Gp * dimp * 4));
    hipLaunchKernelGGL(split_rows_kernel, dim3((uint32_t)(((uint64_t)Gp * dimp + 255) / 256)), dim3(256), 0, 0, L->coarse->sample.as<float>(),
                       G, dim, dimp, L->cent_pad.as<uint16_t>());
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipDeviceSynchronize());
    return GRAB_OK;
}

int entry_layer_build_pivots(grab_entry_layer* L, const uint64_t* d_base_ts, size_t num_base) {
    L->piv_levels = 0;
    L->num_base = num_base;
    L->base_in_ts_order = false;
    if (d_base_ts == nullptr || num_base == 0) return GRAB_OK;
    DeviceScratch flag;
    GRAB_HIP(flag.alloc(4));
    GRAB_HIP(hipMemset(flag.ptr, 0, 4));
    hipLaunchKernelGGL(ts_order_kernel, dim3((uint32_t)((num_base + 255) / 256)), dim3(256), 0, 0, d_base_ts, (uint64_t)num_base,
                       flag.as<uint32_t>());
    GRAB_HIP(hipGetLastError());
    uint32_t unordered = 0;
    GRAB_HIP(hipMemcpy(&unordered, flag.ptr, 4, hipMemcpyDeviceToHost));
    if (unordered) return GRAB_OK;  // the id-interval services of the layer stay off
    // every level is stored in whole blocks of kPivotFan entries, the last block padded with the largest timestamp
    uint32_t cnt = (uint32_t)num_base, total = 0, levels = 0, real[kPivotMaxLevels] = {};
    while (cnt > kPivotFan) {
        GRAB_REQUIRE(levels < kPivotMaxLevels, "too many rows for the pivot levels");
        cnt = (cnt + kPivotFan - 1) / kPivotFan;
        real[levels] = cnt;
        L->piv_off[levels] = total;
        L->piv_cnt[levels] = (cnt + kPivotFan - 1) / kPivotFan * kPivotFan;
        total += L->piv_cnt[levels];
        ++levels;
    }
    GRAB_TRY(L->pivots.ensure((size_t)std::max(total, 1u) * 8));
    const uint64_t* src = d_base_ts;
    uint32_t src_cnt = (uint32_t)num_base;
    for (uint32_t lev = 0; lev < levels; ++lev) {
        uint64_t* dst = L->pivots.as<uint64_t>() + L->piv_off[lev];
        hipLaunchKernelGGL(pivot_level_kernel, dim3((L->piv_cnt[lev] + 255) / 256), dim3(256), 0, 0, src, src_cnt, dst, real[lev], L->piv_cnt[lev]);
        src = dst;
        src_cnt = real[lev];
    }
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipDeviceSynchronize());
    L->piv_levels = levels;
    L->base_in_ts_order = true;
    return GRAB_OK;
}

int entry_layer_list16_async(grab_entry_layer* L, const uint32_t* d_groups, size_t nq, const uint64_t* d_win_start, const uint64_t* d_win_end,
                             uint64_t win_start, uint64_t win_end, int per_query_window, const uint64_t* d_base_ts, uint64_t* d_id_lo,
                             uint64_t* d_id_hi, uint32_t nprobe, uint32_t min_rows, uint32_t max_ids, uint32_t* d_out_ids, hipStream_t st) {
    EntryPivots pv{};
    pv.levels = L->piv_levels;
    for (uint32_t i = 0; i < kPivotMaxLevels; ++i) {
        pv.off[i] = L->piv_off[i];
        pv.cnt[i] = L->piv_cnt[i];
    }
    const uint32_t stretch = (uint32_t)((L->num_base + kIdStretches - 1) / kIdStretches);
    hipLaunchKernelGGL(list_groups16_kernel, dim3((uint32_t)((nq + 15) / 16)), dim3(256), 0, st, d_groups, (uint32_t)nq, nprobe,
                       d_win_start, d_win_end, win_start, win_end, per_query_window, d_base_ts, (uint32_t)L->num_base,
                       L->pivots.as<uint64_t>(), pv, L->group_tbl_id.as<uint32_t>(), stretch, L->group_ids.as<uint32_t>(), min_rows, max_ids,
                       d_out_ids, d_id_lo, d_id_hi);
    if (hipGetLastError() != hipSuccess) {
        set_error("entry layer: group walk launch failed");
        return GRAB_ERR_HIP;
    }
    return GRAB_OK;
}

int entry_layer_probe_async(grab_entry_layer* L, const float* d_queries, size_t nq, int metric, uint32_t nprobe,
                            uint32_t* d_out_groups, float* kernel_ms, hipStream_t st) {
    GRAB_REQUIRE(L && d_queries && d_out_groups, "null pointer");
    GRAB_REQUIRE(L->coarse != nullptr, "the entry layer has no groups (grab_entry_layer_build_groups)");
    GRAB_REQUIRE(nprobe >= 1 && nprobe <= 64, "nprobe must be in [1,64]");
    GRAB_REQUIRE(metric == kMetricL2 || metric == kMetricIP, "bad metric");
    GRAB_REQUIRE(nq < (1ull << 31), "too many queries");
    const uint32_t G = L->num_groups;
    GRAB_REQUIRE(G <= 1024, "grab_entry_layer_probe ranks at most 1024 centroids (the layer has %u groups)", G);
    if (kernel_ms) *kernel_ms = 0.0f;
    if (nq == 0) return GRAB_OK;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (kernel_ms) {
        hipError_t e = hipEventCreate(&e0);
        if (e == hipSuccess) e = hipEventCreate(&e1);
        if (e == hipSuccess) e = hipEventRecord(e0, st);
        if (e != hipSuccess) {
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
            set_error("HIP error %s while setting up the timing of the centroid ranking", hipGetErrorString(e));
            return GRAB_ERR_HIP;
        }
    }
    // three row subtiles a workgroup (fewest centroid reads) once that still gives every CU a workgroup, else one
    const bool wide = nq > (size_t)16 * (size_t)std::max(L->num_cu, 1);
    const uint32_t rows = wide ? 48u : 16u;
    const dim3 grid((uint32_t)((nq + rows - 1) / rows)), block(64 * kProbeWaves);
    const uint32_t dimp = (L->dim + 127u) / 128u * 128u;
    const uint16_t* cent = L->cent_pad.as<uint16_t>();
    const float* cnorm = L->coarse->norm.as<float>();
#define GRAB_RANK2(RR, NS, MET)                                                                                              \
    hipLaunchKernelGGL((centroid_probe_kernel<RR, NS, MET>), grid, block, 0, st, d_queries, (uint32_t)nq, L->dim, cent, dimp, \
                       cnorm, G, nprobe, d_out_groups)
#define GRAB_RANK(NS)                                                                      \
    do {                                                                                   \
        if (metric == kMetricIP) {                                                         \
            if (wide) GRAB_RANK2(3, NS, kMetricIP); else GRAB_RANK2(1, NS, kMetricIP);     \
        } else {                                                                           \
            if (wide) GRAB_RANK2(3, NS, kMetricL2); else GRAB_RANK2(1, NS, kMetricL2);     \
        }                                                                                  \
    } while (0)
    if (G <= 256) GRAB_RANK(2);
    else if (G <= 512) GRAB_RANK(4);
    else if (G <= 768) GRAB_RANK(6);
    else GRAB_RANK(8);
#undef GRAB_RANK
#undef GRAB_RANK2
    int rc = GRAB_OK;
    if (hipGetLastError() != hipSuccess) {
        set_error("entry layer: centroid ranking launch failed");
        rc = GRAB_ERR_HIP;
    }
    if (kernel_ms && rc == GRAB_OK) {
        hipError_t e = hipEventRecord(e1, st);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(kernel_ms, e0, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the centroid ranking", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return rc;
}

}  // namespace grab

extern "C" {

int grab_entry_layer_probe(grab_entry_layer* layer, const float* d_queries, size_t num_queries, int metric, uint32_t nprobe,
                           uint32_t* d_out_groups, float* kernel_ms, void* stream) {
    return grab::entry_layer_probe_async(layer, d_queries, num_queries, metric, nprobe, d_out_groups, kernel_ms,
                                         static_cast<hipStream_t>(stream));
}

int grab_entry_layer_groups(const grab_entry_layer* layer, uint32_t* h_offsets, uint32_t* h_member_ids) {
    GRAB_REQUIRE(layer && h_offsets && h_member_ids, "null pointer");
    GRAB_REQUIRE(layer->coarse != nullptr, "the entry layer has no groups (grab_entry_layer_build_groups)");
    const uint32_t G = layer->num_groups;
    std::vector<uint32_t> tbl((size_t)G * (grab::kIdStretches + 1));
    GRAB_HIP(hipMemcpy(tbl.data(), layer->group_tbl_id.ptr, tbl.size() * 4, hipMemcpyDeviceToHost));
    for (uint32_t g = 0; g < G; ++g) h_offsets[g] = tbl[(size_t)g * (grab::kIdStretches + 1)];
    h_offsets[G] = layer->S;
    GRAB_HIP(hipMemcpy(h_member_ids, layer->group_ids.ptr, (size_t)layer->S * 4, hipMemcpyDeviceToHost));
    return GRAB_OK;
}

int grab_entry_layer_centroids(const grab_entry_layer* layer, float* d_out) {
    GRAB_REQUIRE(layer && d_out, "null pointer");
    GRAB_REQUIRE(layer->coarse != nullptr, "the entry layer has no groups (grab_entry_layer_build_groups)");
    GRAB_HIP(hipMemcpy(d_out, layer->coarse->sample.ptr, (size_t)layer->num_groups * layer->dim * 4, hipMemcpyDeviceToDevice));
    return GRAB_OK;
}

}  // extern "C"
