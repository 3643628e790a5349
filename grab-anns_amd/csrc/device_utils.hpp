// Wave-level device building blocks for gfx950 (wave64): ordered keys, the canonical
// 8-lane distance, the open-addressing visited set and a register bitonic sort.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace grab {
namespace dev {

constexpr uint32_t kInvalidId = 0xFFFFFFFFu;
constexpr uint64_t kInvalidKey = ~0ull;
// The reference spells FLT_MAX as 3.40282e38f (src/index/compute_distance.cuh:162); unfilled
// result slots carry exactly that value.
constexpr float kDistMax = 3.40282e38f;

enum { kMetricL2 = 0, kMetricIP = 1 };
// kFilterIdRange: the admissible rows are an interval of ids (search) / of columns (contraction)
enum { kFilterNone = 0, kFilterRange = 1, kFilterMask = 2, kFilterIdRange = 3, kFilterColRange = 3 };
// contraction only, not a filter: the matrix is a row set against itself and only the tiles on and above the
// diagonal are computed; a tile above it also serves the rows behind its columns (topk_gemm.hip)
enum { kFilterSymmetric = 4 };
// search only, chosen by the host for an id-interval filter that comes with a table of places: the interval is tested
// on the row's place in timestamp order (rank_of_id[id], 4 bytes read per test) instead of on the id itself
enum { kFilterRank = 5 };

// ---- ordered keys --------------------------------------------------------------------------
// float -> uint32 that sorts like the float (scores are negative for the inner product)
__device__ __forceinline__ uint32_t ord_bits(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ord_float(uint32_t o) {
    uint32_t u = (o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o;
    return __uint_as_float(u);
}
// Queue entry: ordered distance | node id | expanded flag.  The reference keeps the flag in
// the id's MSB (src/index/search.cu:49,85); in the LSB it cannot reorder two nodes.
__device__ __forceinline__ uint64_t make_key(float d, uint32_t id) {
    return ((uint64_t)ord_bits(d) << 32) | ((uint64_t)id << 1);
}
__device__ __forceinline__ uint32_t key_id(uint64_t k) { return (uint32_t)(k & 0xFFFFFFFFull) >> 1; }
__device__ __forceinline__ float key_dist(uint64_t k) { return ord_float((uint32_t)(k >> 32)); }
// plain (distance,id) key without a flag bit, for top-k selection outside the search
__device__ __forceinline__ uint64_t make_sel_key(float d, uint32_t id) {
    return ((uint64_t)ord_bits(d) << 32) | (uint64_t)id;
}

// ---- cross-lane moves ----------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}
// sum over groups of 8 consecutive lanes, every lane of the group receives
// ((a0+a1)+(a2+a3)) + ((a4+a5)+(a6+a7)); float addition commutes, so all 8 lanes hold the
// same bits
__device__ __forceinline__ float group8_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]: lane ^ 1
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]: lane ^ 2
    v += dpp_f32<0x141>(v);  // row_half_mirror: lane i <-> 7-i of each 8
    return v;
}

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int lane_mask) {
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    lo = __shfl_xor(lo, lane_mask, 64);
    hi = __shfl_xor(hi, lane_mask, 64);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ uint64_t shfl_u64(uint64_t v, int src_lane) {
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    lo = __shfl(lo, src_lane, 64);
    hi = __shfl(hi, src_lane, 64);
    return ((uint64_t)hi << 32) | lo;
}
// value of the lane below (lane 0 keeps its own): DPP wave_shr:1, no LDS crossbar involved
__device__ __forceinline__ uint64_t shfl_up_u64(uint64_t v) {
    int lo = (int)(uint32_t)v, hi = (int)(uint32_t)(v >> 32);
    lo = __builtin_amdgcn_update_dpp(lo, lo, 0x138, 0xF, 0xF, false);
    hi = __builtin_amdgcn_update_dpp(hi, hi, 0x138, 0xF, 0xF, false);
    return ((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo;
}
// value held by one lane, the same lane for the whole wave (v_readlane)
__device__ __forceinline__ uint64_t readlane_u64(uint64_t v, int uniform_lane) {
    const int l = __builtin_amdgcn_readfirstlane(uniform_lane);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, l);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), l);
    return ((uint64_t)hi << 32) | lo;
}

// ---- canonical distance --------------------------------------------------------------------
// A group of 8 lanes scores one row.  Lane j owns the float4 chunks j, j+8, j+16, ... and
// folds them in that order with fused multiply-adds; the 8 partial sums are combined by
// group8_sum.  `q` may point to LDS or to global memory.  Role of calc_l2_dist_*,
// src/index/compute_distance.cuh:14-139 (32 lanes, stride-32 elements, butterfly 16..1).
template <int METRIC>
__device__ __forceinline__ float fold4(float s, const float4 a, const float4 b) {
    if (METRIC == kMetricIP) {
        s = __builtin_fmaf(a.x, b.x, s);
        s = __builtin_fmaf(a.y, b.y, s);
        s = __builtin_fmaf(a.z, b.z, s);
        s = __builtin_fmaf(a.w, b.w, s);
    } else {
        float d;
        d = a.x - b.x; s = __builtin_fmaf(d, d, s);
        d = a.y - b.y; s = __builtin_fmaf(d, d, s);
        d = a.z - b.z; s = __builtin_fmaf(d, d, s);
        d = a.w - b.w; s = __builtin_fmaf(d, d, s);
    }
    return s;
}

// Rows of any length (a multiple of four floats), query in LDS: lane j of a group of eight folds the chunks j, j + 8, ...
// in that order.  Four chunks of each row are requested before the first is used, so that a wave keeps up to
// 8 x 2 x 4 sixteen-byte loads in flight instead of two per lane.
template <int METRIC, bool TWO>
__device__ __forceinline__ void fold_rows_any(const float4* __restrict__ r0, const float4* __restrict__ r1, const float4* q4,
                                              uint32_t j, uint32_t nchunks, float& d0, float& d1) {
    uint32_t c = j;
    for (; c + 24 < nchunks; c += 32) {
        float4 x0[4], x1[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) x0[u] = r0[c + 8 * u];
        if (TWO) {
#pragma unroll
            for (int u = 0; u < 4; ++u) x1[u] = r1[c + 8 * u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float4 qq = q4[c + 8 * u];
            d0 = fold4<METRIC>(d0, qq, x0[u]);
            if (TWO) d1 = fold4<METRIC>(d1, qq, x1[u]);
        }
    }
    for (; c < nchunks; c += 8) {
        const float4 x0 = r0[c], qq = q4[c];
        d0 = fold4<METRIC>(d0, qq, x0);
        if (TWO) d1 = fold4<METRIC>(d1, qq, r1[c]);
    }
}

template <int METRIC>
__device__ __forceinline__ float group8_distance(const float* q, const float* row, uint32_t dim, int j) {
    const float4* q4 = reinterpret_cast<const float4*>(q);
    const float4* r4 = reinterpret_cast<const float4*>(row);
    const uint32_t nchunks = dim >> 2;
    float s = 0.0f;
    for (uint32_t c = j; c < nchunks; c += 8) s = fold4<METRIC>(s, q4[c], r4[c]);
    s = group8_sum(s);
    return METRIC == kMetricIP ? -s : s;
}

// ---- visited set ---------------------------------------------------------------------------
// hashmap::insert, src/index/hashmap.cuh:59-91: slot0 = (k ^ (k >> bitlen)) & mask, linear
// probing, compare-and-swap on an empty slot.  1 = inserted, 0 = already present, -1 = table
// full (the reference reports "full" as "present").  `full`: the caller knows that every slot is
// taken (it counts the successful inserts); the answer is then -1 without a walk over the whole
// table - present or not, the id is not expanded either way.
__device__ __forceinline__ int hash_insert(uint32_t* table, uint32_t bitlen, uint32_t key, bool full = false) {
    if (full) return -1;
    const uint32_t size = 1u << bitlen, mask = size - 1;
    uint32_t index = (key ^ (key >> bitlen)) & mask;
    for (uint32_t i = 0; i < size; ++i) {
        uint32_t cur = __atomic_load_n(&table[index], __ATOMIC_RELAXED);
        if (cur == kInvalidId) cur = atomicCAS(&table[index], kInvalidId, key);
        if (cur == kInvalidId) return 1;
        if (cur == key) return 0;
        index = (index + 1) & mask;
    }
    return -1;
}

// ---- lower bound through a pivot table ------------------------------------------------------
// A workgroup that answers many lower-bound queries on one ascending array first copies every
// step-th element into LDS (kPivots of them, the last element of each stretch), searches those,
// and only then walks the stretch in device memory: half the dependent global loads.
constexpr uint32_t kPivots = 1024;
// all threads of the workgroup call this, then synchronise
__device__ __forceinline__ uint64_t load_pivots(const uint64_t* __restrict__ a, uint64_t n, uint64_t* piv) {
    const uint64_t step = (n + kPivots - 1) / kPivots;
    for (uint32_t i = threadIdx.x; i < kPivots; i += blockDim.x) {
        const uint64_t idx = ((uint64_t)i + 1) * step - 1;
        piv[i] = idx < n ? a[idx] : (n ? a[n - 1] : 0);
    }
    return step;
}
// first index whose element is >= v (n when there is none)
__device__ __forceinline__ uint64_t lower_bound_pivots(const uint64_t* __restrict__ a, uint64_t n, const uint64_t* piv, uint64_t step,
                                                       uint64_t v) {
    uint32_t plo = 0, phi = kPivots;
    while (plo < phi) {
        const uint32_t mid = (plo + phi) >> 1;
        if (piv[mid] < v) plo = mid + 1; else phi = mid;
    }
    uint64_t lo = (uint64_t)plo * step, hi = lo + step;
    if (lo > n) lo = n;
    if (hi > n) hi = n;
    while (lo < hi) {
        const uint64_t mid = (lo + hi) >> 1;
        if (a[mid] < v) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// ---- register bitonic sort -----------------------------------------------------------------
// Sorts 64*NPL unique 64-bit keys held NPL per lane (blocked: element lane*NPL+i) ascending.
// Role of bitonic::warp_sort, src/index/bitonic.cuh:53-111, widened to a 64-lane wave; the
// key carries (distance,id), so equal distances come out by ascending id.
template <int NPL>
__device__ __forceinline__ void wave_bitonic_sort(uint64_t (&k)[NPL]) {
    const int lane = threadIdx.x & 63;
    constexpr int TOTAL = 64 * NPL;
#pragma unroll 1
    for (int size = 2; size <= TOTAL; size <<= 1) {
#pragma unroll 1
        for (int stride = size >> 1; stride >= NPL; stride >>= 1) {
            const int lm = stride / NPL;
            const bool lower = (lane & lm) == 0;
#pragma unroll
            for (int i = 0; i < NPL; ++i) {
                const bool up = (((lane * NPL + i) & size) == 0);
                const uint64_t o = shfl_xor_u64(k[i], lm);
                const bool take_min = (lower == up);
                const uint64_t mn = k[i] < o ? k[i] : o, mx = k[i] < o ? o : k[i];
                k[i] = take_min ? mn : mx;
            }
        }
#pragma unroll
        for (int s = NPL / 2; s > 0; s >>= 1) {
            if (s < size) {
#pragma unroll
                for (int i = 0; i < NPL; ++i) {
                    const int j = i ^ s;
                    if (i < j) {
                        const bool up = (((lane * NPL + i) & size) == 0);
                        const uint64_t a = k[i], b = k[j];
                        const uint64_t mn = a < b ? a : b, mx = a < b ? b : a;
                        k[i] = up ? mn : mx;
                        k[j] = up ? mx : mn;
                    }
                }
            }
        }
    }
}

}  // namespace dev
}  // namespace grab
