// The entry-point layer: an evenly spaced sample of the base in timestamp order, the seeds of a batch of range
// searches selected from it with the contraction kernels of topk_gemm.hip (its coarse level's probe kernels are in
// entry_probe.hip).
#include <algorithm>
#include <vector>

#include "common.hpp"
#include "device_sort.hpp"
#include "device_utils.hpp"
#include "entry_layer.hpp"
#include "topk_gemm.hpp"
#include "topk_internal.hpp"

namespace grab {
using namespace dev;

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
            launch_row_norms(d_queries, M, L->dim, L->qnorm.as<float>(), st);
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
    int rc = launch_tile_store(t, metric, grid, st);
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
        launch_row_norms(d_queries, M, L->dim, L->qnorm.as<float>(), st);
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
    int rc = launch_tile_any(t, metric, tile_filter, grid, st);
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
    launch_row_norms(L->sample.as<float>(), S, dim, L->norm.as<float>(), nullptr);
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

}  // extern "C"
