// Beam search over the CAGRA graph, one workgroup per query: 256 threads (4 waves), or 1024 threads when the batch
// is so small (<= 256 queries) that 256-thread workgroups would leave most of the device's SIMDs without a wave.
//
// Restates the loop of the reference's search_kernel / search_kernel_bucket /
// search_kernel_range (src/index/search.cu:149-370, :375-586, :589-798) with the expansion
// steps of src/index/compute_distance.cuh:204-269,274-380,386-505,512-614, re-shaped for a
// 64-lane wave and 160 KB of LDS:
//   * all search_width*degree neighbour ids are read, de-duplicated against the LDS visited
//     set and filtered by 256 threads at once; survivors are compacted;
//   * survivors are scored 32 at a time, 8 lanes per row (float4 per lane, three DPP adds);
//   * instead of sorting the whole queue every iteration, candidates that beat the current
//     worst queue entry are merged into the sorted queue by rank counting.  The queue that
//     results is the first itopk entries of sort(queue + candidates) by (distance,id), which
//     is what the reference's full sort leaves in those positions.
#include <mutex>

#include "search_internal.hpp"

namespace grab {

using namespace dev;

namespace {

constexpr int kBlock = 256;       // threads of a workgroup, ordinary batches
constexpr int kBlockSmall = 1024;  // small batches (kSmallBatchQueries queries at most)

enum { M_NSURV = 0, M_NCAND, M_NPAR, M_F, M_FULL, M_USED, M_COUNT };

struct Lds {
    float* query;
    uint64_t* top[2];
    uint64_t* cand;
    uint32_t* surv;
    uint32_t* parents;
    uint32_t* misc;
    uint32_t* parts;
    uint32_t* table;
};

__device__ __forceinline__ Lds carve(uint8_t* smem, const SearchArgs& a) {
    Lds l;
    SearchLdsLayout lay = search_lds_layout(a.itopk, a.dim, a.cmax, a.search_width,
                                            a.global_hash ? 0 : a.hash_bitlen, a.global_hash == nullptr, a.split_merge != 0);
    l.query = reinterpret_cast<float*>(smem + lay.off_query);
    l.top[0] = reinterpret_cast<uint64_t*>(smem + lay.off_top0);
    l.top[1] = reinterpret_cast<uint64_t*>(smem + lay.off_top1);
    l.cand = reinterpret_cast<uint64_t*>(smem + lay.off_cand);
    l.surv = reinterpret_cast<uint32_t*>(smem + lay.off_surv);
    l.parents = reinterpret_cast<uint32_t*>(smem + lay.off_parents);
    l.misc = reinterpret_cast<uint32_t*>(smem + lay.off_misc);
    l.parts = reinterpret_cast<uint32_t*>(smem + lay.off_parts);
    l.table = reinterpret_cast<uint32_t*>(smem + lay.off_hash);
    return l;
}

template <int FILTER>
struct FilterState {
    uint64_t start, end, mask;
};

template <int FILTER>
__device__ __forceinline__ bool filter_pass(const SearchArgs& a, const FilterState<FILTER>& f, uint32_t id) {
    if (FILTER == kFilterRange) {
        const uint64_t t = a.ts[id];
        return t >= f.start && t < f.end;  // [start,end), compute_distance.cuh:580-584
    }
    if (FILTER == kFilterMask) return (f.mask >> (a.labels[id] & 63)) & 1ull;
    if (FILTER == kFilterIdRange) return id >= f.start && id < f.end;  // nothing to read
    if (FILTER == kFilterRank) {
        const uint64_t x = a.rank_of_id[id];  // the row's place in timestamp order
        return x >= f.start && x < f.end;
    }
    return true;
}

// wave-aggregated append of the kept ids to the survivor list
__device__ __forceinline__ void append_survivor(const Lds& l, bool keep, uint32_t id, int lane) {
    const uint64_t b = __ballot(keep);
    if (b == 0) return;
    uint32_t base = 0;
    if (lane == 0) base = atomicAdd(&l.misc[M_NSURV], (uint32_t)__popcll(b));
    base = __shfl(base, 0, 64);
    if (keep) l.surv[base + __popcll(b & ((1ull << lane) - 1ull))] = id;
}

// Scores the survivors and appends those that beat `worst` to the candidate list.
// Two rows per 8-lane group per round, so that 2*CPL row loads are in flight per lane.
//
// Small batches (TB = 1024: fewer queries than CUs, every iteration a chain of two waits for HBM, graph rows then
// vectors) also touch the graph row of every row that joins the list: whichever of them becomes a parent later has
// its row in the second-level cache by then.  The words read stay in `touched` until the next round folds them
// away: nothing depends on them before, so the wait for them falls a round or a whole iteration later.
template <int TB, int CPL, int METRIC>
__device__ __forceinline__ void score_survivors(const SearchArgs& a, const Lds& l, const float4 (&qreg)[CPL ? CPL : 1],
                                                uint64_t worst, int grp, int j, uint32_t (&touched)[3]) {
    const uint32_t ns = l.misc[M_NSURV];
    const uint32_t nchunks = a.dim >> 2;
    const float4* q4 = reinterpret_cast<const float4*>(l.query);
    constexpr uint32_t kGroups = TB / 8;
    const int lane = threadIdx.x & 63;
    const uint64_t lt = (1ull << lane) - 1ull;
    for (uint32_t sbase = 0; sbase < ns; sbase += 2 * kGroups) {  // same trip count for every wave
        const uint32_t s = sbase + grp;
        uint64_t k0 = kInvalidKey, k1 = kInvalidKey;
        if (s < ns) {
            const bool two = (s + kGroups) < ns;
            const uint32_t id0 = l.surv[s];
            const uint32_t id1 = two ? l.surv[s + kGroups] : id0;
            const float4* r0 = reinterpret_cast<const float4*>(a.data + (size_t)id0 * a.dim);
            const float4* r1 = reinterpret_cast<const float4*>(a.data + (size_t)id1 * a.dim);
            float s0 = 0.0f, s1 = 0.0f;
            if (CPL > 0) {
                float4 v0[CPL ? CPL : 1], v1[CPL ? CPL : 1];
#pragma unroll
                for (int c = 0; c < CPL; ++c) v0[c] = r0[c * 8 + j];
#pragma unroll
                for (int c = 0; c < CPL; ++c) v1[c] = r1[c * 8 + j];
#pragma unroll
                for (int c = 0; c < CPL; ++c) s0 = fold4<METRIC>(s0, qreg[c], v0[c]);
#pragma unroll
                for (int c = 0; c < CPL; ++c) s1 = fold4<METRIC>(s1, qreg[c], v1[c]);
            } else {
                fold_rows_any<METRIC, true>(r0, r1, q4, j, nchunks, s0, s1);
            }
            s0 = group8_sum(s0);
            s1 = group8_sum(s1);
            if (METRIC == kMetricIP) {
                s0 = -s0;
                s1 = -s1;
            }
            k0 = make_key(s0, id0);
            if (two) k1 = make_key(s1, id1);
        }
        if (TB == kBlockSmall) {
            const uint32_t line = (uint32_t)j * 32u;  // a lane per 128 bytes of the row
            touched[2] ^= touched[0] ^ touched[1];  // the words of the round before
            touched[0] = touched[1] = 0;
            if (k0 < worst && line < a.degree) touched[0] = a.graph[(size_t)key_id(k0) * a.degree + line];
            if (k1 < worst && line < a.degree) touched[1] = a.graph[(size_t)key_id(k1) * a.degree + line];
        }
        // one reservation in the candidate list per wave, not one per row
        const bool p0 = (j == 0) && k0 < worst, p1 = (j == 0) && k1 < worst;
        const uint64_t b0 = __ballot(p0), b1 = __ballot(p1);
        const uint32_t n0 = (uint32_t)__popcll(b0), n1 = (uint32_t)__popcll(b1);
        if (n0 + n1 != 0) {  // wave-uniform
            uint32_t base = 0;
            if (lane == 0) base = atomicAdd(&l.misc[M_NCAND], n0 + n1);
            base = __shfl(base, 0, 64);
            if (p0) l.cand[base + __popcll(b0 & lt)] = k0;
            if (p1) l.cand[base + n0 + __popcll(b1 & lt)] = k1;
        }
    }
}

// number of entries of the sorted queue that are <= key, expanded flag ignored
__device__ __forceinline__ uint32_t upper_bound_u64(const uint64_t* arr, uint32_t n, uint64_t key) {
    uint32_t lo = 0, hi = n;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if ((arr[mid] & ~1ull) <= key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Number of list entries ordered before `key`: entries that are smaller and, with TIES, equal ones at a lower list
// index than `self`.  The list is read eight entries at a time, so that a thread waits for one LDS latency per
// eight entries, not per entry; the last, partial eight are read again from the list's last entry and not counted.
// The thread that does this for a candidate is the one the whole workgroup waits for, and what it costs is the
// number of instructions per entry: one compare and one addition without TIES.
template <bool TIES>
__device__ __forceinline__ uint32_t count_before(const uint64_t* cand, uint32_t nc, uint64_t key, uint32_t self) {
    uint32_t cnt = 0;
    for (uint32_t c = 0; c < nc; c += 8) {
        uint64_t v[8];
        if (c + 8 <= nc) {
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = cand[c + u];
        } else {
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = c + u < nc ? cand[c + u] : kInvalidKey;  // never smaller than a key, never equal to one
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) cnt += (v[u] < key || (TIES && v[u] == key && c + u < self)) ? 1u : 0u;
    }
    return cnt;
}

// The merge of a small batch (1024 threads a query, LDS with room for partial counts).  A thread that counts a whole
// list for its entry is what the workgroup waits for, so the counting is cut up: the list into kMergeChunks parts,
// and every (64 entries, list part) pair is a task of its own, as is the search of the queue for 64 candidates; the
// tasks go round the 16 waves, the counts to LDS, and after a barrier every entry adds up its counts and moves.
__device__ __forceinline__ void merge_split(const SearchArgs& a, const Lds& l, const uint64_t* src, uint64_t* dst, uint32_t nc_any, int tid) {
    const uint32_t nc = (uint32_t)__builtin_amdgcn_readfirstlane((int)nc_any);  // the same in every thread: the tasks below are picked per wave
    constexpr uint32_t NW = kBlockSmall / 64, NB = kMergeChunks;
    const uint32_t lane = (uint32_t)tid & 63u, wave = (uint32_t)__builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t itopk = a.itopk, cmax = a.cmax;
    const bool ties = a.flags & GRAB_FLAG_STRICT_REFERENCE;  // two candidates of one list are only ever equal when this lets an id in twice
    const uint32_t part_len = ((nc + 8u * NB - 1u) / (8u * NB)) * 8u;  // whole eights
    const uint32_t c64 = (nc + 63u) >> 6, q64 = (itopk + 63u) >> 6;
    uint32_t* cand_part = l.parts;                  // [NB][cmax]
    uint32_t* cand_queue = l.parts + NB * cmax;     // [cmax]
    uint32_t* queue_part = l.parts + (NB + 1u) * cmax;  // [NB][itopk]
    const uint32_t n_tasks = c64 * NB + c64 + q64 * NB;
    for (uint32_t task = wave; task < n_tasks; task += NW) {
        if (task < c64 * NB) {  // candidates task / NB * 64 .. + 63 against list part task % NB
            const uint32_t b = task % NB, x = (task / NB) * 64u + lane;
            const uint32_t from = min(b * part_len, nc), len = min(part_len, nc - from);
            if (x < nc) {
                const uint64_t kx = l.cand[x];
                const uint32_t self = x > from ? x - from : 0u;  // list places before x, counted from the part's start
                cand_part[b * cmax + x] = ties ? count_before<true>(l.cand + from, len, kx, self) : count_before<false>(l.cand + from, len, kx, 0);
            }
        } else if (task < c64 * NB + c64) {  // the queue entries at or below 64 candidates
            const uint32_t x = (task - c64 * NB) * 64u + lane;
            if (x < nc) cand_queue[x] = upper_bound_u64(src, itopk, l.cand[x]);
        } else {  // 64 queue entries against a list part; a queue entry goes ahead of an equal candidate
            const uint32_t t = task - c64 * NB - c64;
            const uint32_t b = t % NB, e = (t / NB) * 64u + lane;
            const uint32_t from = min(b * part_len, nc), len = min(part_len, nc - from);
            if (e < itopk) queue_part[b * itopk + e] = count_before<false>(l.cand + from, len, src[e] & ~1ull, 0);
        }
    }
    __syncthreads();
    for (uint32_t i = kBlockSmall - 1 - tid; i < itopk; i += kBlockSmall) {  // the last threads, as in the plain merge
        uint32_t r = i;
#pragma unroll
        for (uint32_t b = 0; b < NB; ++b) r += queue_part[b * itopk + i];
        if (r < itopk) dst[r] = src[i];
    }
    for (uint32_t x = tid; x < nc; x += kBlockSmall) {
        uint32_t r = cand_queue[x];
#pragma unroll
        for (uint32_t b = 0; b < NB; ++b) r += cand_part[b * cmax + x];
        if (r < itopk) dst[r] = l.cand[x];
    }
}

// Rank-counting merge of the candidate list into the sorted queue.  An entry's new position
// is the number of entries ordered before it by (distance,id); the expanded flag takes no part
// in the order, queue entries go ahead of equal candidates and equal candidates go by list
// index (equal entries only exist when GRAB_FLAG_STRICT_REFERENCE lets duplicates in).  On return `top` points to the merged queue
// and `spare` to the other buffer.
template <int TB>
__device__ __forceinline__ void merge_candidates(const SearchArgs& a, const Lds& l, uint64_t*& top,
                                                 uint64_t*& spare, int tid) {
    const uint32_t nc = l.misc[M_NCAND];
    if (nc == 0) return;
    const uint64_t* src = top;
    uint64_t* dst = spare;
    const uint32_t itopk = a.itopk;
    if (TB == kBlockSmall && a.split_merge) {
        merge_split(a, l, src, dst, nc, tid);
        __syncthreads();
        spare = top;
        top = dst;
        return;
    }
    // the last threads take the queue entries, the first ones the candidates: different waves where there are several
    for (uint32_t i = TB - 1 - tid; i < itopk; i += TB) {
        const uint64_t ki = src[i];
        const uint32_t r = i + count_before<false>(l.cand, nc, ki & ~1ull, 0);  // a queue entry goes ahead of an equal candidate
        if (r < itopk) dst[r] = ki;
    }
    // two candidates of one list are only ever equal when GRAB_FLAG_STRICT_REFERENCE lets an id in twice
    const bool ties = a.flags & GRAB_FLAG_STRICT_REFERENCE;
    for (uint32_t x = tid; x < nc; x += TB) {
        const uint64_t kx = l.cand[x];
        const uint32_t cnt = upper_bound_u64(src, itopk, kx) + (ties ? count_before<true>(l.cand, nc, kx, x) : count_before<false>(l.cand, nc, kx, x));
        if (cnt < itopk) dst[cnt] = kx;
    }
    __syncthreads();
    spare = top;
    top = dst;
}

// insert into the visited set; successful inserts are counted per workgroup (one LDS add per
// wave), and once the count says that every slot is taken the table is not walked any more.
// Must be called by all lanes of a wave together; `active` = this lane has a key.
__device__ __forceinline__ int visited_insert(const Lds& l, uint32_t* table, uint32_t bitlen, bool active, uint32_t key, int lane) {
    const bool full = __atomic_load_n(&l.misc[M_USED], __ATOMIC_RELAXED) >> bitlen;
    int r = 0;
    if (active) r = hash_insert(table, bitlen, key, full);
    const uint64_t b = __ballot(r == 1);
    if (b != 0 && lane == (int)__builtin_ctzll(b)) atomicAdd(&l.misc[M_USED], (uint32_t)__popcll(b));
    return r;
}

template <int TB, int CPL, int METRIC, int FILTER, bool GHASH>
__global__ void __launch_bounds__(TB) search_kernel(const SearchArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    Lds l = carve(smem, a);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int grp = tid >> 3, j = tid & 7;
    const uint32_t q = blockIdx.x;
    const bool strict = a.flags & GRAB_FLAG_STRICT_REFERENCE;
    const bool filter_first = (a.flags & GRAB_FLAG_FILTER_FIRST) && FILTER != kFilterNone;
    const uint32_t itopk = a.itopk;
    uint32_t* table = GHASH ? a.global_hash + ((size_t)q << a.hash_bitlen) : l.table;
    const uint32_t table_size = 1u << a.hash_bitlen;

    // ---- set-up: query, empty queue, empty visited set (search.cu:217-227) ----
    {
        const float* gq = a.queries + (size_t)q * a.dim;
        for (uint32_t i = tid; i < a.dim; i += TB) l.query[i] = gq[i];
        for (uint32_t i = tid; i < itopk; i += TB) l.top[0][i] = kInvalidKey;
        for (uint32_t i = tid; i < table_size; i += TB) table[i] = kInvalidId;
        if (tid < M_COUNT) l.misc[tid] = 0;
    }
    __syncthreads();

    float4 qreg[CPL ? CPL : 1];
    if (CPL > 0) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) qreg[c] = reinterpret_cast<const float4*>(l.query)[c * 8 + j];
    }

    FilterState<FILTER> flt{0, 0, 0};
    if (FILTER == kFilterRange || FILTER == kFilterIdRange || FILTER == kFilterRank) {
        flt.start = a.per_query_window ? a.win_start_arr[q] : a.win_start;
        flt.end = a.per_query_window ? a.win_end_arr[q] : a.win_end;
    } else if (FILTER == kFilterMask) {
        flt.mask = a.masks[q];
    }

    uint32_t my_f = 0, my_full = 0;          // per-thread counts, reduced at the end
    uint32_t c_iters = 0, c_seed = 0, c_par = 0, c_child = 0;  // uniform counts

    // ---- seeds (compute_distance.cuh:144-202, :204-269) ----
    for (uint32_t base = 0; base < a.n_seeds; base += TB) {
        const uint32_t i = base + tid;
        bool keep = false;
        uint32_t id = kInvalidId;
        if (i < a.n_seeds) {
            if (a.seeds != nullptr && i < a.n_provided) id = a.seeds[(size_t)q * a.n_provided + i];
            if ((uint64_t)id >= a.n) id = (uint32_t)((a.rand_xor_mask * (uint64_t)(i + 1)) % a.n);
            keep = true;
        }
        // strict: the reference queues a seed whatever the insert returned, unfiltered
        if (!strict && filter_first && keep) {
            if (FILTER != kFilterIdRange) my_f++;
            keep = filter_pass<FILTER>(a, flt, id);
        }
        const int r = visited_insert(l, table, a.hash_bitlen, keep, id, lane);
        if (r < 0) my_full++;
        if (!strict) {
            keep = keep && (r == 1);
            if (keep && FILTER != kFilterNone && !filter_first) {
                if (FILTER != kFilterIdRange) my_f++;
                keep = filter_pass<FILTER>(a, flt, id);
            }
        }
        append_survivor(l, keep, id, lane);
    }
    __syncthreads();
    c_seed = l.misc[M_NSURV];
    uint32_t touched[3] = {0, 0, 0};
    score_survivors<TB, CPL, METRIC>(a, l, qreg, kInvalidKey, grp, j, touched);
    __syncthreads();

    uint64_t* top = l.top[0];
    uint64_t* spare = l.top[1];
    for (uint32_t iter = 0; iter < a.max_iterations; ++iter) {
        // every 30 iterations the visited set is rebuilt from the queue (search.cu:265-283)
        const bool reset = iter > 0 && (iter % 30u == 0);
        for (int pass = 0; pass < 2; ++pass) {
            if (pass == 1) merge_candidates<TB>(a, l, top, spare, tid);
            if (reset && ((pass == 0) == strict)) {
                for (uint32_t i = tid; i < table_size; i += TB) table[i] = kInvalidId;
                if (tid == 0) l.misc[M_USED] = 0;
                __syncthreads();
                for (uint32_t base = 0; base < itopk; base += TB) {  // hashmap.cuh:103-117
                    const uint32_t i = base + tid;
                    const uint64_t k = i < itopk ? top[i] : kInvalidKey;
                    const bool have = (k != kInvalidKey) || (strict && i < itopk);
                    const int r = visited_insert(l, table, a.hash_bitlen, have, k != kInvalidKey ? key_id(k) : 0x7FFFFFFFu, lane);
                    if (r < 0) my_full++;
                }
                __syncthreads();
            }
        }

        // ---- parents: first search_width unexpanded queue entries (search.cu:38-107) ----
        if (wave == 0) {
            uint32_t found = 0;
            for (uint32_t base = 0; base < itopk && found < a.search_width; base += 64) {
                const uint32_t i = base + lane;
                const uint64_t k = i < itopk ? top[i] : kInvalidKey;
                const bool ok = (k != kInvalidKey) && !(k & 1ull);
                const uint64_t b = __ballot(ok);
                const uint32_t rank = found + (uint32_t)__popcll(b & ((1ull << lane) - 1ull));
                if (ok && rank < a.search_width) {
                    l.parents[rank] = key_id(k);
                    top[i] = k | 1ull;
                }
                found += (uint32_t)__popcll(b);
            }
            if (lane == 0) {
                l.misc[M_NPAR] = found < a.search_width ? found : a.search_width;
                l.misc[M_NSURV] = 0;
                l.misc[M_NCAND] = 0;
            }
        }
        __syncthreads();
        const uint32_t np = l.misc[M_NPAR];
        if (np == 0) break;
        c_iters++;
        c_par += np;

        // ---- expansion: ids, visited set, filter (compute_distance.cuh:274-380 etc.) ----
        const uint32_t total = np * a.degree;
        for (uint32_t base = 0; base < total; base += TB) {
            const uint32_t t = base + tid;
            bool keep = false;
            uint32_t nb = kInvalidId;
            if (t < total) {
                const uint32_t p = t / a.degree, off = t - p * a.degree;
                if (off < a.active_degree) {  // compute_distance.cuh:428-436
                    nb = a.graph[(size_t)l.parents[p] * a.degree + off];
                    keep = (uint64_t)nb < a.n;
                }
            }
            if (filter_first && keep) {
                if (FILTER != kFilterIdRange) my_f++;
                keep = filter_pass<FILTER>(a, flt, nb);
            }
            const int r = visited_insert(l, table, a.hash_bitlen, keep, nb, lane);
            if (r < 0) my_full++;
            keep = keep && (r == 1);
            if (keep && FILTER != kFilterNone && !filter_first) {
                if (FILTER != kFilterIdRange) my_f++;
                keep = filter_pass<FILTER>(a, flt, nb);
            }
            append_survivor(l, keep, nb, lane);
        }
        __syncthreads();
        c_child += l.misc[M_NSURV];
        score_survivors<TB, CPL, METRIC>(a, l, qreg, top[itopk - 1] & ~1ull, grp, j, touched);
        __syncthreads();
    }
    merge_candidates<TB>(a, l, top, spare, tid);
    asm volatile("" ::"v"(touched[0] ^ touched[1] ^ touched[2]));  // the reads above are kept; nothing is done with the words

    // ---- results (search.cu:348-355; ids widened here instead of a second kernel) ----
    for (uint32_t r = tid; r < a.k; r += TB) {
        const uint64_t k = top[r];
        int64_t id = strict ? (int64_t)0x7FFFFFFF : -1;
        float d = kDistMax;
        if (k != kInvalidKey) {
            id = (int64_t)key_id(k);
            d = key_dist(k);
        }
        a.out_ids[(size_t)q * a.k + r] = id;
        a.out_dists[(size_t)q * a.k + r] = d;
    }

    if (a.counters != nullptr) {
        if (my_f) atomicAdd(&l.misc[M_F], my_f);
        if (my_full) atomicAdd(&l.misc[M_FULL], my_full);
        __syncthreads();
        if (tid == 0) {
            grab_counters* c = a.counters + q;
            c->iterations = c_iters;
            c->seed_dists = c_seed;
            c->parents = c_par;
            c->filter_reads = l.misc[M_F];
            c->child_dists = c_child;
            c->hash_full = l.misc[M_FULL];
        }
    }
}

template <int CPL, int METRIC, int FILTER, bool GHASH>
int launch(const SearchArgs& a, size_t lds_bytes, hipStream_t stream) {
    const bool small = a.nq <= kSmallBatchQueries;
    auto kern = small ? search_kernel<kBlockSmall, CPL, METRIC, FILTER, GHASH> : search_kernel<kBlock, CPL, METRIC, FILTER, GHASH>;
    if (lds_bytes > 64 * 1024) {
        GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    }
    hipLaunchKernelGGL(kern, dim3(a.nq), dim3(small ? kBlockSmall : kBlock), lds_bytes, stream, a);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

template <int CPL, bool GHASH>
int dispatch_mf(const SearchArgs& a, int metric, int filter, size_t lds, hipStream_t s) {
#define GRAB_CASE(M, F) \
    if (metric == M && filter == F) return launch<CPL, M, F, GHASH>(a, lds, s);
    GRAB_CASE(kMetricL2, kFilterNone)
    GRAB_CASE(kMetricL2, kFilterRange)
    GRAB_CASE(kMetricL2, kFilterMask)
    GRAB_CASE(kMetricL2, kFilterIdRange)
    GRAB_CASE(kMetricL2, kFilterRank)
    GRAB_CASE(kMetricIP, kFilterNone)
    GRAB_CASE(kMetricIP, kFilterRange)
    GRAB_CASE(kMetricIP, kFilterMask)
    GRAB_CASE(kMetricIP, kFilterIdRange)
    GRAB_CASE(kMetricIP, kFilterRank)
#undef GRAB_CASE
    set_error("unsupported metric %d / filter %d", metric, filter);
    return GRAB_ERR_INVALID;
}

}  // namespace

// Visited sets of grab_search_ex_static, the entry point that allocates nothing: the per-query tables that
// grab_search_ex takes from hipMalloc when they do not fit LDS.  Part of the library's device image, so every
// device holds its own copy, at its own address, from the moment the library is loaded until the process ends.
// In host code the name below only identifies the symbol; the address a kernel may use comes from
// hipGetSymbolAddress with the device current, and is kept per device.
static __device__ __align__(256) uint32_t scratch[kStaticTableSlots];

namespace {
constexpr int kMaxDevices = 64;
uint32_t* g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;
}  // namespace

int static_visited_sets(uint32_t** tables) {
    int dev = -1;
    GRAB_HIP(hipGetDevice(&dev));
    GRAB_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        GRAB_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        GRAB_REQUIRE(p != nullptr, "no device address for the static visited sets");
        g_scratch_ptr[dev] = static_cast<uint32_t*>(p);
    }
    *tables = g_scratch_ptr[dev];
    return GRAB_OK;
}

int launch_search(const SearchArgs& a, int metric, int filter, size_t lds_bytes, hipStream_t stream) {
    if (a.global_hash != nullptr) return dispatch_mf<0, true>(a, metric, filter, lds_bytes, stream);
    if (a.dim == 128) return dispatch_mf<4, false>(a, metric, filter, lds_bytes, stream);
    return dispatch_mf<0, false>(a, metric, filter, lds_bytes, stream);
}

}  // namespace grab
