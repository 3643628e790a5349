// Beam search over the CAGRA graph, one 64-lane wave per query.
//
// Same algorithm and same results as the workgroup-per-query kernel (the loop of the
// reference's search_kernel / search_kernel_bucket / search_kernel_range,
// src/index/search.cu:149-370, :375-586, :589-798), decomposed for throughput on large
// batches: a selective filter leaves only a handful of rows to score per iteration, so the
// time of a query is a chain of dependent memory latencies (graph rows, then vectors) and
// the device is filled by keeping many queries resident per CU.  A wave needs no workgroup
// barrier, counts survivors and candidates in registers through ballots, and its LDS
// footprint (survivor list and visited set; queue and candidate list too when the queue is
// longer than 64 entries) is a few KB, so 20-28 queries share a CU.  Two kernels: the queue in
// LDS with a rank-counting merge (any length, also the reference's literal behaviour), and the
// queue in registers, one to four entries per lane, for queues of at most 256 entries.
#include "search_internal.hpp"

namespace grab {

using namespace dev;

namespace {

#ifndef GRAB_FIX_WAVES
#define GRAB_FIX_WAVES 7
#endif

struct WLds {
    uint64_t* top0;
    uint64_t* top1;
    uint64_t* cand;
    uint32_t* surv;
    uint32_t* parents;
    float* query;
    uint32_t* table;
};

__device__ __forceinline__ WLds carve_wave(uint8_t* smem, const SearchArgs& a, bool query_in_lds) {
    const SearchWaveLdsLayout lay = search_wave_lds_layout(a.itopk, query_in_lds ? a.dim : 0, a.cmax, a.ccap, a.single_queue != 0,
                                                           a.search_width, a.hash_bitlen);
    WLds l;
    l.top0 = reinterpret_cast<uint64_t*>(smem + lay.off_top0);
    l.top1 = reinterpret_cast<uint64_t*>(smem + lay.off_top1);
    l.cand = reinterpret_cast<uint64_t*>(smem + lay.off_cand);
    l.surv = reinterpret_cast<uint32_t*>(smem + lay.off_surv);
    l.parents = reinterpret_cast<uint32_t*>(smem + lay.off_parents);
    l.query = reinterpret_cast<float*>(smem + lay.off_query);
    l.table = reinterpret_cast<uint32_t*>(smem + lay.off_hash);
    return l;
}

// LDS accesses of the lanes of one wave are ordered by this (the workgroup is a single wave,
// so no hardware barrier is involved)
__device__ __forceinline__ void wave_sync() { __syncthreads(); }

template <int FILTER>
struct WFilter {
    uint64_t start, end, mask;
    uint32_t lo32, hi32;  // the id interval of kFilterIdRange (row ids are below 2^31)
};

template <int FILTER>
__device__ __forceinline__ bool wfilter_pass(const SearchArgs& a, const WFilter<FILTER>& f, uint32_t id) {
    if (FILTER == kFilterRange) {
        const uint64_t t = a.ts[id];
        return t >= f.start && t < f.end;  // [start,end), compute_distance.cuh:580-584
    }
    if (FILTER == kFilterMask) return (f.mask >> (a.labels[id] & 63)) & 1ull;
    if (FILTER == kFilterIdRange) return id >= f.lo32 && id < f.hi32;
    if (FILTER == kFilterRank) {
        const uint32_t x = a.rank_of_id[id];  // the row's place in timestamp order
        return x >= f.lo32 && x < f.hi32;
    }
    return true;
}

// whether a filter test reads a word per id (what the filter-read counter counts)
template <int FILTER>
__device__ __forceinline__ bool filter_reads(const SearchArgs&) {
    return FILTER == kFilterRange || FILTER == kFilterMask || FILTER == kFilterRank;
}

template <int FILTER>
__device__ __forceinline__ WFilter<FILTER> load_filter(const SearchArgs& a, uint32_t q) {
    WFilter<FILTER> f{0, 0, 0, 0, 0};
    if (FILTER == kFilterRange || FILTER == kFilterIdRange || FILTER == kFilterRank) {
        f.start = a.per_query_window ? a.win_start_arr[q] : a.win_start;
        f.end = a.per_query_window ? a.win_end_arr[q] : a.win_end;
        f.lo32 = f.start > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)f.start;
        f.hi32 = f.end > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)f.end;
    } else if (FILTER == kFilterMask) {
        f.mask = a.masks[q];
    }
    return f;
}

struct WCounts {
    uint32_t f, full;
    uint32_t used;  // wave-uniform: ids in the visited set
};

// visited set + filter for one id per lane; kept ids are appended to the survivor list
template <int FILTER>
__device__ __forceinline__ void visit(const SearchArgs& a, const WLds& l, const WFilter<FILTER>& flt, bool filter_first,
                                      bool valid, uint32_t id, int lane, uint32_t& nsurv, WCounts& c) {
    bool ok = valid;
    if (FILTER != kFilterNone && filter_first && ok) {
        if (filter_reads<FILTER>(a)) c.f++;
        ok = wfilter_pass<FILTER>(a, flt, id);
    }
    if (ok) {
        const int r = hash_insert(l.table, a.hash_bitlen, id, c.used >> a.hash_bitlen);
        if (r < 0) c.full++;
        ok = (r == 1);
    }
    c.used += (uint32_t)__popcll(__ballot(ok));
    if (FILTER != kFilterNone && !filter_first && ok) {
        if (filter_reads<FILTER>(a)) c.f++;
        ok = wfilter_pass<FILTER>(a, flt, id);
    }
    const uint64_t b = __ballot(ok);
    if (ok) l.surv[nsurv + __popcll(b & ((1ull << lane) - 1ull))] = id;
    nsurv += (uint32_t)__popcll(b);
}

// scores 16 survivors from position s0 on, 8 lanes per row and two rows per group in flight; keys
// that beat `worst` are appended to the candidate list.  Returns the new number of candidates.
template <int CPL, int METRIC>
__device__ __forceinline__ uint32_t score_round(const SearchArgs& a, const WLds& l, const float4 (&qreg)[CPL ? CPL : 1],
                                                uint32_t nsurv, uint32_t s0, uint64_t worst, uint32_t ncand, int lane) {
    const int grp = lane >> 3, j = lane & 7;
    const uint32_t nchunks = a.dim >> 2;
    const float4* q4 = reinterpret_cast<const float4*>(l.query);
    {
        const uint32_t sa = s0 + grp, sb = sa + 8;
        uint64_t k0 = kInvalidKey, k1 = kInvalidKey;
        if (sa < nsurv) {
            const bool two = sb < nsurv;
            const uint32_t id0 = l.surv[sa];
            const uint32_t id1 = two ? l.surv[sb] : id0;
            const float4* r0 = reinterpret_cast<const float4*>(a.data + (size_t)id0 * a.dim);
            const float4* r1 = reinterpret_cast<const float4*>(a.data + (size_t)id1 * a.dim);
            float d0 = 0.0f, d1 = 0.0f;
            if (CPL > 0) {
                float4 v0[CPL ? CPL : 1], v1[CPL ? CPL : 1];
#pragma unroll
                for (int c = 0; c < CPL; ++c) v0[c] = r0[c * 8 + j];
#pragma unroll
                for (int c = 0; c < CPL; ++c) v1[c] = r1[c * 8 + j];
#pragma unroll
                for (int c = 0; c < CPL; ++c) d0 = fold4<METRIC>(d0, qreg[c], v0[c]);
#pragma unroll
                for (int c = 0; c < CPL; ++c) d1 = fold4<METRIC>(d1, qreg[c], v1[c]);
            } else {
                fold_rows_any<METRIC, true>(r0, r1, q4, j, nchunks, d0, d1);
            }
            d0 = group8_sum(d0);
            d1 = group8_sum(d1);
            if (METRIC == kMetricIP) {
                d0 = -d0;
                d1 = -d1;
            }
            k0 = make_key(d0, id0);
            if (two) k1 = make_key(d1, id1);
        }
        const bool p0 = (j == 0) && k0 < worst, p1 = (j == 0) && k1 < worst;
        const uint64_t b0 = __ballot(p0), b1 = __ballot(p1);
        const uint64_t lt = (1ull << lane) - 1ull;
        if (p0) l.cand[ncand + __popcll(b0 & lt)] = k0;
        ncand += (uint32_t)__popcll(b0);
        if (p1) l.cand[ncand + __popcll(b1 & lt)] = k1;
        ncand += (uint32_t)__popcll(b1);
    }
    return ncand;
}

__device__ __forceinline__ uint32_t upper_bound_key(const uint64_t* arr, uint32_t n, uint64_t key) {
    uint32_t lo = 0, hi = n;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if ((arr[mid] & ~1ull) <= key) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// rank-counting merge of the candidate list into the sorted queue: an entry's new position is
// the number of entries ordered before it by (distance,id); the expanded flag takes no part,
// queue entries go ahead of equal candidates, equal candidates go by list index
__device__ __forceinline__ void merge(const WLds& l, uint32_t itopk, uint32_t nc, uint64_t*& top, uint64_t*& spare, int lane) {
    if (nc == 0) return;
    if (spare == nullptr) {
        // One queue buffer (itopk <= 64, at most 128 candidates): every lane works out where its queue
        // entry and its (up to two) candidates go, then all of them are written after the reads.
        const uint64_t ki = (uint32_t)lane < itopk ? top[lane] : kInvalidKey;
        uint32_t rq = itopk;
        if ((uint32_t)lane < itopk) {
            const uint64_t kn = ki & ~1ull;
            uint32_t cnt = 0;
            for (uint32_t c = 0; c < nc; ++c) cnt += (l.cand[c] < kn) ? 1u : 0u;
            rq = lane + cnt;
        }
        uint64_t kx[2] = {kInvalidKey, kInvalidKey};
        uint32_t rx[2] = {itopk, itopk};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t x = lane + 64u * t;
            if (x < nc) {
                kx[t] = l.cand[x];
                uint32_t cnt = upper_bound_key(top, itopk, kx[t]);
                for (uint32_t c = 0; c < nc; ++c) {
                    const uint64_t kc = l.cand[c];
                    cnt += (kc < kx[t] || (kc == kx[t] && c < x)) ? 1u : 0u;
                }
                rx[t] = cnt;
            }
        }
        wave_sync();
        if (rq < itopk) top[rq] = ki;
        if (rx[0] < itopk) top[rx[0]] = kx[0];
        if (rx[1] < itopk) top[rx[1]] = kx[1];
        wave_sync();
        return;
    }
    const uint64_t* src = top;
    uint64_t* dst = spare;
    for (uint32_t i = lane; i < itopk; i += 64) {
        const uint64_t ki = src[i];
        const uint64_t kn = ki & ~1ull;
        uint32_t cnt = 0;
        for (uint32_t c = 0; c < nc; ++c) cnt += (l.cand[c] < kn) ? 1u : 0u;
        const uint32_t r = i + cnt;
        if (r < itopk) dst[r] = ki;
    }
    for (uint32_t x = lane; x < nc; x += 64) {
        const uint64_t kx = l.cand[x];
        uint32_t cnt = upper_bound_key(src, itopk, kx);
        for (uint32_t c = 0; c < nc; ++c) {
            const uint64_t kc = l.cand[c];
            cnt += (kc < kx || (kc == kx && c < x)) ? 1u : 0u;
        }
        if (cnt < itopk) dst[cnt] = kx;
    }
    wave_sync();
    spare = top;
    top = dst;
}

__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

template <int CPL, int METRIC, int FILTER>
__global__ void __launch_bounds__(64) search_wave_kernel(const SearchArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const WLds l = carve_wave(smem, a, CPL == 0);
    const int lane = threadIdx.x;
    const int j = lane & 7;
    const uint32_t q = blockIdx.x;
    const bool strict = a.flags & GRAB_FLAG_STRICT_REFERENCE;
    const bool filter_first = a.flags & GRAB_FLAG_FILTER_FIRST;
    const uint32_t itopk = a.itopk;
    const uint32_t table_size = 1u << a.hash_bitlen;

    // ---- set-up: query, empty queue, empty visited set (search.cu:217-227) ----
    const float* gq = a.queries + (size_t)q * a.dim;
    float4 qreg[CPL ? CPL : 1];
    if (CPL > 0) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) qreg[c] = reinterpret_cast<const float4*>(gq)[c * 8 + j];
    } else {
        for (uint32_t i = lane; i < a.dim; i += 64) l.query[i] = gq[i];
    }
    for (uint32_t i = lane; i < itopk; i += 64) l.top0[i] = kInvalidKey;
    {
        uint4* t4 = reinterpret_cast<uint4*>(l.table);
        const uint4 inv = make_uint4(kInvalidId, kInvalidId, kInvalidId, kInvalidId);
        for (uint32_t i = lane; i < table_size / 4; i += 64) t4[i] = inv;
    }
    const WFilter<FILTER> flt = load_filter<FILTER>(a, q);
    wave_sync();

    WCounts cnt{0, 0, 0};
    uint32_t c_iters = 0, c_seed = 0, c_par = 0, c_child = 0;  // uniform

    uint64_t* top = l.top0;
    uint64_t* spare = a.single_queue ? nullptr : l.top1;  // one buffer: in-place merge
    // The survivor list holds a.cmax ids and the candidate list a.ccap keys, which the host may choose smaller
    // than what one iteration can produce: before 64 more ids are looked at, a list that could
    // overflow is scored and merged.  The queue after the last merge is the same as after one
    // merge of everything: the itopk smallest keys of the queue and all candidates either way.
    // (Under GRAB_FLAG_STRICT_REFERENCE the host keeps the lists at full size, because there the
    // visited set is rebuilt from the queue while the last candidates are still pending.)
    uint32_t nsurv = 0, ncand = 0, scored = 0;
    auto merge_pending = [&]() {
        merge(l, itopk, ncand, top, spare, lane);
        ncand = 0;
    };
    auto score_pending = [&]() {
        wave_sync();
        scored += nsurv;
        for (uint32_t s0 = 0; s0 < nsurv; s0 += 16) {
            // the candidate list may be shorter than the survivor list: merge before it could overflow
            if (ncand + min(16u, nsurv - s0) > a.ccap) {
                wave_sync();
                merge_pending();
            }
            ncand = score_round<CPL, METRIC>(a, l, qreg, nsurv, s0, top[itopk - 1] & ~1ull, ncand, lane);
        }
        nsurv = 0;
        wave_sync();
    };

    // ---- seeds (compute_distance.cuh:144-202, :204-269) ----
    for (uint32_t base = 0; base < a.n_seeds; base += 64) {
        if (nsurv + min(64u, a.n_seeds - base) > a.cmax) {
            score_pending();
            merge_pending();
        }
        const uint32_t i = base + lane;
        uint32_t id = kInvalidId;
        bool keep = false;
        if (i < a.n_seeds) {
            if (a.seeds != nullptr && i < a.n_provided) id = a.seeds[(size_t)q * a.n_provided + i];
            if ((uint64_t)id >= a.n) id = (uint32_t)((a.rand_xor_mask * (uint64_t)(i + 1)) % a.n);
            keep = true;
        }
        if (strict) {  // the reference queues a seed whatever the insert returned, unfiltered
            int r = 0;
            if (keep) r = hash_insert(l.table, a.hash_bitlen, id, cnt.used >> a.hash_bitlen);
            if (r < 0) cnt.full++;
            cnt.used += (uint32_t)__popcll(__ballot(r == 1));
            const uint64_t b = __ballot(keep);
            if (keep) l.surv[nsurv + __popcll(b & ((1ull << lane) - 1ull))] = id;
            nsurv += (uint32_t)__popcll(b);
        } else {
            visit<FILTER>(a, l, flt, filter_first, keep, id, lane, nsurv, cnt);
        }
    }
    score_pending();
    c_seed = scored;
    scored = 0;

    for (uint32_t iter = 0; iter < a.max_iterations; ++iter) {
        // every 30 iterations the visited set is rebuilt from the queue (search.cu:265-283)
        const bool reset = iter > 0 && (iter % 30u == 0);
        for (int pass = 0; pass < 2; ++pass) {
            if (pass == 1) merge_pending();
            if (reset && ((pass == 0) == strict)) {
                for (uint32_t i = lane; i < table_size; i += 64) l.table[i] = kInvalidId;
                cnt.used = 0;
                wave_sync();
                for (uint32_t base = 0; base < itopk; base += 64) {  // hashmap.cuh:103-117
                    const uint32_t i = base + lane;
                    const uint64_t k = i < itopk ? top[i] : kInvalidKey;
                    const bool full = cnt.used >> a.hash_bitlen;
                    int r = 0;
                    if (k != kInvalidKey) r = hash_insert(l.table, a.hash_bitlen, key_id(k), full);
                    else if (strict && i < itopk) r = hash_insert(l.table, a.hash_bitlen, 0x7FFFFFFFu, full);
                    if (r < 0) cnt.full++;
                    cnt.used += (uint32_t)__popcll(__ballot(r == 1));
                }
                wave_sync();
            }
        }

        // ---- parents: first search_width unexpanded queue entries (search.cu:38-107) ----
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
        const uint32_t np = found < a.search_width ? found : a.search_width;
        if (np == 0) break;
        wave_sync();
        c_iters++;
        c_par += np;

        // ---- expansion: ids, visited set, filter (compute_distance.cuh:274-380 etc.);
        // the rows of four parents are requested before any is processed ----
        for (uint32_t p0 = 0; p0 < np; p0 += 4) {
            for (uint32_t off0 = 0; off0 < a.active_degree; off0 += 64) {
                const uint32_t off = off0 + lane;
                uint32_t nb[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    nb[u] = kInvalidId;
                    if (p0 + u < np && off < a.active_degree) nb[u] = a.graph[(size_t)l.parents[p0 + u] * a.degree + off];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (p0 + u < np) {
                        if (nsurv + min(64u, a.active_degree - off0) > a.cmax) {
                            score_pending();
                            merge_pending();
                        }
                        visit<FILTER>(a, l, flt, filter_first, (uint64_t)nb[u] < a.n, nb[u], lane, nsurv, cnt);
                    }
                }
            }
        }
        score_pending();
        c_child += scored;
        scored = 0;
    }
    merge_pending();

    // ---- results (search.cu:348-355; ids widened here instead of a second kernel) ----
    for (uint32_t r = lane; r < a.k; r += 64) {
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
        const uint32_t f = wave_sum(cnt.f), full = wave_sum(cnt.full);
        if (lane == 0) {
            grab_counters* c = a.counters + q;
            c->iterations = c_iters;
            c->seed_dists = c_seed;
            c->parents = c_par;
            c->filter_reads = f;
            c->child_dists = c_child;
            c->hash_full = full;
        }
    }
}

// ---- the same search with the queue in registers (itopk <= 256, not the strict mode) ----------
// Lane i holds queue entries i, i + 64, ... (one, two or four registers).  A scored row that beats the worst entry is inserted at once: its
// position is the number of entries ordered before it (a ballot), the entries behind move one lane up
// (DPP wave_shr).  Inserting the candidates of an iteration one by one leaves the itopk smallest keys of
// queue and candidates in (distance,id) order, which is what the rank-counting merge leaves; an entry's
// expanded flag travels with it.  Parents are read from lanes with v_readlane, so neither the queue nor
// the candidate and parent lists exist in LDS: a query keeps the survivor list and the visited set there.
template <int NQ>
__device__ __forceinline__ void queue_insert(uint64_t (&qk)[NQ], uint64_t kc, uint32_t itopk, int lane) {
    // entry j lives in lane j % 64, register j / 64: every register is a sorted run and the runs follow each other
    bool before[NQ];
    uint32_t pos = 0;
#pragma unroll
    for (int s = 0; s < NQ; ++s) {
        before[s] = (qk[s] & ~1ull) <= kc;  // queue entries go ahead of an equal candidate
        pos += (uint32_t)__popcll(__ballot(before[s]));
    }
    if (pos >= itopk) return;
    const uint32_t ps = pos >> 6, pl = pos & 63u;
#pragma unroll
    for (int s = NQ - 1; s >= 0; --s) {
        if (NQ > 1 && (uint32_t)s < ps) continue;  // wave-uniform
        const uint64_t up = shfl_up_u64(qk[s]);
        if (NQ == 1 || (uint32_t)s == ps) {
            qk[s] = before[s] ? qk[s] : ((uint32_t)lane == pl ? kc : up);
        } else {  // the whole run moves up; its first lane takes the last entry of the run before
            const uint64_t carry = readlane_u64(qk[s > 0 ? s - 1 : 0], 63);
            qk[s] = lane == 0 ? carry : up;
        }
    }
}

// entry `index` of the queue (wave-uniform index)
template <int NQ>
__device__ __forceinline__ uint64_t queue_entry(const uint64_t (&qk)[NQ], uint32_t index) {
    uint64_t v = readlane_u64(qk[0], (int)(index & 63u));
#pragma unroll
    for (int s = 1; s < NQ; ++s)
        if ((index >> 6) == (uint32_t)s) v = readlane_u64(qk[s], (int)(index & 63u));
    return v;
}

// scores up to 16 survivors from s0 on (8 lanes per row; a second row per group only when more than 8
// are left) and inserts those that beat the worst queue entry
template <int CPL, int METRIC, bool TWO, int NQ>
__device__ __forceinline__ void score_insert_round(const SearchArgs& a, const WLds& l, const float4 (&qreg)[CPL ? CPL : 1],
                                                   uint32_t nsurv, uint32_t s0, uint64_t (&qk)[NQ], int lane) {
    const int grp = lane >> 3, j = lane & 7;
    const uint32_t nchunks = a.dim >> 2;
    const float4* q4 = reinterpret_cast<const float4*>(l.query);
    const uint32_t sa = s0 + grp, sb = sa + 8;
    uint64_t k0 = kInvalidKey, k1 = kInvalidKey;
    if (sa < nsurv) {
        const bool two = TWO && sb < nsurv;
        const uint32_t id0 = l.surv[sa];
        const uint32_t id1 = two ? l.surv[sb] : id0;
        const float4* r0 = reinterpret_cast<const float4*>(a.data + (size_t)id0 * a.dim);
        const float4* r1 = reinterpret_cast<const float4*>(a.data + (size_t)id1 * a.dim);
        float d0 = 0.0f, d1 = 0.0f;
        if (CPL > 0) {
            float4 v0[CPL ? CPL : 1], v1[CPL ? CPL : 1];
#pragma unroll
            for (int c = 0; c < CPL; ++c) v0[c] = r0[c * 8 + j];
            if (TWO) {
#pragma unroll
                for (int c = 0; c < CPL; ++c) v1[c] = r1[c * 8 + j];
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c) d0 = fold4<METRIC>(d0, qreg[c], v0[c]);
            if (TWO) {
#pragma unroll
                for (int c = 0; c < CPL; ++c) d1 = fold4<METRIC>(d1, qreg[c], v1[c]);
            }
        } else {
            fold_rows_any<METRIC, TWO>(r0, r1, q4, j, nchunks, d0, d1);
        }
        d0 = group8_sum(d0);
        if (METRIC == kMetricIP) d0 = -d0;
        k0 = make_key(d0, id0);
        if (TWO) {
            d1 = group8_sum(d1);
            if (METRIC == kMetricIP) d1 = -d1;
            if (two) k1 = make_key(d1, id1);
        }
    }
    const uint64_t worst = queue_entry<NQ>(qk, a.itopk - 1) & ~1ull;
    constexpr uint64_t kFirstOfEight = 0x0101010101010101ull;  // the lanes with j == 0 (the mask of a compare is free to combine, a lane's boolean is not)
    uint64_t b0 = __ballot(k0 < worst) & kFirstOfEight;
    while (b0) {  // wave-uniform
        const int src = __builtin_ctzll(b0);
        b0 &= b0 - 1;
        queue_insert<NQ>(qk, readlane_u64(k0, src), a.itopk, lane);
    }
    if (TWO) {
        uint64_t b1 = __ballot(k1 < worst) & kFirstOfEight;
        while (b1) {
            const int src = __builtin_ctzll(b1);
            b1 &= b1 - 1;
            queue_insert<NQ>(qk, readlane_u64(k1, src), a.itopk, lane);
        }
    }
}

// Seeds from the entry-point layer, listed by the wave itself.  The window (timestamps) becomes the interval of row
// ids [id_lo, id_hi): lanes 0-31 search the start, lanes 32-63 the end, one block of 32 consecutive pivots per level
// and one block of the base's timestamps at the end - a coalesced 256-byte read each.  Lane p then cuts the members
// of the query's p-th nearest group that lie in the interval out of the group's (ascending) id list: the stretch
// table brackets each bound, a short binary search finds it.  Groups are taken nearest first until min_rows members
// are reached (the group that crosses the mark is taken whole); the ids are laid end to end into `list`, at most
// max_ids of them.  Returns how many were written.
__device__ __forceinline__ uint32_t entry_walk(const SearchArgs& a, uint32_t q, uint32_t max_ids, uint32_t* list, int lane,
                                               uint32_t& id_lo, uint32_t& id_hi) {
    const EntryWalk& e = a.entry;
    const int half = lane >> 5, c = lane & 31;
    // lane p: the query's p-th nearest group (the read is in flight during the pivot search)
    const uint32_t grp = (uint32_t)lane < e.nprobe ? e.groups[(size_t)q * e.nprobe + lane] : kInvalidId;
    const uint64_t w = half ? (a.per_query_window ? a.win_end_arr[q] : a.win_end) : (a.per_query_window ? a.win_start_arr[q] : a.win_start);
    uint32_t blk = 0;  // per half: block of the next level that holds the bound
#pragma unroll
    for (int lev = 5; lev >= 0; --lev) {
        if ((uint32_t)lev < e.nlev) {  // uniform
            const uint32_t idx = blk * 32u + (uint32_t)c;
            const uint64_t t = e.piv[e.piv_off[lev] + min(idx, e.piv_cnt[lev] - 1u)];  // levels hold whole blocks of 32
            const bool less = (idx < e.piv_cnt[lev]) & (t < w);
            blk = blk * 32u + (uint32_t)__popc((uint32_t)(__ballot(less) >> (32 * half)));
        }
    }
    {
        const uint32_t idx = blk * 32u + (uint32_t)c;
        const uint64_t t = a.ts[min(idx, e.n_base - 1u)];
        const bool less = (idx < e.n_base) & (t < w);
        blk = min(blk * 32u + (uint32_t)__popc((uint32_t)(__ballot(less) >> (32 * half))), e.n_base);
    }
    id_lo = (uint32_t)__builtin_amdgcn_readlane((int)blk, 0);
    id_hi = max((uint32_t)__builtin_amdgcn_readlane((int)blk, 32), id_lo);
    uint32_t first = 0, len = 0;
    {
        bool act = false;
        uint32_t l0 = 0, h0 = 0, l1 = 0, h1 = 0;
        if ((uint32_t)lane < e.nprobe && grp != kInvalidId) {
            const uint32_t* tbl = e.tbl + (size_t)grp * 65u;
            const uint32_t s_lo = min(id_lo / e.stretch, 63u), s_hi = min(id_hi / e.stretch, 63u);
            l0 = tbl[s_lo], h0 = tbl[s_lo + 1], l1 = tbl[s_hi], h1 = tbl[s_hi + 1];
            act = true;
        }
        if (__ballot(act && (h0 - l0 > 4u || h1 - l1 > 4u)) == 0) {
            // the usual case - a stretch holds a member or two: the members of both stretches in one round of reads
            uint32_t below0 = 0, below1 = 0;
            if (act) {
                // the eight reads are issued together: clamped places, what lies beyond a stretch is left out of the count
                // afterwards (a read under a condition would be a branch and a wait for memory of its own)
                uint32_t m0[4], m1[4];
                const uint32_t last0 = h0 > 0u ? h0 - 1u : 0u, last1 = h1 > 0u ? h1 - 1u : 0u;  // places that exist
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    m0[j] = e.ids[min(l0 + j, last0)];
                    m1[j] = e.ids[min(l1 + j, last1)];
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
                if (e.ids[mid] < id_lo) l0 = mid + 1; else h0 = mid;
            }
            while (l1 < h1) {
                const uint32_t mid = (l1 + h1) >> 1;
                if (e.ids[mid] < id_hi) l1 = mid + 1; else h1 = mid;
            }
        }
        first = l0;
        len = l1 > l0 ? l1 - l0 : 0;
    }
    auto scan = [&](uint32_t x) {  // inclusive prefix sum over the lanes: four DPP shifts inside each row of 16, two broadcasts across rows
        int v = (int)x;
        v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1
        v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
        v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
        v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
        v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
        v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
        return (uint32_t)v;
    };
    if (scan(len) - len >= e.min_rows) len = 0;  // the walk ended before this group
    const uint32_t incl = scan(len), excl = incl - len;
    for (uint32_t i0 = 0; i0 < len && excl + i0 < max_ids; i0 += 8) {  // eight ids in flight, not one wait for memory per id
        uint32_t v[8];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) v[u] = e.ids[first + min(i0 + u, len - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u) asm volatile("" : "+v"(v[u]));  // all read here: none is put off into the branch that stores it
#pragma unroll
        for (uint32_t u = 0; u < 8; ++u)
            if (i0 + u < len && excl + i0 + u < max_ids) list[excl + i0 + u] = v[u];
    }
    return min((uint32_t)__builtin_amdgcn_readlane((int)incl, 63), max_ids);
}

// NQ: queue entries per lane (queues of up to 64 * NQ entries).
// FIX: the usual shape as compile-time facts - adjacency rows of 64 slots, all followed, at most four parents per
// iteration, at most 64 seeds, the filter tested first, and a survivor list that holds a whole iteration (256 ids):
// one block of row requests per iteration, no loop over parents or row pieces, and no path on which the list fills up.
template <int CPL, int METRIC, int FILTER, int NQ, bool FIX>
__global__ void __launch_bounds__(64)
__attribute__((amdgpu_waves_per_eu(FILTER == kFilterRange ? 5 : FILTER == kFilterRank ? 6 : (NQ == 1 ? (FIX ? GRAB_FIX_WAVES : 7) : 6),
                                   FILTER == kFilterRange ? 5 : FILTER == kFilterRank ? 6 : (NQ == 1 ? (FIX ? GRAB_FIX_WAVES : 7) : 6))))
search_wave_reg_kernel(const SearchArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    WLds l;
    {
        const SearchWaveLdsLayout lay = search_wave_lds_layout(0, CPL == 0 ? a.dim : 0, a.cmax, 0, true, 0, a.hash_bitlen);
        l.top0 = l.top1 = l.cand = nullptr;
        l.parents = nullptr;
        l.surv = reinterpret_cast<uint32_t*>(smem + lay.off_surv);
        l.query = reinterpret_cast<float*>(smem + lay.off_query);
        l.table = reinterpret_cast<uint32_t*>(smem + lay.off_hash);
    }
    const int lane = threadIdx.x;
    const int j = lane & 7;
    const uint32_t q = blockIdx.x;
    const bool filter_first = FIX || (a.flags & GRAB_FLAG_FILTER_FIRST);
    const uint32_t itopk = a.itopk;
    const uint32_t table_size = 1u << a.hash_bitlen;
    const uint32_t n32 = (uint32_t)a.n;
    const uint32_t degree = FIX ? 64u : a.degree, active_degree = FIX ? 64u : a.active_degree;

    const float* gq = a.queries + (size_t)q * a.dim;
    float4 qreg[CPL ? CPL : 1];
    if (CPL > 0) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) qreg[c] = reinterpret_cast<const float4*>(gq)[c * 8 + j];
    } else {
        for (uint32_t i = lane; i < a.dim; i += 64) l.query[i] = gq[i];
    }
    {
        uint4* t4 = reinterpret_cast<uint4*>(l.table);
        const uint4 inv = make_uint4(kInvalidId, kInvalidId, kInvalidId, kInvalidId);
        for (uint32_t i = lane; i < table_size / 4; i += 64) t4[i] = inv;
    }
    // seeds listed from the entry-point layer: the window holds timestamps and becomes the id interval of the filter
    const bool walk = FILTER == kFilterIdRange && a.entry.groups != nullptr;
    WFilter<FILTER> flt = walk ? WFilter<FILTER>{0, 0, 0, 0, 0} : load_filter<FILTER>(a, q);
    uint32_t n_listed = 0;
    if (FILTER == kFilterIdRange && walk) n_listed = entry_walk(a, q, a.n_seeds, l.surv, lane, flt.lo32, flt.hi32);
    wave_sync();

    WCounts cnt{0, 0, 0};
    uint32_t c_iters = 0, c_seed = 0, c_par = 0, c_child = 0;  // uniform
    uint64_t qk[NQ];                                           // queue entry lane + 64 * s in qk[s]
#pragma unroll
    for (int s = 0; s < NQ; ++s) qk[s] = kInvalidKey;
    uint32_t nsurv = 0, scored = 0;
    auto score_pending = [&]() {
        wave_sync();
        scored += nsurv;
        for (uint32_t s0 = 0; s0 < nsurv; s0 += 16) {
            if (nsurv - s0 > 8) score_insert_round<CPL, METRIC, true, NQ>(a, l, qreg, nsurv, s0, qk, lane);
            else score_insert_round<CPL, METRIC, false, NQ>(a, l, qreg, nsurv, s0, qk, lane);
        }
        nsurv = 0;
        wave_sync();
    };

    // ---- seeds (compute_distance.cuh:144-202, :204-269) ----
    for (uint32_t base = 0; base < a.n_seeds; base += 64) {
        if (nsurv + min(64u, a.n_seeds - base) > a.cmax) score_pending();
        const uint32_t i = base + lane;
        uint32_t id = kInvalidId;
        bool keep = false;
        if (i < a.n_seeds) {
            if (walk) {
                if (i < n_listed) id = l.surv[i];  // at most 64 of them: one round of this loop
            } else if (a.seeds != nullptr && i < a.n_provided) {
                id = a.seeds[(size_t)q * a.n_provided + i];
            }
            if ((uint64_t)id >= a.n) id = (uint32_t)((a.rand_xor_mask * (uint64_t)(i + 1)) % a.n);
            keep = true;
        }
        if (walk) wave_sync();  // the list shares the survivor list's memory
        visit<FILTER>(a, l, flt, filter_first, keep, id, lane, nsurv, cnt);
    }
    score_pending();
    c_seed = scored;
    scored = 0;

    for (uint32_t iter = 0; iter < a.max_iterations; ++iter) {
        // every 30 iterations the visited set is rebuilt from the queue (search.cu:265-283, hashmap.cuh:103-117)
        if (iter > 0 && (iter % 30u == 0)) {
            for (uint32_t i = lane; i < table_size; i += 64) l.table[i] = kInvalidId;
            cnt.used = 0;
            wave_sync();
#pragma unroll
            for (int s = 0; s < NQ; ++s) {
                int r = 0;
                if ((uint32_t)(lane + 64 * s) < itopk && qk[s] != kInvalidKey)
                    r = hash_insert(l.table, a.hash_bitlen, key_id(qk[s]), cnt.used >> a.hash_bitlen);
                if (r < 0) cnt.full++;
                cnt.used += (uint32_t)__popcll(__ballot(r == 1));
            }
            wave_sync();
        }

        // ---- parents: first search_width unexpanded queue entries (search.cu:38-107) ----
        // one entry per lane: the parents are read out of the lanes as they are needed.  More: lane u of `par`
        // collects parent u (the host sends search_width > 64 to the other kernel)
        int par = 0;
        uint32_t np = 0;
        uint64_t pb1 = 0;
        if (NQ == 1) {
            // an empty place holds the all-ones key, whose expanded flag is set like that of a used entry
            const bool open = ((uint32_t)qk[0] & 1u) == 0u && (itopk >= 64u || (uint32_t)lane < itopk);
            pb1 = __ballot(open);
            const uint32_t found = (uint32_t)__popcll(pb1);
            np = found < a.search_width ? found : a.search_width;
            if (open && (uint32_t)__popcll(pb1 & ((1ull << lane) - 1ull)) < a.search_width) qk[0] |= 1ull;
            par = (int)key_id(qk[0]);
        }
#pragma unroll
        for (int s = 0; s < (NQ == 1 ? 0 : NQ); ++s) {
            const bool open = (uint32_t)(lane + 64 * s) < itopk && qk[s] != kInvalidKey && !(qk[s] & 1ull);
            uint64_t pb = __ballot(open);
            if (np < a.search_width && pb != 0) {  // wave-uniform
                if (open && np + (uint32_t)__popcll(pb & ((1ull << lane) - 1ull)) < a.search_width) qk[s] |= 1ull;
                const int my_id = (int)key_id(qk[s]);
                while (np < a.search_width && pb != 0) {
                    const int src = __builtin_ctzll(pb);
                    pb &= pb - 1;
                    const int id = __builtin_amdgcn_readlane(my_id, src);
                    par = (uint32_t)lane == np ? id : par;
                    ++np;
                }
            }
        }
        if (np == 0) break;
        c_iters++;
        c_par += np;

        // ---- expansion: ids, visited set, filter (compute_distance.cuh:274-380 etc.);
        // the rows of four parents are requested before any is processed ----
        for (uint32_t p0 = 0; FIX ? p0 < 1u : p0 < np; p0 += 4) {
            uint32_t parent[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (NQ == 1) {
                    parent[u] = 0;
                    if (p0 + u < np) {
                        const int src = __builtin_ctzll(pb1);
                        pb1 &= pb1 - 1;
                        parent[u] = (uint32_t)__builtin_amdgcn_readlane(par, src);
                    }
                } else {
                    parent[u] = (uint32_t)__builtin_amdgcn_readlane(par, (int)((p0 + u) & 63u));
                }
            }
            for (uint32_t off0 = 0; FIX ? off0 < 64u : off0 < active_degree; off0 += 64) {
                const uint32_t off = off0 + lane;
                uint32_t nb[4];
                uint64_t nts[FILTER == kFilterRange ? 4 : 1];  // the neighbours' timestamps when they are stored like the graph
                uint32_t nrk[FILTER == kFilterRank ? 4 : 1];  // their places in timestamp order, likewise
                const bool row_ts = FILTER == kFilterRange && a.graph_ts != nullptr && filter_first;
                const bool row_rank = FILTER == kFilterRank && a.graph_rank != nullptr && filter_first;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    nb[u] = kInvalidId;
                    if (FILTER == kFilterRank) nrk[u] = 0xFFFFFFFFu;  // the place of a neighbour that is not there: beyond every interval
                    if (p0 + u < np && off < active_degree) {
                        nb[u] = a.graph[(size_t)parent[u] * degree + off];
                        if (FILTER == kFilterRange && row_ts) nts[u] = a.graph_ts[(size_t)parent[u] * degree + off];
                        if (FILTER == kFilterRank && row_rank) nrk[u] = a.graph_rank[(size_t)parent[u] * degree + off];
                    }
                }
                if (FILTER != kFilterNone && filter_first) {
                    // the filter leaves few of the 4 x 64 ids: they are gathered first and meet the visited
                    // set in one pass (same ids in the same order as four separate passes)
                    bool ok[4];
                    uint64_t bb[4];
                    uint32_t passing = 0;
                    // id interval: one subtraction and one unsigned compare per id - an id below the interval wraps
                    // round to a huge number, the invalid id (and with it the slots of parents that are not there)
                    // lies beyond every interval of row ids, and an interval never reaches past the last row
                    const uint32_t id_hi = min(flt.hi32, n32), id_span = id_hi > flt.lo32 ? id_hi - flt.lo32 : 0u;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (FILTER == kFilterIdRange) {
                            ok[u] = nb[u] - flt.lo32 < id_span;
                            bb[u] = __ballot(ok[u]);
                            passing += (uint32_t)__popcll(bb[u]);
                            continue;
                        }
                        if (FILTER == kFilterRank && row_rank) {  // the same test on the neighbours' places (invalid ids carry the place ~0)
                            cnt.f += nb[u] < n32 ? 1u : 0u;
                            ok[u] = nrk[u] - flt.lo32 < id_span;
                            bb[u] = __ballot(ok[u]);
                            passing += (uint32_t)__popcll(bb[u]);
                            continue;
                        }
                        ok[u] = p0 + u < np && nb[u] < n32;
                        if (ok[u]) {
                            if (filter_reads<FILTER>(a)) cnt.f++;
                            if (FILTER == kFilterRange && row_ts) ok[u] = nts[u] >= flt.start && nts[u] < flt.end;
                            else if (FILTER == kFilterRank && row_rank) ok[u] = nrk[u] >= flt.lo32 && nrk[u] < flt.hi32;
                            else ok[u] = wfilter_pass<FILTER>(a, flt, nb[u]);
                        }
                        bb[u] = __ballot(ok[u]);
                        passing += (uint32_t)__popcll(bb[u]);
                    }
                    if (FIX || nsurv + passing <= a.cmax) {
                        const uint64_t below = (1ull << lane) - 1ull;
                        uint32_t w = nsurv;
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            if (ok[u]) l.surv[w + __popcll(bb[u] & below)] = nb[u];
                            w += (uint32_t)__popcll(bb[u]);
                        }
                        wave_sync();
                        const uint32_t first = nsurv;
                        for (uint32_t base = 0; base < passing; base += 64) {
                            const bool valid = base + lane < passing;
                            const uint32_t id = valid ? l.surv[first + base + lane] : 0u;
                            int r = 0;
                            if (valid) r = hash_insert(l.table, a.hash_bitlen, id, cnt.used >> a.hash_bitlen);
                            if (r < 0) cnt.full++;
                            const uint64_t b = __ballot(r == 1);
                            cnt.used += (uint32_t)__popcll(b);
                            if (r == 1) l.surv[nsurv + __popcll(b & below)] = id;  // at or below the slots read so far
                            nsurv += (uint32_t)__popcll(b);
                        }
                        continue;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (p0 + u < np) {
                        if (nsurv + min(64u, active_degree - off0) > a.cmax) score_pending();
                        visit<FILTER>(a, l, flt, filter_first, nb[u] < n32, nb[u], lane, nsurv, cnt);
                    }
                }
            }
        }
        score_pending();
        c_child += scored;
        scored = 0;
    }

    // ---- results (search.cu:348-355; ids widened here instead of a second kernel) ----
#pragma unroll
    for (int s = 0; s < NQ; ++s) {
        const uint32_t r = (uint32_t)(lane + 64 * s);
        if (r < a.k) {
            int64_t id = -1;
            float d = kDistMax;
            if (qk[s] != kInvalidKey) {
                id = (int64_t)key_id(qk[s]);
                d = key_dist(qk[s]);
            }
            a.out_ids[(size_t)q * a.k + r] = id;
            a.out_dists[(size_t)q * a.k + r] = d;
        }
    }

    if (a.counters != nullptr) {
        const uint32_t f = wave_sum(cnt.f), full = wave_sum(cnt.full);
        if (lane == 0) {
            grab_counters* c = a.counters + q;
            c->iterations = c_iters;
            c->seed_dists = c_seed;
            c->parents = c_par;
            c->filter_reads = f;
            c->child_dists = c_child;
            c->hash_full = full;
        }
    }
}

template <int CPL, int METRIC, int FILTER>
int launch_wave(const SearchArgs& a, size_t lds_bytes, hipStream_t stream) {
    auto kern = !a.reg_queue       ? search_wave_kernel<CPL, METRIC, FILTER>
                : a.itopk <= 64  ? (a.fixed_shape && FILTER != kFilterNone ? search_wave_reg_kernel<CPL, METRIC, FILTER, 1, FILTER != kFilterNone>
                                                                           : search_wave_reg_kernel<CPL, METRIC, FILTER, 1, false>)
                : a.itopk <= 128 ? search_wave_reg_kernel<CPL, METRIC, FILTER, 2, false>
                                 : search_wave_reg_kernel<CPL, METRIC, FILTER, 4, false>;
    if (lds_bytes > 64 * 1024) {
        GRAB_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    }
    hipLaunchKernelGGL(kern, dim3(a.nq), dim3(64), lds_bytes, stream, a);
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

template <int CPL>
int dispatch_wave(const SearchArgs& a, int metric, int filter, size_t lds, hipStream_t s) {
#define GRAB_CASE(M, F) \
    if (metric == M && filter == F) return launch_wave<CPL, M, F>(a, lds, s);
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

int launch_search_wave(const SearchArgs& a, int metric, int filter, size_t lds_bytes, hipStream_t stream) {
    if (a.dim == 128) return dispatch_wave<4>(a, metric, filter, lds_bytes, stream);
    return dispatch_wave<0>(a, metric, filter, lds_bytes, stream);
}

}  // namespace grab
