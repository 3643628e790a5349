// CPU oracle for the GRAB-ANNS hot path.  TEST INFRASTRUCTURE ONLY: see oracle.h.
// Every function cites the reference lines (hxlou/GRAB-ANNS) that it restates.
// Build: g++ -O2 -ffp-contract=off -fopenmp -shared -fPIC oracle.cpp -o liboracle.so
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <unordered_map>
#include <utility>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// The reference writes "FLT_MAX" as the literal 3.40282e38f (compute_distance.cuh:162),
// which is a few ulps below the true FLT_MAX.  Unfilled result slots carry this value.
constexpr float kDistMax = 3.40282e38f;
constexpr uint64_t kInvalidKey = ~0ull;

inline int nthreads(int threads) {
#ifdef _OPENMP
    return threads > 0 ? threads : omp_get_max_threads();
#else
    (void)threads;
    return 1;
#endif
}

// monotone map float -> uint32 (negative scores occur for the inner-product metric)
inline uint32_t ord_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
inline float ord_float(uint32_t o) {
    uint32_t u = (o & 0x80000000u) ? (o & 0x7FFFFFFFu) : ~o;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
// queue key: ordered distance | node id | "already expanded" flag (the reference keeps the
// flag in the id's MSB, search.cu:49,85; here it is the LSB so that it never reorders nodes)
inline uint64_t make_key(float d, uint32_t id) { return ((uint64_t)ord_bits(d) << 32) | ((uint64_t)id << 1); }
inline uint32_t key_id(uint64_t k) { return (uint32_t)((k & 0xFFFFFFFFull) >> 1); }
inline float key_dist(uint64_t k) { return ord_float((uint32_t)(k >> 32)); }

inline float dist_metric(const float* a, const float* b, uint32_t dim, int metric) {
    return metric == ORC_METRIC_IP ? orc_ip_canon(a, b, dim) : orc_l2_canon(a, b, dim);
}

struct Filter {
    int kind;
    const uint64_t* ts;
    uint64_t start, end;
    const uint8_t* labels;
    uint64_t mask;
    bool pass(uint32_t id) const {
        if (kind == ORC_FILTER_RANGE) {
            uint64_t t = ts[id];
            return t >= start && t < end;  // compute_distance.cuh:580-584, [start,end)
        }
        if (kind == ORC_FILTER_MASK) return (mask >> (labels[id] & 63)) & 1ull;
        if (kind == ORC_FILTER_ID_RANGE) return id >= start && id < end;  // no memory read
        return true;
    }
};

Filter make_filter(int kind, const uint64_t* ts, const uint64_t* ws, const uint64_t* we, int per_query,
                   const uint8_t* labels, const uint64_t* masks, size_t q) {
    Filter f{kind, ts, 0, 0, labels, 0};
    if (kind == ORC_FILTER_RANGE || kind == ORC_FILTER_ID_RANGE) {
        f.start = per_query ? ws[q] : ws[0];
        f.end = per_query ? we[q] : we[0];
    } else if (kind == ORC_FILTER_MASK) {
        f.mask = masks[q];
    }
    return f;
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------------------------------------
// closed forms
// ---------------------------------------------------------------------------------------------
// src/index/smem_cal.cuh:13-23
uint32_t orc_next_power_of_2(uint32_t n) {
    if (n == 0) return 1;
    n--;
    n |= n >> 1;
    n |= n >> 2;
    n |= n >> 4;
    n |= n >> 8;
    n |= n >> 16;
    n++;
    return n;
}

// src/index/smem_cal.cuh:43-46, src/index/cagra.cu:871-873 (BLOCK_SIZE = 256, config.cuh:17)
uint32_t orc_queue_capacity(uint32_t itopk, uint32_t search_width, uint32_t degree) {
    uint32_t raw = itopk + search_width * degree;
    return std::max(256u, orc_next_power_of_2(raw));
}

// src/index/smem_cal.cuh:28-76
size_t orc_smem_bytes(uint32_t itopk, uint32_t dim, uint32_t search_width, uint32_t degree,
                      uint32_t hash_bitlen) {
    size_t smem = 0;
    smem += ((size_t)dim * 4 + 15) & ~(size_t)15;
    size_t hash_size = ((size_t)1 << hash_bitlen) * 4;
    smem += (hash_size + 15) & ~(size_t)15;
    size_t queue_mem = (size_t)orc_queue_capacity(itopk, search_width, degree) * 8;
    smem += (queue_mem + 15) & ~(size_t)15;
    smem += ((size_t)search_width * 4 + 15) & ~(size_t)15;
    smem += 256;
    if (hash_bitlen >= 14) smem -= ((size_t)1 << hash_bitlen) * 4;
    return smem;
}

// cagra.cu:862-864,887 | cagra_opt.cu:1127-1129,1158-1160 | :1241-1243,1275-1276 | :1352-1354,1387-1388
void orc_search_plan(int wrapper, uint32_t k, uint32_t itopk_param, uint32_t search_width,
                     uint32_t degree, uint32_t n_provided, uint32_t* itopk_eff, uint32_t* n_seeds,
                     uint32_t* queue_capacity) {
    uint32_t itopk = std::max(k, itopk_param);
    uint32_t floor_itopk = wrapper == ORC_WRAP_BUCKET ? 128u : 64u;
    if (itopk < floor_itopk) itopk = floor_itopk;
    uint32_t seeds = 0;
    switch (wrapper) {
        case ORC_WRAP_SEARCH: seeds = itopk_param / 4; break;  // uses the raw parameter
        case ORC_WRAP_SEARCH_OPT: seeds = std::min(std::max(32u, n_provided), itopk); break;
        default: seeds = std::min(n_provided, itopk); break;
    }
    *itopk_eff = itopk;
    *n_seeds = seeds;
    *queue_capacity = orc_queue_capacity(itopk, search_width, degree);
}

// ---------------------------------------------------------------------------------------------
// sorting
// ---------------------------------------------------------------------------------------------
// src/index/bitonic.cuh:53-111 executed lane by lane.  The element at (lane, i) has global
// index lane*per_lane+i; a compare-exchange leaves equal keys in place (bitonic.cuh:18,33).
void orc_bitonic_network(float* keys, uint32_t* vals, uint32_t lanes, uint32_t per_lane, int asc) {
    const uint32_t total = lanes * per_lane;
    for (uint32_t size = 2; size <= total; size <<= 1) {
        for (uint32_t stride = size / 2; stride > 0; stride >>= 1) {
            // every compare-exchange pair is disjoint inside one (size,stride) stage, so the
            // stage can be evaluated pair by pair
            for (uint32_t g = 0; g < total; ++g) {
                uint32_t p = g ^ stride;
                if (g > p) continue;
                bool direction = ((g & size) == 0) != !asc;
                bool want_min_at_g = direction;  // g < p
                float kg = keys[g], kp = keys[p];
                if (kg != kp && ((kg < kp) != want_min_at_g)) {
                    std::swap(keys[g], keys[p]);
                    std::swap(vals[g], vals[p]);
                }
            }
        }
    }
}

void orc_sort_pairs(float* keys, uint32_t* vals, size_t n) {
    std::vector<std::pair<float, uint32_t>> v(n);
    for (size_t i = 0; i < n; ++i) v[i] = {keys[i], vals[i]};
    std::sort(v.begin(), v.end());
    for (size_t i = 0; i < n; ++i) {
        keys[i] = v[i].first;
        vals[i] = v[i].second;
    }
}

// ---------------------------------------------------------------------------------------------
// visited set
// ---------------------------------------------------------------------------------------------
// src/index/hashmap.cuh:30-36
void orc_hash_init(uint32_t* table, uint32_t bitlen) {
    std::fill(table, table + ((size_t)1 << bitlen), ORC_INVALID);
}

// src/index/hashmap.cuh:59-91 (hash_func :43-46); returns -1 when the table is full so that
// callers can count overflows, the reference folds that into "false"
static int hash_insert3(uint32_t* table, uint32_t bitlen, uint32_t key) {
    const uint32_t size = 1u << bitlen, mask = size - 1;
    uint32_t index = (key ^ (key >> bitlen)) & mask;
    for (uint32_t i = 0; i < size; ++i) {
        uint32_t old = table[index];
        if (old == ORC_INVALID) {
            table[index] = key;
            return 1;
        }
        if (old == key) return 0;
        index = (index + 1) & mask;
    }
    return -1;
}

int orc_hash_insert(uint32_t* table, uint32_t bitlen, uint32_t key) {
    return hash_insert3(table, bitlen, key) == 1;
}

void orc_hash_insert_many(uint32_t* table, uint32_t bitlen, const uint32_t* keys, size_t n,
                          uint32_t* results) {
    for (size_t i = 0; i < n; ++i) results[i] = (uint32_t)orc_hash_insert(table, bitlen, keys[i]);
}

// ---------------------------------------------------------------------------------------------
// distances
// ---------------------------------------------------------------------------------------------
// Canonical order of the product (role of compute_distance.cuh:14-139): eight partial sums,
// partial j takes the float4 chunks j, j+8, j+16, ... in order, each element folded with a
// fused multiply-add; the partials are combined pairwise (0+1)+(2+3) then +((4+5)+(6+7)).
float orc_l2_canon(const float* a, const float* b, uint32_t dim) {
    float acc[8];
    const uint32_t nchunks = dim / 4;
    for (uint32_t j = 0; j < 8; ++j) {
        float s = 0.0f;
        for (uint32_t c = j; c < nchunks; c += 8) {
            for (uint32_t e = 0; e < 4; ++e) {
                float d = a[c * 4 + e] - b[c * 4 + e];
                s = std::fmaf(d, d, s);
            }
        }
        acc[j] = s;
    }
    float s01 = acc[0] + acc[1], s23 = acc[2] + acc[3], s45 = acc[4] + acc[5], s67 = acc[6] + acc[7];
    float s0123 = s01 + s23, s4567 = s45 + s67;
    return s0123 + s4567;
}

float orc_ip_canon(const float* a, const float* b, uint32_t dim) {
    float acc[8];
    const uint32_t nchunks = dim / 4;
    for (uint32_t j = 0; j < 8; ++j) {
        float s = 0.0f;
        for (uint32_t c = j; c < nchunks; c += 8) {
            for (uint32_t e = 0; e < 4; ++e) s = std::fmaf(a[c * 4 + e], b[c * 4 + e], s);
        }
        acc[j] = s;
    }
    float s01 = acc[0] + acc[1], s23 = acc[2] + acc[3], s45 = acc[4] + acc[5], s67 = acc[6] + acc[7];
    float s0123 = s01 + s23, s4567 = s45 + s67;
    return -(s0123 + s4567);
}

// tests/test_cagra_auto.cu:48-50, src/index/cagra.cu:58-61
float orc_l2_natural(const float* a, const float* b, uint32_t dim) {
    float r = 0;
    for (uint32_t i = 0; i < dim; ++i) {
        float d = a[i] - b[i];
        r += d * d;
    }
    return r;
}

// src/index/compute_distance.cuh:120-139: lane l sums elements i*32+l, then xor butterfly
// with offsets 16,8,4,2,1 (value seen by lane 0)
float orc_l2_ref_warp(const float* a, const float* b, uint32_t dim) {
    float lane[32];
    for (uint32_t l = 0; l < 32; ++l) {
        float s = 0.0f;
        for (uint32_t i = 0; i * 32 + l < dim; ++i) {
            float d = a[i * 32 + l] - b[i * 32 + l];
            s += d * d;
        }
        lane[l] = s;
    }
    for (uint32_t off = 16; off > 0; off >>= 1) {
        float next[32];
        for (uint32_t l = 0; l < 32; ++l) next[l] = lane[l] + lane[l ^ off];
        std::memcpy(lane, next, sizeof(lane));
    }
    return lane[0];
}

void orc_l2_canon_many(const float* q, const float* data, const uint32_t* ids, size_t n, uint32_t dim,
                       int metric, float* out) {
    for (size_t i = 0; i < n; ++i) out[i] = dist_metric(q, data + (size_t)ids[i] * dim, dim, metric);
}

// ---------------------------------------------------------------------------------------------
// exact filtered top-k: tests/test_cagra_auto.cu:57-89 with the (dist,id) tie rule
// ---------------------------------------------------------------------------------------------
void orc_bruteforce_topk(const float* data, size_t n, uint32_t dim, const float* queries, size_t nq,
                         uint32_t k, int metric, int filter_kind, const uint64_t* ts,
                         const uint64_t* win_start, const uint64_t* win_end, int per_query_window,
                         const uint8_t* labels, const uint64_t* masks, int64_t* out_ids,
                         float* out_dists, int threads) {
#pragma omp parallel for schedule(dynamic, 1) num_threads(nthreads(threads))
    for (long long qi = 0; qi < (long long)nq; ++qi) {
        const float* q = queries + (size_t)qi * dim;
        Filter f = make_filter(filter_kind, ts, win_start, win_end, per_query_window, labels, masks, qi);
        std::vector<uint64_t> cand;
        cand.reserve(1024);
        for (size_t j = 0; j < n; ++j) {
            if (!f.pass((uint32_t)j)) continue;
            float d = dist_metric(q, data + j * dim, dim, metric);
            cand.push_back(((uint64_t)ord_bits(d) << 32) | (uint64_t)j);
            if (cand.size() >= (size_t)k * 8 + 4096) {  // bounded memory: keep the k best so far
                std::nth_element(cand.begin(), cand.begin() + k, cand.end());
                cand.resize(k);
            }
        }
        size_t keep = std::min((size_t)k, cand.size());
        std::partial_sort(cand.begin(), cand.begin() + keep, cand.end());
        for (uint32_t r = 0; r < k; ++r) {
            if (r < keep) {
                out_ids[qi * k + r] = (int64_t)(cand[r] & 0xFFFFFFFFull);
                out_dists[qi * k + r] = ord_float((uint32_t)(cand[r] >> 32));
            } else {
                out_ids[qi * k + r] = -1;
                out_dists[qi * k + r] = kDistMax;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// graph build
// ---------------------------------------------------------------------------------------------
// Post-processing rule of src/index/cagra.cu:156-197 applied to exact candidates: sort by
// (dist,id), drop the row's own id, keep k, pad with 0xFFFFFFFF.
void orc_knn_graph(const float* data, size_t n, uint32_t dim, uint32_t k, int metric, uint32_t* out,
                   int threads) {
#pragma omp parallel for schedule(dynamic, 16) num_threads(nthreads(threads))
    for (long long i = 0; i < (long long)n; ++i) {
        std::vector<uint64_t> cand(n);
        const float* a = data + (size_t)i * dim;
        for (size_t j = 0; j < n; ++j)
            cand[j] = ((uint64_t)ord_bits(dist_metric(a, data + j * dim, dim, metric)) << 32) | j;
        size_t keep = std::min(n, (size_t)k + 1);
        std::partial_sort(cand.begin(), cand.begin() + keep, cand.end());
        uint32_t filled = 0;
        for (size_t r = 0; r < keep && filled < k; ++r) {
            uint32_t id = (uint32_t)(cand[r] & 0xFFFFFFFFull);
            if (id != (uint32_t)i) out[(size_t)i * k + filled++] = id;
        }
        while (filled < k) out[(size_t)i * k + filled++] = ORC_INVALID;
    }
}

// src/index/cagra.cu:219-276 (kern_prune).  For node A and each D = row[kAD] (kAD < deg-1,
// D valid), every entry Bc of D's row adds one to the first position kAB > kAD of A's row that
// holds Bc.  Counts saturate at 255 when stored (:274).  An id lookup replaces the innermost
// linear scan; it returns the same "first position after kAD".
void orc_detour_counts(const uint32_t* knn, size_t n, uint32_t degree, uint8_t* counts, int threads) {
#pragma omp parallel for schedule(dynamic, 64) num_threads(nthreads(threads))
    for (long long a = 0; a < (long long)n; ++a) {
        const uint32_t* row = knn + (size_t)a * degree;
        std::unordered_map<uint32_t, std::vector<uint32_t>> pos;
        pos.reserve(degree * 2);
        for (uint32_t p = 0; p < degree; ++p) pos[row[p]].push_back(p);  // ascending positions
        std::vector<uint32_t> cnt(degree, 0);
        for (uint32_t kAD = 0; kAD + 1 < degree; ++kAD) {
            uint32_t D = row[kAD];
            if (D == ORC_INVALID) continue;
            if ((size_t)D >= n) continue;  // the reference would read out of bounds here
            const uint32_t* drow = knn + (size_t)D * degree;
            for (uint32_t kDB = 0; kDB < degree; ++kDB) {
                auto it = pos.find(drow[kDB]);
                if (it == pos.end()) continue;
                for (uint32_t p : it->second) {
                    if (p > kAD) {
                        cnt[p]++;
                        break;
                    }
                }
            }
        }
        for (uint32_t p = 0; p < degree; ++p)
            counts[(size_t)a * degree + p] = cnt[p] > 255 ? 255 : (uint8_t)cnt[p];
    }
}

// src/index/cagra.cu:367-392: stable sort of positions by detour count, keep out_degree
void orc_prune(const uint32_t* knn, size_t n, uint32_t in_degree, uint32_t out_degree, uint32_t* out,
               int threads) {
    std::vector<uint8_t> counts(n * in_degree);
    orc_detour_counts(knn, n, in_degree, counts.data(), threads);
#pragma omp parallel for num_threads(nthreads(threads))
    for (long long i = 0; i < (long long)n; ++i) {
        const uint8_t* c = counts.data() + (size_t)i * in_degree;
        std::vector<int> idx(in_degree);
        for (uint32_t p = 0; p < in_degree; ++p) idx[p] = (int)p;
        std::stable_sort(idx.begin(), idx.end(), [&](int x, int y) { return c[x] < c[y]; });
        for (uint32_t p = 0; p < out_degree; ++p)
            out[(size_t)i * out_degree + p] = knn[(size_t)i * in_degree + idx[p]];
    }
}

// src/index/cagra.cu:418-444,496-517 executed sequentially: column by column, sources in
// ascending order inside a column.  rev_counts keeps counting past degree (:437).
void orc_reverse_graph(const uint32_t* graph, size_t n, uint32_t degree, uint32_t* rev,
                       uint32_t* rev_counts) {
    std::fill(rev, rev + n * degree, ORC_INVALID);
    std::fill(rev_counts, rev_counts + n, 0u);
    for (uint32_t k = 0; k < degree; ++k) {
        for (size_t src = 0; src < n; ++src) {
            uint32_t dest = graph[src * degree + k];
            if ((size_t)dest >= n) continue;
            uint32_t p = rev_counts[dest]++;
            if (p < degree) rev[(size_t)dest * degree + p] = (uint32_t)src;
        }
    }
}

// src/index/cagra.cu:574-650: alternate next usable forward edge / next usable reverse edge;
// slots past the number of accepted neighbours keep their previous forward value (:645-648).
void orc_merge_graphs(uint32_t* graph, const uint32_t* rev, const uint32_t* rev_counts, size_t n,
                      uint32_t degree, int threads) {
#pragma omp parallel for num_threads(nthreads(threads))
    for (long long j = 0; j < (long long)n; ++j) {
        const uint32_t* fwd = graph + (size_t)j * degree;
        const uint32_t* rv = rev + (size_t)j * degree;
        uint32_t rev_count = std::min(rev_counts[j], degree);
        std::vector<uint32_t> nb;
        nb.reserve(degree);
        auto dup = [&](uint32_t v) { return std::find(nb.begin(), nb.end(), v) != nb.end(); };
        uint32_t cf = 0, cr = 0;
        while (nb.size() < degree) {
            bool added = false;
            while (cf < degree) {
                uint32_t c = fwd[cf++];
                if (c == (uint32_t)j) continue;
                if (dup(c)) continue;
                nb.push_back(c);
                added = true;
                break;
            }
            if (nb.size() >= degree) break;
            while (cr < rev_count) {
                uint32_t c = rv[cr++];
                if ((size_t)c >= n) continue;
                if (c == (uint32_t)j) continue;
                if (dup(c)) continue;
                nb.push_back(c);
                added = true;
                break;
            }
            if (!added) break;
        }
        uint32_t* dst = graph + (size_t)j * degree;
        for (size_t p = 0; p < nb.size(); ++p) dst[p] = nb[p];
    }
}

// src/index/cagra.cu:665-711
void orc_optimize(const uint32_t* knn, size_t n, uint32_t in_degree, uint32_t out_degree,
                  uint32_t* out, int threads) {
    orc_prune(knn, n, in_degree, out_degree, out, threads);
    std::vector<uint32_t> rev(n * out_degree), cnt(n);
    orc_reverse_graph(out, n, out_degree, rev.data(), cnt.data());
    orc_merge_graphs(out, rev.data(), cnt.data(), n, out_degree, threads);
}

// ---------------------------------------------------------------------------------------------
// beam search: src/index/search.cu:149-370 (+ :375-586 bucket, :589-798 range) with the
// expansion steps of src/index/compute_distance.cuh:204-269,274-380,386-505,512-614
// ---------------------------------------------------------------------------------------------
static void search_one(const float* data, size_t n, uint32_t dim, const uint32_t* graph, uint32_t degree,
                       uint32_t active_degree, const float* q, uint32_t k, uint32_t itopk, uint32_t sw,
                       uint32_t max_iter, uint32_t bitlen, uint32_t n_seeds, const uint32_t* seeds,
                       uint32_t n_provided, uint64_t mask, int metric, const Filter& flt, uint32_t flags,
                       int64_t* out_ids, float* out_dists, orc_counters* ctr, std::vector<uint32_t>& table) {
    const bool strict = flags & ORC_FLAG_STRICT_REFERENCE;
    // filter-first: the filter is evaluated before the visited-set insert, so rows outside the
    // filter never occupy the table.  Membership of admissible rows is unchanged, hence so are
    // the results as long as the table never fills; not a reference mode.
    const bool filter_first = (flags & ORC_FLAG_FILTER_FIRST) && flt.kind != ORC_FILTER_NONE;
    orc_counters c{};
    table.assign((size_t)1 << bitlen, ORC_INVALID);
    std::vector<uint64_t> top(itopk, kInvalidKey);
    std::vector<uint64_t> cands;  // in slot order
    cands.reserve((size_t)sw * degree + n_seeds);

    // Once every slot is taken an insert fails whether or not the id is in the table
    // (hashmap.cuh:89-90 reports "full" as "present"), so the walk over the table is skipped and
    // the attempt is counted as an overflow.
    size_t used = 0;
    auto insert = [&](uint32_t id) -> bool {
        if (used == table.size()) {
            c.hash_full++;
            return false;
        }
        int r = hash_insert3(table.data(), bitlen, id);
        if (r < 0) c.hash_full++;
        if (r == 1) used++;
        return r == 1;
    };
    auto merge = [&]() {
        if (cands.empty()) return;
        // top is sorted by (distance,id); appending the candidates in slot order and sorting
        // stably with the expanded flag masked out keeps queue entries ahead of equal
        // candidates and equal candidates in slot order, which is the tie rule of the device
        // merge (the reference sorts by distance alone and leaves ties to the sort routine)
        std::vector<uint64_t> all(top);
        all.insert(all.end(), cands.begin(), cands.end());
        std::stable_sort(all.begin(), all.end(), [](uint64_t x, uint64_t y) { return (x >> 1) < (y >> 1); });
        std::copy(all.begin(), all.begin() + itopk, top.begin());
        cands.clear();
    };
    auto reset_restore = [&]() {  // search.cu:273-283, hashmap.cuh:103-117
        std::fill(table.begin(), table.end(), ORC_INVALID);
        used = 0;
        bool any_invalid = false;
        for (uint32_t i = 0; i < itopk; ++i) {
            if (top[i] == kInvalidKey) {
                any_invalid = true;
                continue;
            }
            insert(key_id(top[i]));
        }
        // hashmap.cuh:109-113 strips the MSB before comparing with 0xFFFFFFFF, so an empty
        // queue slot re-enters the table as key 0x7FFFFFFF
        if (strict && any_invalid) insert(0x7FFFFFFFu);
    };

    // seeds: compute_distance.cuh:144-202 / :204-269
    for (uint32_t i = 0; i < n_seeds; ++i) {
        uint32_t id = ORC_INVALID;
        if (seeds != nullptr && i < n_provided) id = seeds[i];
        if ((size_t)id >= n) id = (uint32_t)((mask * (uint64_t)(i + 1)) % (uint64_t)n);
        if (!strict && filter_first) {
            if (flt.kind != ORC_FILTER_ID_RANGE) c.filter_reads++;
            if (!flt.pass(id)) continue;
        }
        bool fresh = insert(id);
        if (!strict) {
            if (!fresh) continue;
            if (flt.kind != ORC_FILTER_NONE && !filter_first) {
                if (flt.kind != ORC_FILTER_ID_RANGE) c.filter_reads++;
                if (!flt.pass(id)) continue;
            }
        }
        c.seed_dists++;
        cands.push_back(make_key(dist_metric(q, data + (size_t)id * dim, dim, metric), id));
    }

    for (uint32_t iter = 0; iter < max_iter; ++iter) {
        const bool reset = iter > 0 && (iter % 30 == 0);
        if (reset && strict) reset_restore();
        merge();
        if (reset && !strict) reset_restore();

        // search.cu:38-107
        std::vector<uint32_t> parents;
        for (uint32_t i = 0; i < itopk && parents.size() < sw; ++i) {
            if (top[i] == kInvalidKey || (top[i] & 1ull)) continue;
            parents.push_back(key_id(top[i]));
            top[i] |= 1ull;
        }
        if (parents.empty()) break;
        c.iterations++;

        for (uint32_t p : parents) {
            c.parents++;
            const uint32_t* row = graph + (size_t)p * degree;
            for (uint32_t off = 0; off < degree; ++off) {
                if (off >= active_degree) continue;      // compute_distance.cuh:428-436
                uint32_t nb = row[off];
                if (nb == ORC_INVALID) continue;
                if (filter_first) {
                    if (flt.kind != ORC_FILTER_ID_RANGE) c.filter_reads++;
                    if (!flt.pass(nb)) continue;
                }
                bool fresh = insert(nb);
                if (!fresh) continue;
                if (flt.kind != ORC_FILTER_NONE && !filter_first) {  // compute_distance.cuh:580-584
                    if (flt.kind != ORC_FILTER_ID_RANGE) c.filter_reads++;
                    if (!flt.pass(nb)) continue;
                }
                c.child_dists++;
                cands.push_back(make_key(dist_metric(q, data + (size_t)nb * dim, dim, metric), nb));
            }
        }
    }
    merge();

    for (uint32_t r = 0; r < k; ++r) {  // search.cu:348-355
        if (r < itopk && top[r] != kInvalidKey) {
            out_ids[r] = (int64_t)key_id(top[r]);
            out_dists[r] = key_dist(top[r]);
        } else {
            out_ids[r] = strict ? (int64_t)0x7FFFFFFF : -1;
            out_dists[r] = kDistMax;
        }
    }
    if (ctr) *ctr = c;
}

void orc_search(const float* data, size_t n, uint32_t dim, const uint32_t* graph, uint32_t degree,
                uint32_t active_degree, const float* queries, size_t nq, uint32_t k, uint32_t itopk,
                uint32_t search_width, uint32_t max_iterations, uint32_t hash_bitlen, uint32_t n_seeds,
                const uint32_t* seeds, uint32_t n_provided, uint64_t rand_xor_mask, int metric,
                int filter_kind, const uint64_t* ts, const uint64_t* win_start, const uint64_t* win_end,
                int per_query_window, const uint8_t* labels, const uint64_t* masks, uint32_t flags,
                int64_t* out_ids, float* out_dists, orc_counters* counters, int threads) {
#pragma omp parallel num_threads(nthreads(threads))
    {
        std::vector<uint32_t> table;
#pragma omp for schedule(dynamic, 1)
        for (long long qi = 0; qi < (long long)nq; ++qi) {
            Filter f = make_filter(filter_kind, ts, win_start, win_end, per_query_window, labels, masks, qi);
            search_one(data, n, dim, graph, degree, active_degree, queries + (size_t)qi * dim, k, itopk,
                       search_width, max_iterations, hash_bitlen, n_seeds,
                       seeds ? seeds + (size_t)qi * n_provided : nullptr, n_provided, rand_xor_mask,
                       metric, f, flags, out_ids + (size_t)qi * k, out_dists + (size_t)qi * k,
                       counters ? counters + qi : nullptr, table);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// time-partitioned graph: src/index/cagra_opt.cu:209-303 (remote edges), :457-600 (reverse
// injection), :739-907 (drivers), :928-1106 (local phase)
// ---------------------------------------------------------------------------------------------
// cagra_opt.cu:808-810
uint32_t orc_remote_global_k(uint32_t total_degree, uint32_t local_degree) {
    uint32_t gk = (total_degree - local_degree) * 4;
    gk = std::max(64u, (gk + 32) - (gk % 32));
    return std::min(256u, gk);
}

// cagra_opt.cu:34-41
static inline uint32_t wang_hash(uint32_t seed) {
    seed = (seed ^ 61u) ^ (seed >> 16);
    seed *= 9u;
    seed = seed ^ (seed >> 4);
    seed *= 0x27d4eb2du;
    seed = seed ^ (seed >> 15);
    return seed;
}

// update_remote_edges_kernel, cagra_opt.cu:209-303.  cand: [n, gk] global neighbours of every row,
// nearest first (the reference takes them from IVF-PQ + exact re-ranking; here they are exact).
// ts: bucket index per row, 0..B-1, non-decreasing.  Slots [local_degree, total_degree) of every
// row are overwritten as far as candidates last; the rest keeps what the local phase wrote.
void orc_remote_edges(const uint32_t* cand_in, const uint64_t* ts, size_t n, uint32_t gk, uint32_t total_degree,
                      uint32_t local_degree, uint32_t* graph) {
    const uint64_t total_buckets = ts[n - 1] + 1;
    const uint64_t span = std::max<uint64_t>(1, total_buckets / 5);
    std::vector<uint32_t> cand(gk);
    for (size_t i = 0; i < n; ++i) {
        std::copy(cand_in + i * gk, cand_in + (i + 1) * gk, cand.begin());
        uint32_t* row = graph + i * total_degree;
        const uint64_t my = ts[i];
        const uint64_t lo = my >= span ? my - span : 0;
        const uint64_t hi = my + span >= total_buckets ? total_buckets - 1 : my + span;
        int nearby = 0;
        const int nearby_max = (int)(total_degree - local_degree) / 3;
        for (uint32_t k = 0; k < gk && nearby < nearby_max; ++k) {  // other buckets within +-20 %
            const uint32_t c = cand[k];
            if (c == (uint32_t)i || c == ORC_INVALID) continue;
            if (ts[c] == my || ts[c] < lo || ts[c] > hi) continue;
            row[local_degree + nearby++] = c;
            cand[k] = ORC_INVALID;
        }
        int far = 0;
        const int far_max = (int)(total_degree - local_degree) - nearby;
        for (uint32_t k = 0; k < gk && far < far_max; ++k) {  // buckets farther away
            const uint32_t c = cand[k];
            if (c == (uint32_t)i || c == ORC_INVALID) continue;
            if (ts[c] == my || (ts[c] >= lo && ts[c] <= hi)) continue;
            row[local_degree + nearby + far++] = c;
            cand[k] = ORC_INVALID;
        }
        for (uint32_t k = 0; k < gk && far < far_max; ++k) {  // whatever other bucket is left
            const uint32_t c = cand[k];
            if (c == (uint32_t)i || c == ORC_INVALID) continue;
            if (ts[c] == my) continue;
            row[local_degree + nearby + far++] = c;
        }
    }
}

// enhance_global_connectivity, cagra_opt.cu:739-793 with kern_make_global_rev_graph (:457-483) and
// kern_inject_global_reverse_edges (:488-600).  The reference's reverse lists are in atomic arrival
// order; here: ascending source id, then slot - what a sequential run of the kernel's loop gives.
void orc_inject_reverse_remote(uint32_t* graph, size_t n, uint32_t total_degree, uint32_t local_degree) {
    const uint32_t max_rev = 32, num_remote = total_degree - local_degree;
    if (num_remote == 0) return;
    std::vector<uint32_t> rev(n * max_rev), cnt(n, 0);
    for (size_t src = 0; src < n; ++src)
        for (uint32_t k = local_degree; k < total_degree; ++k) {
            const uint32_t dst = graph[src * total_degree + k];
            if (dst != ORC_INVALID && dst < n) {
                const uint32_t pos = cnt[dst]++;
                if (pos < max_rev) rev[(size_t)dst * max_rev + pos] = (uint32_t)src;
            }
        }
    const uint32_t num_strong = num_remote / 2, num_weak = num_remote - num_strong;
    std::vector<uint32_t> cur(num_remote);
    for (size_t i = 0; i < n; ++i) {
        uint32_t* row = graph + i * total_degree;
        std::copy(row + local_degree, row + total_degree, cur.begin());
        uint32_t rc = std::min(cnt[i], max_rev);
        if (rc == 0) continue;
        uint32_t rng = wang_hash((uint32_t)i);
        for (uint32_t r = 0; r < rc; ++r) {
            const uint32_t c = rev[i * max_rev + r];
            bool exists = std::find(cur.begin(), cur.end(), c) != cur.end() ||
                          std::find(row, row + local_degree, c) != row + local_degree;
            if (exists) continue;
            bool injected = false;
            for (uint32_t w = num_strong; w < num_remote; ++w)
                if (cur[w] == ORC_INVALID) {
                    cur[w] = c;
                    injected = true;
                    break;
                }
            if (!injected && num_weak > 0) {
                rng = wang_hash(rng);
                cur[num_strong + (rng % num_weak)] = c;
            }
        }
        std::copy(cur.begin(), cur.end(), row + local_degree);
    }
}

// build_time_partitioned_graph, cagra_opt.cu:928-1106: per bucket a full-width graph from the
// bucket's own kNN (k = 2*total_degree) through prune / reverse / merge, ids shifted by the bucket's
// first row; then the remote slots are overwritten from the global neighbours and the reverse
// remote edges injected.  Rows of a bucket are contiguous; ts = bucket index.
void orc_build_time_partitioned(const float* data, size_t n, uint32_t dim, const uint64_t* ts, const size_t* bucket_sizes,
                                size_t num_buckets, uint32_t total_degree, uint32_t local_degree, int metric,
                                uint32_t* graph, int threads) {
    const uint32_t inter = total_degree * 2;
    size_t off = 0;
    for (size_t b = 0; b < num_buckets; ++b) {
        const size_t bs = bucket_sizes[b];
        if (bs == 0) continue;
        std::vector<uint32_t> knn(bs * inter), g(bs * total_degree);
        orc_knn_graph(data + off * dim, bs, dim, inter, metric, knn.data(), threads);
        orc_optimize(knn.data(), bs, inter, total_degree, g.data(), threads);
        for (size_t i = 0; i < bs * total_degree; ++i)
            graph[off * total_degree + i] = g[i] == ORC_INVALID ? ORC_INVALID : g[i] + (uint32_t)off;
        off += bs;
    }
    if (total_degree > local_degree) {
        const uint32_t gk = orc_remote_global_k(total_degree, local_degree);
        std::vector<uint32_t> cand(n * gk);
        orc_knn_graph(data, n, dim, gk, metric, cand.data(), threads);
        orc_remote_edges(cand.data(), ts, n, gk, total_degree, local_degree, graph);
        orc_inject_reverse_remote(graph, n, total_degree, local_degree);
    }
}

// ---------------------------------------------------------------------------------------------
// k-means for the two-level index (role of faiss::Clustering in src/timeStampIndex.cu:163-178):
// Lloyd iterations, k distinct initial rows drawn with splitmix64 (partial Fisher-Yates), exact
// nearest centroid with the lower id on ties, means summed in double in row order, a centroid
// without rows stays.  FAISS is absent: PARITY UNPINNED against the reference's centroids.
// ---------------------------------------------------------------------------------------------
void orc_kmeans(const float* data, size_t n, uint32_t dim, uint32_t k, uint32_t niter, uint64_t seed, float* centroids,
                int64_t* assign_out, int threads) {
    std::vector<uint32_t> perm(n);
    for (size_t i = 0; i < n; ++i) perm[i] = (uint32_t)i;
    uint64_t state = seed;
    for (uint32_t c = 0; c < k; ++c) {
        const size_t j = c + (size_t)(orc_splitmix64(&state) % (n - c));
        std::swap(perm[c], perm[j]);
        std::copy(data + (size_t)perm[c] * dim, data + (size_t)(perm[c] + 1) * dim, centroids + (size_t)c * dim);
    }
    std::vector<int64_t> assign(n);
    std::vector<float> dist(n);
    for (uint32_t it = 0; it <= niter; ++it) {
        orc_bruteforce_topk(centroids, k, dim, data, n, 1, ORC_METRIC_L2, ORC_FILTER_NONE, nullptr, nullptr, nullptr, 0, nullptr,
                            nullptr, assign.data(), dist.data(), threads);
        if (it == niter) break;
        std::vector<double> sums((size_t)k * dim, 0.0);
        std::vector<uint32_t> counts(k, 0);
        for (size_t i = 0; i < n; ++i) {
            const size_t c = (size_t)assign[i];
            counts[c]++;
            for (uint32_t d = 0; d < dim; ++d) sums[c * dim + d] += (double)data[i * dim + d];
        }
        for (uint32_t c = 0; c < k; ++c)
            if (counts[c])
                for (uint32_t d = 0; d < dim; ++d) centroids[(size_t)c * dim + d] = (float)(sums[(size_t)c * dim + d] / (double)counts[c]);
    }
    if (assign_out) std::copy(assign.begin(), assign.end(), assign_out);
}

// ---------------------------------------------------------------------------------------------
// seed sampling extension: one id per stratum of the window's id list
// ---------------------------------------------------------------------------------------------
uint64_t orc_splitmix64(uint64_t* state) {
    uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline uint64_t mix64(uint64_t x) {
    uint64_t s = x;
    return orc_splitmix64(&s);
}

void orc_sample_window_seeds(const uint64_t* sorted_ts, const uint32_t* ids_by_ts, size_t n,
                             const uint64_t* win_start, const uint64_t* win_end, size_t nq,
                             int per_query_window, uint32_t n_seeds, uint64_t seed, uint32_t* out) {
    for (size_t q = 0; q < nq; ++q) {
        uint64_t s = per_query_window ? win_start[q] : win_start[0];
        uint64_t e = per_query_window ? win_end[q] : win_end[0];
        size_t lo = std::lower_bound(sorted_ts, sorted_ts + n, s) - sorted_ts;
        size_t hi = std::lower_bound(sorted_ts, sorted_ts + n, e) - sorted_ts;
        if (hi < lo) hi = lo;
        uint64_t w = hi - lo;
        for (uint32_t i = 0; i < n_seeds; ++i) {
            uint32_t v = ORC_INVALID;
            if (w <= n_seeds) {
                if (i < w) v = ids_by_ts[lo + i];
            } else {
                uint64_t b0 = (uint64_t)i * w / n_seeds, b1 = (uint64_t)(i + 1) * w / n_seeds;
                uint64_t r = mix64(seed ^ (q * 0x100000001B3ull + i)) % (b1 - b0);
                v = ids_by_ts[lo + b0 + r];
            }
            out[q * n_seeds + i] = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// insert: src/index/cagra.cu:938-1015, src/index/insert.cu:140-440
// ---------------------------------------------------------------------------------------------
void orc_insert_batch(const float* data, uint32_t dim, size_t n_existing, size_t n_new, uint32_t* graph,
                      uint32_t degree, uint32_t itopk_param, uint32_t search_width,
                      uint32_t max_iterations, uint32_t hash_bitlen, uint64_t* rng_state, int metric,
                      uint32_t flags, int striped_sort, int threads) {
    if (n_new == 0) return;
    const uint32_t search_k = degree * 2;  // cagra.cu:951
    std::vector<int64_t> ids(n_new * search_k);
    std::vector<float> dists(n_new * search_k);
    const float* new_data = data + n_existing * dim;

    // find_near_nodes, insert.cu:140-219: searches in groups of 64 new rows
    uint32_t itopk, n_seeds, cap;
    orc_search_plan(ORC_WRAP_SEARCH, search_k, itopk_param, search_width, degree, 0, &itopk, &n_seeds, &cap);
    for (size_t off = 0; off < n_new; off += 64) {
        size_t cur = std::min<size_t>(64, n_new - off);
        uint64_t mask = orc_splitmix64(rng_state) & 0xFFFFFFFFull;
        orc_search(data, n_existing, dim, graph, degree, degree, new_data + off * dim, cur, search_k, itopk,
                   search_width, max_iterations, hash_bitlen, n_seeds, nullptr, 0, mask, metric,
                   ORC_FILTER_NONE, nullptr, nullptr, nullptr, 0, nullptr, nullptr, flags,
                   ids.data() + off * search_k, dists.data() + off * search_k, nullptr, threads);
    }
    // insert_refine_kernel_warp (insert.cu:24-72) + insert_sort_kernel (:80-133)
    const uint32_t per_lane = search_k <= 64 ? 2 : search_k <= 128 ? 4 : search_k <= 256 ? 8 : 16;
    for (size_t i = 0; i < n_new; ++i) {
        std::vector<uint64_t> v(search_k);
        for (uint32_t r = 0; r < search_k; ++r) {
            int64_t id = ids[i * search_k + r];
            float d = kDistMax;
            if (id >= 0 && id < (int64_t)n_existing)
                d = dist_metric(new_data + i * dim, data + (size_t)id * dim, dim, metric);
            // the sort carries ids as uint32 and widens them again afterwards (insert.cu:106,129)
            v[r] = ((uint64_t)ord_bits(d) << 32) | (uint32_t)id;
        }
        std::sort(v.begin(), v.end());
        for (uint32_t p = 0; p < search_k; ++p) {
            uint32_t src = p;
            if (striped_sort) {
                // striped load into a blocked network: slot p = lane + e*32 receives the
                // element of sorted rank lane*per_lane + e (insert.cu:104 vs bitonic.cuh:74);
                // ranks past search_k are the network's (FLT_MAX, 0xFFFFFFFF) padding
                uint32_t lane = p % 32, e = p / 32;
                src = lane * per_lane + e;
            }
            ids[i * search_k + p] =
                src < search_k ? (int64_t)(uint32_t)(v[src] & 0xFFFFFFFFull) : (int64_t)ORC_INVALID;
        }
    }
    // fill_new_nodes_kernel, insert.cu:225-257
    for (size_t i = 0; i < n_new; ++i)
        for (uint32_t kk = 0; kk < degree; ++kk) {
            uint32_t v = ORC_INVALID;
            if (kk < search_k) {
                int64_t id = ids[i * search_k + kk];
                if (id >= 0 && id < (int64_t)n_existing) v = (uint32_t)id;
            }
            graph[(n_existing + i) * degree + kk] = v;
        }
    // generate_update_requests_kernel, insert.cu:263-290, then a stable sort by target
    // (thrust::sort_by_key on 32-bit keys, :422-424)
    const size_t total = n_new * search_k;
    std::vector<std::pair<uint32_t, uint32_t>> req(total);
    for (size_t t = 0; t < total; ++t) {
        int64_t id = ids[t];
        if (id >= 0 && id < (int64_t)n_existing)
            req[t] = {(uint32_t)id, (uint32_t)(n_existing + t / search_k)};
        else
            req[t] = {ORC_INVALID, ORC_INVALID};
    }
    std::stable_sort(req.begin(), req.end(),
                     [](const std::pair<uint32_t, uint32_t>& x, const std::pair<uint32_t, uint32_t>& y) {
                         return x.first < y.first;
                     });
    // apply_topology_updates_kernel, insert.cu:296-368
    for (size_t tid = 0; tid < total; ++tid) {
        uint32_t target = req[tid].first;
        if (target == ORC_INVALID) continue;
        if (tid != 0 && req[tid - 1].first == target) continue;  // not the leader
        uint32_t* nb = graph + (size_t)target * degree;
        const uint32_t num_protected = degree / 2, num_unprotected = degree - num_protected;
        uint64_t rng = (uint64_t)target * 0x9e3779b97f4a7c15ull + (uint64_t)tid;
        for (size_t idx = tid; idx < total && req[idx].first == target; ++idx) {
            uint32_t nid = req[idx].second;
            bool exists = false;
            for (uint32_t x = 0; x < degree; ++x)
                if (nb[x] == nid) {
                    exists = true;
                    break;
                }
            if (exists) continue;
            rng = rng * 6364136223846793005ull + 1;
            uint32_t r1 = (uint32_t)(rng >> 32);
            bool upd_protected = (r1 % 10 == 0);
            rng = rng * 6364136223846793005ull + 1;
            uint32_t r2 = (uint32_t)(rng >> 32);
            uint32_t slot = upd_protected ? (r2 % num_protected) : num_protected + (r2 % num_unprotected);
            nb[slot] = nid;
        }
    }
    (void)threads;
}

// ---------------------------------------------------------------------------------------------
// insert into the time-partitioned graph: src/index/cagra_opt.cu:1674-1981,
// src/index/insert.cu:444-727, :1398-1529 (the v1 branch, which is the one compiled in)
// ---------------------------------------------------------------------------------------------
// brute-force neighbours inside the batch (cagra_opt.cu:1847-1915) merged into the bucket search's
// list (merge_topk_kernel, :1475-1527): both lists ordered by (distance, id), ties included
void orc_merge_batch_neighbours(const float* new_data, size_t n_new, uint32_t dim, size_t n_existing, uint32_t search_k,
                                int metric, int64_t* local_ids, const float* local_dists) {
    const size_t tmp_size = std::min<size_t>(n_new, search_k / 2);  // :1853
    for (size_t i = 0; i < n_new; ++i) {
        std::vector<uint64_t> batch(n_new);
        for (size_t j = 0; j < n_new; ++j)
            batch[j] = ((uint64_t)ord_bits(dist_metric(new_data + i * dim, new_data + j * dim, dim, metric)) << 32) |
                       (uint32_t)(n_existing + j);  // add_offset_kernel, :1890-1896
        std::sort(batch.begin(), batch.end());
        std::vector<uint64_t> all(batch.begin(), batch.begin() + tmp_size);
        for (uint32_t r = 0; r < search_k; ++r) {
            const int64_t id = local_ids[i * search_k + r];
            if (id < 0 || id >= (int64_t)n_existing) continue;  // an empty result slot
            all.push_back(((uint64_t)ord_bits(local_dists[i * search_k + r]) << 32) | (uint32_t)id);
        }
        std::sort(all.begin(), all.end());
        for (uint32_t r = 0; r < search_k; ++r)
            local_ids[i * search_k + r] = r < all.size() ? (int64_t)(uint32_t)(all[r] & 0xFFFFFFFFull) : -1;
    }
}

// update_topology_gpu_opt with use_v1 (insert.cu:1398-1529).  local_ids / global_ids are consumed
// (used entries become -1, as in the reference).  Mailboxes list their requests by ascending
// (new row, slot) where the reference has atomic arrival order.  Ids outside the graph count as
// empty result slots (the reference reads the timestamp array out of bounds for them).
void orc_insert_partitioned_update(uint32_t* graph, const uint64_t* ts, int64_t* local_ids, int64_t* global_ids,
                                   size_t n_existing, size_t n_new, uint64_t target_ts, uint32_t total_degree,
                                   uint32_t local_degree, uint32_t search_k) {
    const int64_t n_total = (int64_t)(n_existing + n_new);
    // fill_new_nodes_kernel_opt, insert.cu:444-566
    for (size_t t = 0; t < n_new; ++t) {
        const uint32_t me = (uint32_t)(n_existing + t);
        const uint64_t my_ts = ts[me];
        uint32_t* row = graph + (size_t)me * total_degree;
        int64_t* lc = local_ids + t * search_k;
        int64_t* gc = global_ids + t * search_k;
        for (uint32_t x = 0; x < total_degree; ++x) row[x] = ORC_INVALID;  // the reference leaves what the fresh mapping holds
        uint32_t filled = 0;
        for (uint32_t k = 0; k < search_k && filled < local_degree; ++k) {  // :471-507
            const int64_t c = lc[k];
            if (c < 0 || c >= n_total || c >= 0x7fffffff) continue;
            if ((uint32_t)c == me) continue;
            if (ts[c] != my_ts) continue;
            row[filled++] = (uint32_t)c;
            lc[k] = -1;
        }
        for (uint32_t k = 0; k < search_k && filled < local_degree; ++k) {  // :510-522
            const int64_t c = lc[k];
            if (c < 0 || c >= n_total) continue;
            if ((uint32_t)c == me) continue;
            if (ts[c] != my_ts) continue;
            row[filled++] = (uint32_t)c;
            lc[k] = -1;
        }
        uint32_t filled_remote = 0;
        const uint32_t max_remote = total_degree - local_degree;
        for (uint32_t k = 0; k < search_k && filled_remote < max_remote; ++k) {  // :528-553
            const int64_t c = gc[k];
            if (c < 0 || c >= n_total) continue;
            if ((uint32_t)c == me) continue;
            bool in_local = false;
            for (uint32_t x = 0; x < local_degree; ++x)
                if (row[x] == (uint32_t)c) {
                    in_local = true;
                    break;
                }
            if (in_local) continue;
            if (ts[c] != my_ts) {
                row[local_degree + filled_remote++] = (uint32_t)c;
                gc[k] = -1;
            }
        }
        for (uint32_t k = 0; k < search_k && filled_remote < max_remote; ++k) {  // :556-565
            const int64_t c = gc[k];
            if (c < 0 || c >= n_total) continue;
            if ((uint32_t)c == me) continue;
            row[local_degree + filled_remote++] = (uint32_t)c;
            gc[k] = -1;
        }
    }
    // generate_update_requests_kernel_opt, insert.cu:568-635
    const uint32_t local_max = local_degree / 2, remote_max = (total_degree - local_degree) / 2;  // :1470-1471
    std::vector<std::vector<uint32_t>> local_box(n_existing), remote_box(n_existing);
    for (size_t t = 0; t < n_new; ++t) {
        const uint32_t src = (uint32_t)(n_existing + t);
        for (uint32_t i = 0; i < total_degree; ++i) {
            const uint32_t dest = graph[(size_t)src * total_degree + i];
            if (dest == ORC_INVALID || (int64_t)dest >= n_total) continue;
            if (i >= local_degree && ts[dest] == target_ts) continue;  // :626-628
            if (dest >= n_existing) continue;  // counted by the reference, never applied (:654)
            std::vector<uint32_t>& box = i < local_degree ? local_box[dest] : remote_box[dest];
            if (box.size() < (i < local_degree ? local_max : remote_max)) box.push_back(src);
        }
    }
    // apply_topology_updates_kernel_opt, insert.cu:637-727
    for (size_t tid = 0; tid < n_existing; ++tid) {
        uint32_t* row = graph + tid * total_degree;
        uint32_t rng = wang_hash((uint32_t)tid);
        const uint32_t local_half = local_degree / 2;
        for (uint32_t cand : local_box[tid]) {
            rng = wang_hash(rng);
            const bool strong = (rng % 100) < 10;
            const uint32_t start = strong ? 0 : local_half, len = strong ? local_half : local_degree - local_half;
            if (len > 0) {
                rng = wang_hash(rng);
                row[start + rng % len] = cand;
            }
        }
        const uint32_t remote_degree = total_degree - local_degree;
        for (uint32_t cand : remote_box[tid]) {
            const int64_t mine = (int64_t)ts[tid], theirs = (int64_t)ts[cand];
            const bool nearby = theirs >= mine - 20 && theirs <= mine + 20;  // :706
            const uint32_t near_len = remote_degree / 3;
            const uint32_t start = nearby ? local_degree : local_degree + near_len;
            const uint32_t len = nearby ? near_len : remote_degree - near_len;
            if (len > 0) {
                rng = wang_hash(rng);
                row[start + rng % len] = cand;
            }
        }
    }
}

// cagra::insert of the partitioned index, src/index/cagra_opt.cu:1674-1981
void orc_insert_partitioned_batch(const float* data, uint32_t dim, const uint64_t* ts, size_t n_existing, size_t n_new,
                                  uint64_t target_ts, uint32_t* graph, uint32_t total_degree, uint32_t local_degree,
                                  const uint32_t* seeds, uint32_t n_seeds_per_query, uint32_t itopk_param,
                                  uint32_t search_width, uint32_t max_iterations, uint32_t hash_bitlen,
                                  uint64_t* rng_state, int metric, uint32_t flags, int threads) {
    if (n_new == 0) return;
    const uint32_t search_k = itopk_param;  // :1693
    const float* new_data = data + n_existing * dim;
    std::vector<int64_t> gi(n_new * search_k), li(n_new * search_k);
    std::vector<float> gd(n_new * search_k), ld(n_new * search_k);
    uint32_t itopk, n_seeds, cap;
    const uint64_t mask_global = orc_splitmix64(rng_state) & 0xFFFFFFFFull;
    const uint64_t mask_local = orc_splitmix64(rng_state) & 0xFFFFFFFFull;
    orc_search_plan(ORC_WRAP_SEARCH_OPT, search_k, itopk_param, search_width, total_degree, 0, &itopk, &n_seeds, &cap);
    orc_search(data, n_existing, dim, graph, total_degree, total_degree, new_data, n_new, search_k, itopk, search_width,
               max_iterations, hash_bitlen, n_seeds, nullptr, 0, mask_global, metric, ORC_FILTER_NONE, nullptr, nullptr,
               nullptr, 0, nullptr, nullptr, flags, gi.data(), gd.data(), nullptr, threads);
    orc_search_plan(ORC_WRAP_BUCKET, search_k, itopk_param, search_width, total_degree, n_seeds_per_query, &itopk, &n_seeds,
                    &cap);
    orc_search(data, n_existing, dim, graph, total_degree, local_degree, new_data, n_new, search_k, itopk, search_width,
               max_iterations, hash_bitlen, n_seeds, seeds, n_seeds_per_query, mask_local, metric, ORC_FILTER_NONE, nullptr,
               nullptr, nullptr, 0, nullptr, nullptr, flags, li.data(), ld.data(), nullptr, threads);
    orc_merge_batch_neighbours(new_data, n_new, dim, n_existing, search_k, metric, li.data(), ld.data());
    orc_insert_partitioned_update(graph, ts, li.data(), gi.data(), n_existing, n_new, target_ts, total_degree, local_degree,
                                  search_k);
}

}  // extern "C"
