// Exact top-k where a graph is the wrong tool: queries restricted to sets of buckets of a base stored bucket by bucket,
// and queries restricted to intervals of row ids (timestamp windows over rows in timestamp order).  The admitted rows
// are scanned with the contraction kernels of topk_gemm.hip; candidates are re-scored and proven as there.
#include <algorithm>
#include <cstring>
#include <functional>
#include <vector>

#include "common.hpp"
#include "device_sort.hpp"
#include "device_utils.hpp"
#include "topk_gemm.hpp"
#include "topk_internal.hpp"

// ---- exact top-k over sets of buckets, for bases stored bucket by bucket --------------------------------------
namespace grab {
using namespace dev;
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
        launch_spaced_mean(d_dataset, num_dataset, (uint32_t)std::min<size_t>(num_dataset, 8192), dim, mean_out->as<float>(), st);
        mu = mean_out->as<float>();
    }
    launch_split_rows_chunked(d_dataset, num_dataset, dim, mu, d_split, d_norm, st);
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
    void** staging = nullptr;         // page-locked host memory for a call's tables, grown as needed (null: none kept)
    size_t* staging_bytes = nullptr;
};

// what a call starts from: no row unproven yet, no largest norm yet, the work counters of its launches at zero, every
// candidate list empty (`keys` may be null)
__global__ void __launch_bounds__(256) scan_init_kernel(uint32_t* __restrict__ doubt, uint32_t nq, uint32_t counters, uint64_t* __restrict__ keys, size_t count) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i == 0) {
        doubt[0] = 0;
        doubt[nq + 1] = 0;
        doubt[nq + 2] = 0;
    }
    if (i < counters) doubt[nq + 3 + i] = 0;
    for (size_t g = i; g < count; g += (size_t)gridDim.x * 256) keys[g] = kInvalidKey;
}

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
    knn_stats().flop = knn_stats().flop_bf16 = 0.0;
    knn_stats().redone_rows = knn_stats().exact_rows = 0;
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
                            : knn_bf16_allowed() && dim % KC == 0 && rows >= 1024 && num_dataset >= 4096;
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
    // [0] rows not proven, [1..nq] which, [nq+1] max norm of the base rows, from [nq+3] a work counter per launch
    const uint32_t n_counters = (uint32_t)std::min<size_t>(passes.size() + 1, 256);
    GRAB_HIP(doubt.alloc(((size_t)nq + 3 + n_counters) * 4));
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
    {
        // a prepared base keeps page-locked memory for the tables: the upload is queued and the host goes on (from
        // pageable memory the call waits for the copy)
        const void* src = tab.data();
        if (base && base->staging) {
            if (*base->staging_bytes < tab.size() * 4) {
                if (*base->staging) (void)hipHostFree(*base->staging);
                *base->staging = nullptr;
                *base->staging_bytes = 0;
                const size_t want = tab.size() * 4 + tab.size() + 4096;
                if (hipHostMalloc(base->staging, want, hipHostMallocDefault) == hipSuccess) *base->staging_bytes = want;
                else (void)hipGetLastError();
            }
            if (*base->staging) {
                std::memcpy(*base->staging, tab.data(), tab.size() * 4);
                src = *base->staging;
            }
        }
        GRAB_HIP(hipMemcpyAsync(d_tab.ptr, src, tab.size() * 4, hipMemcpyHostToDevice, st));
    }
    const uint32_t* d_rq = d_tab.as<uint32_t>() + at_rq;
    const uint32_t* d_lo = d_tab.as<uint32_t>() + at_lo;
    const uint32_t* d_hi = d_tab.as<uint32_t>() + at_hi;
    const uint32_t* d_loff = d_tab.as<uint32_t>() + at_loff;
    const uint32_t* d_lists = d_tab.as<uint32_t>() + at_lists;
    const uint32_t* d_sched_all = d_tab.as<uint32_t>() + at_sched;
    {
        const size_t fill = dense_way ? (size_t)nq * kk : 0;  // the dense way: a query without a row keeps an empty list
        hipLaunchKernelGGL(scan_init_kernel, dim3((uint32_t)std::min<size_t>(std::max<size_t>((fill + 255) / 256, 1), 1024)), dim3(256), 0, st,
                           doubt.as<uint32_t>(), nq, n_counters, merged.as<uint64_t>(), fill);
        GRAB_HIP(hipGetLastError());
    }
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
        launch_split_rows_chunked(d_queries, nq, dim, mu, split_a.as<uint16_t>(), norm_a.as<float>(), st);
        t.A = split_a.as<float>();
        t.B = base ? reinterpret_cast<const float*>(base->rows_split) : split_b.as<float>();
    } else {
        if (!base) launch_row_norms(d_dataset, num_dataset, dim, norm_b.as<float>(), st);
        launch_row_norms(d_queries, nq, dim, norm_a.as<float>(), st);
    }
    if (!base) launch_max_float(norm_b.as<float>(), num_dataset, doubt.as<uint32_t>() + nq + 1, st);
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
            tp.work_counter = pi < n_counters ? doubt.as<uint32_t>() + nq + 3 + pi : nullptr;
            rc = launch_tile_store(tp, metric, target, st, split);
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
        t.work_counter = doubt.as<uint32_t>() + nq + 3;
        rc = launch_tile_any(t, metric, kFilterColRange, grid, st, split);
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
    if (split) knn_stats().flop_bf16 = 3.0 * flop;  // three instructions a product
    else knn_stats().flop = flop;
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
    rc = launch_refine_any(r, metric, st);
    uint32_t n_doubt = 0;
    if (rc == GRAB_OK && hipMemcpyAsync(&n_doubt, doubt.ptr, 4, hipMemcpyDeviceToHost, st) != hipSuccess) rc = GRAB_ERR_HIP;
    if (hipStreamSynchronize(st) != hipSuccess && rc == GRAB_OK) rc = GRAB_ERR_HIP;
    if (rc != GRAB_OK) {
        set_error("scan: re-scoring failed");
        return rc;
    }
    knn_stats().exact_rows = n_doubt;
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
    const double flop_fp32 = knn_stats().flop, flop_bf16 = knn_stats().flop_bf16;
    GRAB_TRY(bucket_scan_by_rows(d_dataset, num_dataset, dim, sub, sub_q.as<float>(), n_doubt, k, metric, sub_ids.as<int64_t>(),
                                 sub_dist.as<float>(), st));
    knn_stats().flop = flop_fp32;  // the figures of the main pass
    knn_stats().flop_bf16 = flop_bf16;
    knn_stats().exact_rows = n_doubt;
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
    void* staging = nullptr;  // page-locked host memory for a call's tables
    size_t staging_bytes = 0;
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
    b->view.split = knn_bf16_allowed() && dim % KC == 0 && num_dataset >= 4096;
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
        launch_row_norms(d_dataset, num_dataset, dim, b->norm.as<float>(), nullptr);
    }
    if (rc != GRAB_OK) return fail(rc);
    if (hipMemsetAsync(b->max_norm.ptr, 0, 4, nullptr) != hipSuccess) return fail(GRAB_ERR_HIP);
    launch_max_float(b->norm.as<float>(), num_dataset, b->max_norm.as<uint32_t>(), nullptr);
    if (hipGetLastError() != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
        set_error("scan base: preparing the rows failed");
        return fail(GRAB_ERR_HIP);
    }
    b->view.rows_split = b->rows_split.as<uint16_t>();
    b->view.norm = b->norm.as<float>();
    b->view.mean = b->mean.as<float>();
    b->view.max_norm = b->max_norm.as<float>();
    b->view.staging = &b->staging;
    b->view.staging_bytes = &b->staging_bytes;
    *out = b;
    return GRAB_OK;
}

void grab_scan_base_destroy(grab_scan_base* b) {
    if (!b) return;
    if (b->block) (void)hipFree(b->block);
    if (b->staging) (void)hipHostFree(b->staging);
    delete b;
}

namespace {
// a scan with the calls' scratch taken from the base's block; the block follows what the call asked for (up to 8 GiB:
// beyond that, and on the first call, scratch is allocated as ever)
int scan_on_base(grab_scan_base* b, const std::function<int()>& run) {
    ScratchArena arena{static_cast<char*>(b->block), b->block_bytes, 0, 0};
    struct Lend {  // the calling thread's scratch comes from the block until this scope ends, however it ends
        ScratchArena*& slot;
        ScratchArena* const before;
        Lend(ScratchArena* a) : slot(scratch_arena()), before(slot) { slot = a; }
        ~Lend() { slot = before; }
    };
    int rc;
    {
        Lend lend(&arena);
        rc = run();  // returns with the stream drained: nothing of the block is in use any more
    }
    if (rc != GRAB_OK) (void)hipDeviceSynchronize();  // a call that gave up half way may have left kernels queued
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

}  // extern "C"
