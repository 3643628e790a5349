// CAGRA graph optimisation on the device: detour counting + rank-based pruning, reverse
// graph, interleaved merge.  Restates optimize_prune / optimize_create_reverse_graph /
// optimize_merge_graphs (src/index/cagra.cu:286-401, :455-548, :574-650), which in the
// reference bounce between GPU kernels, host OpenMP loops and PCIe copies; here the graph
// never leaves device memory.
#include <algorithm>

#include "common.hpp"
#include "device_utils.hpp"
#include "graph_internal.hpp"

namespace grab {
using namespace dev;
namespace {

constexpr uint64_t kEmptySlot = ~0ull;

// ---------------------------------------------------------------------------------------------
// Detour counts and pruning.  One wave per node A.
//
// kern_prune (cagra.cu:219-276) walks, for each neighbour D = row[kAD] (kAD < deg-1, D valid),
// every entry Bc of D's row and scans A's row from kAD+1 for the first position holding Bc,
// whose count it increments.  Here A's row is put into an LDS hash table id -> first
// position, so the scan becomes one probe; if that first position is not after kAD the
// (rare: duplicate ids in a row) linear scan is done as written.
// ---------------------------------------------------------------------------------------------
// Nearly all lookups miss (a neighbour's neighbour is rarely A's neighbour too), and a miss in the table walks to
// the next free slot, as long as the longest walk among the wave's 64 lanes.  So a bit set of 8192 bits over the
// row's ids answers first: one LDS read, no loop, and only the few ids whose bit is set go to the table.
template <int MAXDEG>
struct PruneLds {
    static constexpr uint32_t kSlots = MAXDEG <= 256 ? 4 * MAXDEG : 2 * MAXDEG;  // a quarter full (half at 512: LDS)
    uint64_t table[4][kSlots];  // (id << 32 | first position), kEmptySlot when free
    uint32_t bits[4][256];      // bit (id * 0x9E3779B1) >> 19 is set for every id of the row
    uint32_t row[4][MAXDEG];
    uint32_t cnt[4][MAXDEG];
};

template <int MAXDEG, bool SELECT>
__global__ void __launch_bounds__(256) prune_kernel(const uint32_t* __restrict__ knn, uint32_t n, uint32_t deg,
                                                    uint32_t out_deg, uint8_t* __restrict__ counts_out,
                                                    uint32_t* __restrict__ graph_out) {
    __shared__ PruneLds<MAXDEG> s;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t a = blockIdx.x * 4 + wave;
    if (a >= n) return;  // wave-uniform; no workgroup barrier is used below
    uint64_t* table = s.table[wave];
    uint32_t* row = s.row[wave];
    uint32_t* cnt = s.cnt[wave];
    uint32_t* bits = s.bits[wave];
    constexpr uint32_t mask = PruneLds<MAXDEG>::kSlots - 1;

    for (uint32_t i = lane; i < PruneLds<MAXDEG>::kSlots; i += 64) table[i] = kEmptySlot;
    for (uint32_t i = lane; i < 256; i += 64) bits[i] = 0;
    for (uint32_t p = lane; p < deg; p += 64) {
        row[p] = knn[(size_t)a * deg + p];
        cnt[p] = 0;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    bool saw_duplicate = false;
    for (uint32_t p = lane; p < deg; p += 64) {
        const uint32_t id = row[p];
        const uint64_t packed = ((uint64_t)id << 32) | p;
        const uint32_t hb = (id * 0x9E3779B1u) >> 19;
        atomicOr(&bits[hb >> 5], 1u << (hb & 31u));
        uint32_t h = (id * 2654435761u) & mask;
        for (uint32_t i = 0; i <= mask; ++i) {
            uint64_t cur = atomicCAS(reinterpret_cast<unsigned long long*>(&table[h]), kEmptySlot, packed);
            if (cur == kEmptySlot) break;
            if ((uint32_t)(cur >> 32) == id) {
                atomicMin(reinterpret_cast<unsigned long long*>(&table[h]), packed);
                saw_duplicate = true;
                break;
            }
            h = (h + 1) & mask;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // an id that occurs once in A's row has no position after its first one: the scan of
    // cagra.cu:262-271 can only find something when the row holds an id twice (padding included)
    const bool row_has_duplicates = __ballot(saw_duplicate) != 0;

    // eight D rows per round: their reads are in flight together, and so are the eight reads of the bit set
    constexpr int U = 8;
    for (uint32_t k0 = 0; k0 + 1 < deg; k0 += U) {
        uint32_t dnode[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t kAD = k0 + u;
            dnode[u] = (kAD + 1 < deg) ? row[kAD] : kInvalidId;
            if (dnode[u] >= n) dnode[u] = kInvalidId;  // padding, or an id the reference would read out of bounds
        }
        for (uint32_t kDB = lane; kDB < deg; kDB += 64) {
            uint32_t bc[U], w[U];
#pragma unroll
            for (int u = 0; u < U; ++u) bc[u] = dnode[u] != kInvalidId ? knn[(size_t)dnode[u] * deg + kDB] : 0u;
#pragma unroll
            for (int u = 0; u < U; ++u) w[u] = bits[((bc[u] * 0x9E3779B1u) >> 19) >> 5];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (dnode[u] == kInvalidId) continue;
                if (!((w[u] >> (((bc[u] * 0x9E3779B1u) >> 19) & 31u)) & 1u)) continue;  // not an id of the row
                const uint32_t kAD = k0 + u;
                // first position of the id in the row, if the table holds it
                uint32_t p = 0xFFFFFFFFu, hh = (bc[u] * 2654435761u) & mask;
                uint64_t ee = table[hh];
                for (uint32_t i = 0; i <= mask; ++i) {
                    if (ee == kEmptySlot) break;
                    if ((uint32_t)(ee >> 32) == bc[u]) {
                        p = (uint32_t)(ee & 0xFFFFFFFFull);
                        break;
                    }
                    hh = (hh + 1) & mask;
                    ee = table[hh];
                }
                if (p == 0xFFFFFFFFu) continue;
                if (p <= kAD) {  // cagra.cu:262-271 as written
                    if (!row_has_duplicates) continue;
                    p = 0xFFFFFFFFu;
                    for (uint32_t kAB = kAD + 1; kAB < deg; ++kAB)
                        if (row[kAB] == bc[u]) {
                            p = kAB;
                            break;
                        }
                    if (p == 0xFFFFFFFFu) continue;
                }
                atomicAdd(&cnt[p], 1u);
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    if (!SELECT) {
        for (uint32_t p = lane; p < deg; p += 64) counts_out[(size_t)a * deg + p] = cnt[p] > 255u ? 255u : (uint8_t)cnt[p];
        return;
    }
    // cagra.cu:274,381-391: counts saturate at 255, positions are ordered by a stable sort on
    // the count and the first out_deg are kept
    for (uint32_t p = lane; p < deg; p += 64) {
        const uint32_t c = cnt[p] > 255u ? 255u : cnt[p];
        uint32_t rank = 0;
        for (uint32_t x = 0; x < deg; ++x) {
            const uint32_t cx = cnt[x] > 255u ? 255u : cnt[x];
            rank += (cx < c || (cx == c && x < p)) ? 1u : 0u;
        }
        if (rank < out_deg) graph_out[(size_t)a * out_deg + rank] = row[p];
    }
}

// ---------------------------------------------------------------------------------------------
// Reverse graph.  kern_make_rev_graph (cagra.cu:418-444) is launched once per column and
// appends sources in atomic arrival order; a sequential execution gives "column by column,
// ascending source", which is what this builds deterministically: count in-degrees, scan,
// scatter keys column*n+source into per-destination segments, keep the `deg` smallest sorted.
// ---------------------------------------------------------------------------------------------
// columns [col_lo, col_lo + width) of the graph take part
__global__ void __launch_bounds__(256) indegree_kernel(const uint32_t* __restrict__ g, uint32_t n, uint32_t deg, uint32_t col_lo,
                                                       uint32_t width, uint32_t* __restrict__ indeg) {
    const size_t total = (size_t)n * width;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
        const uint32_t src = (uint32_t)(e / width), k = (uint32_t)(e - (size_t)src * width);
        const uint32_t dest = g[(size_t)src * deg + col_lo + k];
        if (dest < n) atomicAdd(&indeg[dest], 1u);
    }
}

// exclusive scan of n uint32 in three steps: per-block sums, scan of the block sums by one
// block, per-block scan with the block's base
constexpr int kScanBlock = 1024;
__global__ void __launch_bounds__(256) block_sums_kernel(const uint32_t* __restrict__ in, uint32_t n, uint32_t* __restrict__ sums) {
    __shared__ uint32_t red[256];
    const uint32_t base = blockIdx.x * kScanBlock;
    uint32_t v = 0;
    for (int i = 0; i < 4; ++i) {
        const uint32_t idx = base + threadIdx.x * 4 + i;
        if (idx < n) v += in[idx];
    }
    red[threadIdx.x] = v;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if ((int)threadIdx.x < st) red[threadIdx.x] += red[threadIdx.x + st];
        __syncthreads();
    }
    if (threadIdx.x == 0) sums[blockIdx.x] = red[0];
}
__global__ void __launch_bounds__(256) scan_sums_kernel(uint32_t* sums, uint32_t nblocks) {
    // single block, sequential over chunks of 256 with a running carry
    __shared__ uint32_t tmp[256];
    __shared__ uint32_t carry;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    for (uint32_t base = 0; base < nblocks; base += 256) {
        const uint32_t idx = base + threadIdx.x;
        const uint32_t v = idx < nblocks ? sums[idx] : 0;
        tmp[threadIdx.x] = v;
        __syncthreads();
        for (int off = 1; off < 256; off <<= 1) {
            const uint32_t add = (int)threadIdx.x >= off ? tmp[threadIdx.x - off] : 0;
            __syncthreads();
            tmp[threadIdx.x] += add;
            __syncthreads();
        }
        const uint32_t incl = tmp[threadIdx.x];
        if (idx < nblocks) sums[idx] = carry + incl - v;
        __syncthreads();
        if (threadIdx.x == 255) carry += incl;
        __syncthreads();
    }
}
__global__ void __launch_bounds__(256) block_scan_kernel(const uint32_t* __restrict__ in, uint32_t n,
                                                         const uint32_t* __restrict__ sums, uint32_t* __restrict__ out) {
    __shared__ uint32_t tmp[256];
    const uint32_t base = blockIdx.x * kScanBlock;
    uint32_t v[4], local = 0;
    for (int i = 0; i < 4; ++i) {
        const uint32_t idx = base + threadIdx.x * 4 + i;
        v[i] = idx < n ? in[idx] : 0;
        local += v[i];
    }
    tmp[threadIdx.x] = local;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        const uint32_t add = (int)threadIdx.x >= off ? tmp[threadIdx.x - off] : 0;
        __syncthreads();
        tmp[threadIdx.x] += add;
        __syncthreads();
    }
    uint32_t run = sums[blockIdx.x] + tmp[threadIdx.x] - local;
    for (int i = 0; i < 4; ++i) {
        const uint32_t idx = base + threadIdx.x * 4 + i;
        if (idx < n) out[idx] = run;
        run += v[i];
    }
}

__global__ void __launch_bounds__(256) scatter_rev_kernel(const uint32_t* __restrict__ g, uint32_t n, uint32_t deg, uint32_t col_lo,
                                                          uint32_t width, int by_source, const uint32_t* __restrict__ offsets,
                                                          uint32_t* __restrict__ cursor, uint32_t* __restrict__ csr) {
    const size_t total = (size_t)n * width;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (size_t)gridDim.x * 256) {
        const uint32_t src = (uint32_t)(e / width), k = (uint32_t)(e - (size_t)src * width);
        const uint32_t dest = g[(size_t)src * deg + col_lo + k];
        if (dest >= n) continue;
        const uint32_t pos = atomicAdd(&cursor[dest], 1u);
        // the key orders the sources of a destination: by (column, source), or by (source, column)
        csr[offsets[dest] + pos] = by_source ? src * width + k : k * n + src;
    }
}

// one wave per destination: the `deg` smallest keys of its segment, ascending
template <int NPL>
__global__ void __launch_bounds__(256) select_rev_kernel(const uint32_t* __restrict__ csr, const uint32_t* __restrict__ offsets,
                                                         const uint32_t* __restrict__ indeg, uint32_t n, uint32_t deg,
                                                         uint32_t width, int by_source, uint32_t* __restrict__ rev) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t dest = blockIdx.x * 4 + wave;
    if (dest >= n) return;
    const uint32_t m = indeg[dest];
    const uint32_t* seg = csr + offsets[dest];
    constexpr uint32_t TOTAL = 64 * NPL;
    const uint32_t chunk = TOTAL - deg;  // deg <= TOTAL/2
    uint64_t k[NPL];
#pragma unroll
    for (int i = 0; i < NPL; ++i) k[i] = kInvalidKey;
    for (uint32_t done = 0; done < m; done += chunk) {
#pragma unroll
        for (int i = 0; i < NPL; ++i) {
            const uint32_t g = lane * NPL + i;
            if (g >= deg) {
                const uint32_t src = done + (g - deg);
                k[i] = src < m ? (uint64_t)seg[src] : kInvalidKey;
            }
        }
        wave_bitonic_sort<NPL>(k);
    }
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        const uint32_t g = lane * NPL + i;
        if (g < deg)
            rev[(size_t)dest * deg + g] = k[i] == kInvalidKey ? kInvalidId : by_source ? (uint32_t)(k[i] / width) : (uint32_t)(k[i] % n);
    }
}

// ---------------------------------------------------------------------------------------------
// Merge.  optimize_merge_graphs (cagra.cu:574-650) is sequential per node; one wave runs
// that sequence with uniform control flow and answers "already accepted?" with one ballot.
// ---------------------------------------------------------------------------------------------
template <int MAXDEG>
__global__ void __launch_bounds__(256) merge_kernel(uint32_t* __restrict__ graph, const uint32_t* __restrict__ rev,
                                                    const uint32_t* __restrict__ rev_counts, uint32_t n, uint32_t deg) {
    __shared__ uint32_t fwd_s[4][MAXDEG], rev_s[4][MAXDEG], acc_s[4][MAXDEG];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t j = blockIdx.x * 4 + wave;
    if (j >= n) return;
    uint32_t* fwd = fwd_s[wave];
    uint32_t* rv = rev_s[wave];
    uint32_t* acc = acc_s[wave];
    for (uint32_t p = lane; p < deg; p += 64) {
        fwd[p] = graph[(size_t)j * deg + p];
        rv[p] = rev[(size_t)j * deg + p];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const uint32_t rev_count = min(rev_counts[j], deg);
    uint32_t count = 0, cf = 0, cr = 0;
    auto is_dup = [&](uint32_t c) -> bool {
        bool hit = false;
        for (uint32_t p = lane; p < count; p += 64) hit = hit || (acc[p] == c);
        return __ballot(hit) != 0;
    };
    auto accept = [&](uint32_t c) {
        if (lane == 0) acc[count] = c;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        ++count;
    };
    while (count < deg) {
        bool added = false;
        while (cf < deg) {
            const uint32_t c = fwd[cf++];
            if (c == j) continue;
            if (is_dup(c)) continue;
            accept(c);
            added = true;
            break;
        }
        if (count >= deg) break;
        while (cr < rev_count) {
            const uint32_t c = rv[cr++];
            if (c >= n) continue;
            if (c == j) continue;
            if (is_dup(c)) continue;
            accept(c);
            added = true;
            break;
        }
        if (!added) break;
    }
    // only the accepted prefix is written; the tail keeps its old value (cagra.cu:645-648)
    for (uint32_t p = lane; p < count; p += 64) graph[(size_t)j * deg + p] = acc[p];
}

int check_graph_args(size_t n, uint32_t deg) {
    GRAB_REQUIRE(n > 0 && n < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(deg >= 1 && deg <= GRAB_MAX_DEGREE, "Input degree too large for prune kernel (max 512).");
    return GRAB_OK;
}

int run_prune(const uint32_t* knn, size_t n, uint32_t deg, uint32_t out_deg, uint8_t* counts, uint32_t* out, hipStream_t st) {
    const uint32_t nn = (uint32_t)n, grid = (nn + 3) / 4;
#define GRAB_PRUNE(MD)                                                                                          \
    if (counts) hipLaunchKernelGGL((prune_kernel<MD, false>), dim3(grid), dim3(256), 0, st, knn, nn, deg, out_deg, counts, out); \
    else hipLaunchKernelGGL((prune_kernel<MD, true>), dim3(grid), dim3(256), 0, st, knn, nn, deg, out_deg, counts, out);
    if (deg <= 64) { GRAB_PRUNE(64) }
    else if (deg <= 128) { GRAB_PRUNE(128) }
    else if (deg <= 256) { GRAB_PRUNE(256) }
    else { GRAB_PRUNE(512) }
#undef GRAB_PRUNE
    GRAB_HIP(hipGetLastError());
    return GRAB_OK;
}

}  // namespace

// Reverse lists of the columns [col_lo, col_lo + width) of a graph: for every destination its first
// `cap` sources in the order (column, source) or (source, column), and the full in-degree.
int reverse_lists(const uint32_t* d_graph, size_t num_dataset, uint32_t degree, uint32_t col_lo, uint32_t width, int by_source,
                  uint32_t cap, uint32_t* d_rev, uint32_t* d_counts, hipStream_t st) {
    GRAB_REQUIRE((uint64_t)num_dataset * width < (1ull << 32), "num_dataset*degree must be below 2^32");
    GRAB_REQUIRE(cap >= 1 && cap <= 512, "reverse list width out of range");
    const uint32_t n = (uint32_t)num_dataset;
    const size_t edges = (size_t)n * width;
    const uint32_t nblocks = (n + kScanBlock - 1) / kScanBlock;
    DeviceScratch offsets, cursor, sums, csr;
    GRAB_HIP(offsets.alloc((size_t)n * 4));
    GRAB_HIP(cursor.alloc((size_t)n * 4));
    GRAB_HIP(sums.alloc((size_t)nblocks * 4));
    GRAB_HIP(csr.alloc(std::max<size_t>(edges, 1) * 4));
    GRAB_HIP(hipMemsetAsync(d_counts, 0, (size_t)n * 4, st));
    GRAB_HIP(hipMemsetAsync(cursor.ptr, 0, (size_t)n * 4, st));
    const uint32_t egrid = (uint32_t)std::min<size_t>((edges + 255) / 256, 65536);
    hipLaunchKernelGGL(indegree_kernel, dim3(egrid), dim3(256), 0, st, d_graph, n, degree, col_lo, width, d_counts);
    hipLaunchKernelGGL(block_sums_kernel, dim3(nblocks), dim3(256), 0, st, d_counts, n, sums.as<uint32_t>());
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(256), 0, st, sums.as<uint32_t>(), nblocks);
    hipLaunchKernelGGL(block_scan_kernel, dim3(nblocks), dim3(256), 0, st, d_counts, n, sums.as<uint32_t>(), offsets.as<uint32_t>());
    hipLaunchKernelGGL(scatter_rev_kernel, dim3(egrid), dim3(256), 0, st, d_graph, n, degree, col_lo, width, by_source,
                       offsets.as<uint32_t>(), cursor.as<uint32_t>(), csr.as<uint32_t>());
    const uint32_t sgrid = (n + 3) / 4;
#define GRAB_SEL(NPL) \
    hipLaunchKernelGGL(select_rev_kernel<NPL>, dim3(sgrid), dim3(256), 0, st, csr.as<uint32_t>(), offsets.as<uint32_t>(), d_counts, n, \
                       cap, width, by_source, d_rev)
    if (cap <= 64) GRAB_SEL(2);
    else if (cap <= 128) GRAB_SEL(4);
    else if (cap <= 256) GRAB_SEL(8);
    else GRAB_SEL(16);
#undef GRAB_SEL
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));  // the scratch buffers go out of scope
    return GRAB_OK;
}

}  // namespace grab

using namespace grab;

extern "C" {

int grab_detour_counts(const uint32_t* d_knn_graph, uint8_t* d_counts, size_t num_dataset, uint32_t degree, void* stream) {
    GRAB_REQUIRE(d_knn_graph && d_counts, "null pointer");
    GRAB_TRY(check_graph_args(num_dataset, degree));
    hipStream_t st = static_cast<hipStream_t>(stream);
    GRAB_TRY(run_prune(d_knn_graph, num_dataset, degree, degree, d_counts, nullptr, st));
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_optimize_prune(const uint32_t* d_knn_graph, uint32_t* d_new_graph, size_t num_dataset, uint32_t input_degree,
                        uint32_t output_degree, void* stream) {
    GRAB_REQUIRE(d_knn_graph && d_new_graph, "null pointer");
    GRAB_TRY(check_graph_args(num_dataset, input_degree));
    GRAB_REQUIRE(output_degree >= 1 && output_degree <= input_degree, "output degree must be in [1, input degree]");
    hipStream_t st = static_cast<hipStream_t>(stream);
    GRAB_TRY(run_prune(d_knn_graph, num_dataset, input_degree, output_degree, nullptr, d_new_graph, st));
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_optimize_create_reverse_graph(const uint32_t* d_input_graph, uint32_t* d_rev_graph, uint32_t* d_rev_counts,
                                       size_t num_dataset, uint32_t degree, void* stream) {
    GRAB_REQUIRE(d_input_graph && d_rev_graph && d_rev_counts, "null pointer");
    GRAB_TRY(check_graph_args(num_dataset, degree));
    hipStream_t st = static_cast<hipStream_t>(stream);
    GRAB_TRY(grab::reverse_lists(d_input_graph, num_dataset, degree, 0, degree, 0, degree, d_rev_graph, d_rev_counts, st));
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_optimize_merge_graphs(uint32_t* d_graph, const uint32_t* d_rev_graph, const uint32_t* d_rev_counts,
                               size_t num_dataset, uint32_t degree, void* stream) {
    GRAB_REQUIRE(d_graph && d_rev_graph && d_rev_counts, "null pointer");
    GRAB_TRY(check_graph_args(num_dataset, degree));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t n = (uint32_t)num_dataset, grid = (n + 3) / 4;
    if (degree <= 64) hipLaunchKernelGGL(merge_kernel<64>, dim3(grid), dim3(256), 0, st, d_graph, d_rev_graph, d_rev_counts, n, degree);
    else if (degree <= 128) hipLaunchKernelGGL(merge_kernel<128>, dim3(grid), dim3(256), 0, st, d_graph, d_rev_graph, d_rev_counts, n, degree);
    else if (degree <= 256) hipLaunchKernelGGL(merge_kernel<256>, dim3(grid), dim3(256), 0, st, d_graph, d_rev_graph, d_rev_counts, n, degree);
    else hipLaunchKernelGGL(merge_kernel<512>, dim3(grid), dim3(256), 0, st, d_graph, d_rev_graph, d_rev_counts, n, degree);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_build_graph(const float* d_dataset, size_t num_dataset, const uint32_t* d_raw_knn_graph, grab_build_params params,
                     uint32_t* d_graph, void* stream) {
    (void)d_dataset;  // unused by the reference's build as well (src/index/cagra.cu:665-711)
    GRAB_REQUIRE(d_raw_knn_graph && d_graph, "null pointer");
    DeviceScratch rev, cnt;
    GRAB_HIP(rev.alloc(num_dataset * params.graph_degree * 4));
    GRAB_HIP(cnt.alloc(num_dataset * 4));
    GRAB_TRY(grab_optimize_prune(d_raw_knn_graph, d_graph, num_dataset, params.intermediate_degree, params.graph_degree, stream));
    GRAB_TRY(grab_optimize_create_reverse_graph(d_graph, rev.as<uint32_t>(), cnt.as<uint32_t>(), num_dataset, params.graph_degree, stream));
    GRAB_TRY(grab_optimize_merge_graphs(d_graph, rev.as<uint32_t>(), cnt.as<uint32_t>(), num_dataset, params.graph_degree, stream));
    return GRAB_OK;
}

}  // extern "C"
