// Time-partitioned graph: every bucket of rows (one timestamp) gets a full-width CAGRA graph of its
// own, then the last slots of every row are overwritten with "remote" edges into other buckets and
// reverse remote edges are injected.  Restates build_time_partitioned_graph,
// build_global_remote_edges and enhance_global_connectivity with their kernels
// (src/index/cagra_opt.cu:928-1106, :796-907, :739-793, :209-303, :457-600).  The reference takes
// the global candidates from FAISS IVF-PQ with exact re-ranking and bounces the per-bucket graphs
// through host memory; here candidates are exact (the MFMA contraction) and nothing leaves the device.
#include <algorithm>
#include <vector>

#include "common.hpp"
#include "device_utils.hpp"
#include "graph_internal.hpp"

namespace grab {
using namespace dev;
namespace {

// ids of a bucket's graph are local to the bucket: shift them by the bucket's first row
__global__ void __launch_bounds__(256) shift_ids_kernel(uint32_t* __restrict__ g, size_t count, uint32_t offset) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count && g[i] != kInvalidId) g[i] += offset;
}

// update_remote_edges_kernel, cagra_opt.cu:209-303.  The reference walks a row's global candidates (nearest first)
// three times with one thread: other buckets within +-20 % of the bucket range (at most a third of the remote
// slots), then buckets farther away, then whatever other bucket is left.  Here a wave takes the row: lane l holds
// candidates l, l + 64, ... (at most 256), their timestamps are gathered in one round, and a candidate's slot is the
// number of candidates of its class before it - a ballot and a popcount - which is the slot the sequential walk
// gives it.  The third pass can only meet nearby candidates that the first pass left over (it runs while remote
// slots are open, and then the second pass has taken every far candidate).
__global__ void __launch_bounds__(256) remote_edges_kernel(uint32_t* __restrict__ graph, const uint64_t* __restrict__ ts,
                                                           const uint32_t* __restrict__ cand, uint32_t n, uint32_t total_degree,
                                                           uint32_t local_degree, uint32_t gk) {
    const int lane = threadIdx.x & 63;
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n) return;  // wave-uniform
    uint32_t* row = graph + (size_t)i * total_degree;
    const uint32_t* c = cand + (size_t)i * gk;
    const uint64_t my = ts[i];
    const uint64_t total_buckets = ts[n - 1] + 1;
    const uint64_t span = total_buckets / 5 > 1 ? total_buckets / 5 : 1;
    const uint64_t lo = my >= span ? my - span : 0;
    const uint64_t hi = my + span >= total_buckets ? total_buckets - 1 : my + span;
    const uint32_t remote = total_degree - local_degree, nearby_max = remote / 3;
    uint32_t id[4];
    bool near[4], far[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t k = 64u * j + lane;
        id[j] = k < gk ? c[k] : kInvalidId;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const bool valid = id[j] != i && id[j] < n;
        const uint64_t t = valid ? ts[id[j]] : my;
        const bool other = valid && t != my;
        near[j] = other && t >= lo && t <= hi;
        far[j] = other && !near[j];
    }
    const uint64_t below = (1ull << lane) - 1ull;
    uint32_t near_before[4], far_before[4], n_near = 0, n_far = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint64_t bn = __ballot(near[j]), bf = __ballot(far[j]);
        near_before[j] = n_near + (uint32_t)__popcll(bn & below);
        far_before[j] = n_far + (uint32_t)__popcll(bf & below);
        n_near += (uint32_t)__popcll(bn);
        n_far += (uint32_t)__popcll(bf);
    }
    const uint32_t nearby = min(n_near, nearby_max), far_max = remote - nearby, taken_far = min(n_far, far_max);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (near[j]) {
            if (near_before[j] < nearby_max) {
                row[local_degree + near_before[j]] = id[j];
            } else {  // left over by the first pass: the third pass takes it while slots are open
                const uint32_t at = taken_far + (near_before[j] - nearby_max);
                if (at < far_max) row[local_degree + nearby + at] = id[j];
            }
        } else if (far[j] && far_before[j] < far_max) {
            row[local_degree + nearby + far_before[j]] = id[j];
        }
    }
}

// cagra_opt.cu:34-41
__device__ __forceinline__ uint32_t wang_hash(uint32_t seed) {
    seed = (seed ^ 61u) ^ (seed >> 16);
    seed *= 9u;
    seed = seed ^ (seed >> 4);
    seed *= 0x27d4eb2du;
    seed = seed ^ (seed >> 15);
    return seed;
}

// kern_inject_global_reverse_edges, cagra_opt.cu:488-600: the sources that point at a row through a
// remote slot go into the weak half of the row's remote slots - an empty slot first, else a slot
// drawn with wang_hash - unless the row already has them.  A wave takes the row, slot x in lane x % 64 (up to eight
// registers a lane); the sources are taken one after the other as in the reference (each sees what the ones before
// it did to the row), but "already there?" and "first empty weak slot" are a ballot each instead of a scan.
constexpr uint32_t kMaxRev = 32;
__global__ void __launch_bounds__(256) inject_reverse_kernel(uint32_t* __restrict__ graph, const uint32_t* __restrict__ rev,
                                                             const uint32_t* __restrict__ counts, uint32_t n,
                                                             uint32_t total_degree, uint32_t local_degree) {
    const int lane = threadIdx.x & 63;
    const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n) return;  // wave-uniform
    const uint32_t num_remote = total_degree - local_degree;
    const uint32_t num_strong = num_remote / 2, num_weak = num_remote - num_strong;
    uint32_t rc = counts[i];
    if (rc == 0) return;
    if (rc > kMaxRev) rc = kMaxRev;
    uint32_t* row = graph + (size_t)i * total_degree;
    const uint32_t weak0 = local_degree + num_strong;  // first weak slot of the row
    uint32_t val[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t x = 64u * j + lane;
        val[j] = x < total_degree ? row[x] : 0xFFFFFFFEu;  // a value no source and no empty slot has
    }
    const uint32_t mine = (uint32_t)lane < rc ? rev[(size_t)i * kMaxRev + lane] : kInvalidId;
    uint32_t rng = wang_hash(i);
    for (uint32_t r = 0; r < rc; ++r) {
        const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)mine, (int)r);
        bool exists = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) exists = exists || __ballot(val[j] == c) != 0;
        if (exists) continue;
        uint32_t target = kInvalidId;  // the slot that takes the source
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t x = 64u * j + lane;
            const uint64_t empty = __ballot(x >= weak0 && x < total_degree && val[j] == kInvalidId);
            if (target == kInvalidId && empty != 0) target = 64u * j + (uint32_t)__builtin_ctzll(empty);
        }
        if (target == kInvalidId && num_weak > 0) {
            rng = wang_hash(rng);
            target = weak0 + (rng % num_weak);
        }
        if (target != kInvalidId) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (64u * j + lane == target) val[j] = c;
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t x = 64u * j + lane;
        if (x >= weak0 && x < total_degree) row[x] = val[j];
    }
}

}  // namespace
}  // namespace grab

using namespace grab;

extern "C" {

uint32_t grab_remote_global_k(uint32_t total_degree, uint32_t local_degree) {
    uint32_t gk = (total_degree - local_degree) * 4;
    gk = std::max(64u, (gk + 32) - (gk % 32));
    return std::min(256u, gk);
}

int grab_update_remote_edges(uint32_t* d_graph, const uint64_t* d_ts, const uint32_t* d_candidates, size_t num_dataset,
                             uint32_t total_degree, uint32_t local_degree, uint32_t global_k, void* stream) {
    GRAB_REQUIRE(d_graph && d_ts && d_candidates, "null pointer");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(local_degree <= total_degree && total_degree <= GRAB_MAX_DEGREE, "bad degrees");
    GRAB_REQUIRE(global_k >= 1 && global_k <= 256, "global_k must be in [1,256]");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t n = (uint32_t)num_dataset;
    hipLaunchKernelGGL(remote_edges_kernel, dim3((n + 3) / 4), dim3(256), 0, st, d_graph, d_ts, d_candidates, n, total_degree,
                       local_degree, global_k);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_enhance_global_connectivity(size_t num_dataset, uint32_t* d_graph, uint32_t total_degree, uint32_t local_degree,
                                     void* stream) {
    GRAB_REQUIRE(d_graph != nullptr, "null pointer");
    GRAB_REQUIRE(num_dataset > 0 && num_dataset < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(local_degree <= total_degree && total_degree <= GRAB_MAX_DEGREE, "bad degrees");
    if (total_degree == local_degree) return GRAB_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t n = (uint32_t)num_dataset;
    DeviceScratch rev, cnt;
    GRAB_HIP(rev.alloc((size_t)n * kMaxRev * 4));
    GRAB_HIP(cnt.alloc((size_t)n * 4));
    // sources of every row through remote slots, ascending source id (the reference: atomic arrival order)
    GRAB_TRY(reverse_lists(d_graph, n, total_degree, local_degree, total_degree - local_degree, 1, kMaxRev, rev.as<uint32_t>(),
                           cnt.as<uint32_t>(), st));
    hipLaunchKernelGGL(inject_reverse_kernel, dim3((n + 3) / 4), dim3(256), 0, st, d_graph, rev.as<uint32_t>(), cnt.as<uint32_t>(),
                       n, total_degree, local_degree);
    GRAB_HIP(hipGetLastError());
    GRAB_HIP(hipStreamSynchronize(st));
    return GRAB_OK;
}

int grab_build_global_remote_edges(const float* d_dataset, size_t num_dataset, uint32_t dim, uint32_t* d_graph,
                                   const uint64_t* d_ts, uint32_t total_degree, uint32_t local_degree, int metric,
                                   void* stream) {
    GRAB_REQUIRE(d_dataset && d_graph && d_ts, "null pointer");
    GRAB_REQUIRE(local_degree <= total_degree, "local_degree exceeds the graph degree");
    if (total_degree == local_degree) return GRAB_OK;
    const uint32_t gk = grab_remote_global_k(total_degree, local_degree);
    DeviceScratch cand;
    GRAB_HIP(cand.alloc(num_dataset * (size_t)gk * 4));
    GRAB_TRY(grab_generate_knn_graph(d_dataset, num_dataset, dim, gk, metric, cand.as<uint32_t>(), nullptr, stream));
    GRAB_TRY(grab_update_remote_edges(d_graph, d_ts, cand.as<uint32_t>(), num_dataset, total_degree, local_degree, gk, stream));
    return grab_enhance_global_connectivity(num_dataset, d_graph, total_degree, local_degree, stream);
}

int grab_build_time_partitioned_graph(const float* d_dataset, size_t total_num, uint32_t dim, uint32_t* d_graph,
                                      const uint64_t* d_ts, const size_t* bucket_sizes, size_t num_buckets,
                                      uint32_t total_degree, uint32_t local_degree, int metric, void* stream) {
    GRAB_REQUIRE(d_dataset && d_graph && d_ts && bucket_sizes, "null pointer");
    GRAB_REQUIRE(total_num > 0 && total_num < (1ull << 31), "total_num must be in [1, 2^31)");
    GRAB_REQUIRE(local_degree <= total_degree && total_degree >= 1 && total_degree <= GRAB_MAX_DEGREE / 2, "bad degrees");
    size_t sum = 0;
    for (size_t b = 0; b < num_buckets; ++b) sum += bucket_sizes[b];
    GRAB_REQUIRE(sum == total_num, "bucket sizes do not add up to the number of rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t inter = total_degree * 2;  // cagra_opt.cu:945
    size_t max_bucket = 0;
    for (size_t b = 0; b < num_buckets; ++b) max_bucket = std::max(max_bucket, bucket_sizes[b]);
    DeviceScratch knn;
    GRAB_HIP(knn.alloc(std::max<size_t>(max_bucket, 1) * inter * 4));
    const grab_build_params bp{inter, total_degree};
    // A bucket's build allocates and frees a dozen scratch buffers, each a wait for the device, and at 10,000 rows spends
    // as long in that as in its kernels.  The first bucket runs as ever and tells how much it asked for; the others take
    // their scratch from one block of that size (a bucket that wants more gets the rest the usual way).
    ScratchArena arena;
    DeviceScratch arena_mem;
    struct ArenaScope {  // the thread's arena is this one for the length of the loop, whatever way the loop is left
        explicit ArenaScope(ScratchArena* a) { scratch_arena() = a; }
        ~ArenaScope() { scratch_arena() = nullptr; }
    };
    int rc = GRAB_OK;
    {
        ArenaScope scope(&arena);
        size_t off = 0;
        bool first = true;
        for (size_t b = 0; b < num_buckets && rc == GRAB_OK; ++b) {
            const size_t bs = bucket_sizes[b];
            if (bs == 0) continue;
            arena.used = 0;
            arena.wanted = 0;
            uint32_t* g = d_graph + off * total_degree;
            rc = grab_generate_knn_graph(d_dataset + off * dim, bs, dim, inter, metric, knn.as<uint32_t>(), nullptr, stream);
            if (rc == GRAB_OK) rc = grab_build_graph(d_dataset + off * dim, bs, knn.as<uint32_t>(), bp, g, stream);
            if (rc == GRAB_OK && off > 0) {
                const size_t count = bs * total_degree;
                hipLaunchKernelGGL(shift_ids_kernel, dim3((uint32_t)((count + 255) / 256)), dim3(256), 0, st, g, count, (uint32_t)off);
                if (hipGetLastError() != hipSuccess) {
                    set_error("bucket %zu: the id shift could not be launched", b);
                    rc = GRAB_ERR_HIP;
                }
            }
            if (first && rc == GRAB_OK && num_buckets > 1) {
                // every buffer of the bucket just built has been freed by now, and its kernels are queued on `st`: the block
                // is used by the next bucket's kernels, which are queued behind them
                first = false;
                scratch_arena() = nullptr;  // the block itself is not to come out of the (empty) arena
                // `wanted` adds up everything the first bucket asked for (an arena gives nothing back), so the block is
                // generous; it never takes more than a quarter of what the device has free, and a bucket that wants more
                // than the block holds gets the rest the usual way
                size_t cap = arena.wanted + arena.wanted / 8 + (1u << 20), free_b = 0, total_b = 0;
                if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) cap = std::min(cap, free_b / 4);
                if (cap >= (1u << 20) && arena_mem.alloc(cap) == hipSuccess) {
                    arena.base = static_cast<char*>(arena_mem.ptr);
                    arena.cap = cap;
                } else {
                    (void)hipGetLastError();  // no room for the block: every bucket allocates as the first did
                    arena_mem.ptr = nullptr;
                }
                scratch_arena() = &arena;
            }
            off += bs;
        }
    }
    // The arena rests on one invariant: every kernel of the bucket builds is queued on `st`, so a block handed out again
    // is only written behind the kernels that read it before.  Once `st` has drained nothing uses the block any more,
    // and it goes back before the global pass asks for its own (larger) scratch.
    const hipError_t drained = hipStreamSynchronize(st);
    if (arena_mem.ptr != nullptr) {
        (void)hipFree(arena_mem.ptr);
        arena_mem.ptr = nullptr;
    }
    GRAB_TRY(rc);
    GRAB_HIP(drained);
    return grab_build_global_remote_edges(d_dataset, total_num, dim, d_graph, d_ts, total_degree, local_degree, metric, stream);
}

}  // extern "C"
