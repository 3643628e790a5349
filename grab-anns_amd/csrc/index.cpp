// Index handle: host mirrors, growable device buffers, seed sampling and staging around the
// stateless kernels.  Follows cagra::CagraIndex (src/cagraIndex.hpp:12-119, src/cagraIndex.cu)
// and the search surface of cagra::CagraIndexOpt (src/cagraIndexOpt.cu:223-551).
#include <algorithm>
#include <atomic>
#include <memory>
#include <chrono>
#include <condition_variable>
#include <cstring>
#include <fstream>
#include <iterator>
#include <map>
#include <mutex>
#include <numeric>
#include <random>
#include <thread>
#include <vector>

#include "entry_layer.hpp"
#include "insert_internal.hpp"
#include "search_internal.hpp"

namespace grab {
int sample_window_seeds_async(const uint64_t* d_sorted_ts, const uint32_t* d_ids_by_ts, size_t n,
                              const uint64_t* d_win_start, const uint64_t* d_win_end, uint64_t win_start,
                              uint64_t win_end, int per_query_window, size_t num_queries, uint32_t n_seeds,
                              uint64_t seed, uint32_t* d_out_seeds, hipStream_t st);
}

using namespace grab;

// grow-only device scratch owned by the handle (no allocation per call once warmed up)
struct ScratchBuf {
    void* ptr = nullptr;
    size_t bytes = 0;
    int ensure(size_t need) {
        if (need <= bytes) return GRAB_OK;
        if (ptr) GRAB_HIP(hipFree(ptr));
        ptr = nullptr;
        bytes = 0;
        const size_t want = std::max(need, (size_t)4096);
        GRAB_HIP(hipMalloc(&ptr, want));
        bytes = want;
        return GRAB_OK;
    }
    void release() {
        if (ptr) (void)hipFree(ptr);
        ptr = nullptr;
        bytes = 0;
    }
};

// What a large range-search batch that is cut into chunks (grab_index_search_range_batch) works with: two streams
// that the chunks alternate between, device and page-locked host staging for the whole batch (a chunk owns its
// slice, so nothing waits for a buffer), and a helper thread that shares the copying of the caller's rows into the
// page-locked staging with the calling thread.
struct BatchPipe {
    static constexpr int kStreams = 4;
    hipStream_t stream[kStreams] = {nullptr, nullptr, nullptr, nullptr};
    std::vector<hipEvent_t> done;  // one per chunk
    ScratchBuf in, id_lo, id_hi, seeds, probe;  // a chunk's slice of `in`: queries, window starts, window ends
    void* h_in = nullptr;    // hipHostMalloc, laid out like `in`
    void* h_out = nullptr;   // hipHostMalloc; a chunk's slice: int64 ids, float distances - written by the search kernel itself
    size_t h_in_bytes = 0, h_out_bytes = 0;
    // helper threads: they share out the copies of a call among themselves, marking each as it is done
    struct Copy {
        char* dst;
        const char* src[3];
        size_t bytes[3];
    };
    static constexpr int kHelpers = 3;
    std::thread helper[kHelpers];
    std::mutex mu;
    std::condition_variable cv;
    std::vector<Copy> jobs;          // written under mu while every helper is parked; read by the helpers during a call
    uint64_t epoch = 0;              // guarded by mu: counts the calls that posted jobs
    int parked = 0;                  // guarded by mu: helpers waiting for the next call
    bool quit = false;               // guarded by mu
    std::atomic<size_t> next{0};     // the next job to take
    std::unique_ptr<std::atomic<uint8_t>[]> done_flag;  // one per job of the call
    size_t flags = 0;
};

struct grab_index {
    uint32_t dim = 0, degree = 0, local_degree = 0;
    size_t size = 0;  // rows present on host and device
    std::vector<float> h_data;
    std::vector<uint32_t> h_graph;
    std::vector<uint64_t> h_ts;
    std::vector<uint8_t> h_labels;
    std::map<uint64_t, std::vector<uint32_t>> ts_to_ids;
    grab_vmm* d_data = nullptr;
    grab_vmm* d_graph = nullptr;
    grab_vmm* d_ts = nullptr;
    grab_build_params build_params{};
    grab_search_params search_params{};
    grab_search_params insert_params{};
    int metric = GRAB_METRIC_L2;
    uint32_t flags = 0;
    uint64_t rng = 0x243F6A8885A308D3ull;
    bool built = false;
    bool host_graph_stale = false;
    bool ts_order_stale = true;
    bool labels_stale = true;
    float last_kernel_ms = 0.0f;
    double knn_s = 0, opt_s = 0, total_s = 0;
    hipStream_t stream = nullptr;
    SideStream side;  // created by the first insert into the time-partitioned graph
    ScratchBuf q, out_i, out_d, seeds, win_s, win_e, masks, ins_ws, sorted_ts, ids_by_ts, labels;
    std::vector<std::vector<uint32_t>> label_ids;  // ids per label, for mask-filter seeds
    // optional entry-point layer for range searches: rebuilt when rows were added since it was made
    uint32_t entry_samples = 0, entry_seeds = 0;
    uint32_t entry_groups = 0, entry_nprobe = 16, entry_min_rows = 32;  // coarse level of the layer (0 groups = none)
    grab_entry_layer* entry = nullptr;
    size_t entry_rows = 0;
    std::mt19937 seed_rng{1234};  // sample_seeds_by_time draws from a generator seeded like the reference's
    bool ts_monotone = true;  // timestamps never decrease with the row id: a window is an id interval
    ScratchBuf id_lo, id_hi;
    ScratchBuf graph_ts;  // timestamps of every row's neighbours (grab_neighbor_timestamps), made on demand
    size_t graph_ts_rows = 0;
    uint32_t entry_list = 0;  // > 0: the in-window rows of the nearest groups are listed (at most this many) instead of scored
    int fail_insert_at = -1;  // test hook: the next insert fails before this inner step (grab_index_debug_fail_insert)
    std::vector<uint64_t> ts_pivots;  // every 256th timestamp of rows in timestamp order: the first level of a window's lookup
    size_t ts_pivot_rows = 0;
    double scan_below = 0.0;  // range batches: windows of at most this fraction of the rows are scanned exactly (0 = none)
    grab_scan_base* scan = nullptr;  // the rows prepared for grab_index_scan_range_batch, remade when rows were added
    size_t scan_rows = 0;
    BatchPipe pipe;
    size_t chunk_queries = 5000;  // most queries in a chunk of a pipelined batch; 0 switches the pipeline off
};

namespace {

uint64_t next_mask(grab_index* h) { return splitmix64(&h->rng) & 0xFFFFFFFFull; }  // 32 random bits, as std::random_device

int upload(grab_index* h, ScratchBuf& b, const void* src, size_t bytes) {
    GRAB_TRY(b.ensure(bytes));
    if (bytes) GRAB_HIP(hipMemcpyAsync(b.ptr, src, bytes, hipMemcpyHostToDevice, h->stream));
    return GRAB_OK;
}

int stage_queries(grab_index* h, const float* queries, size_t nq, int k) {
    GRAB_REQUIRE(queries != nullptr, "null queries");
    GRAB_REQUIRE(k >= 1, "k must be positive");
    GRAB_TRY(upload(h, h->q, queries, nq * h->dim * sizeof(float)));
    GRAB_TRY(h->out_i.ensure(nq * (size_t)k * sizeof(int64_t)));
    GRAB_TRY(h->out_d.ensure(nq * (size_t)k * sizeof(float)));
    return GRAB_OK;
}

int fetch_results(grab_index* h, size_t nq, int k, int64_t* indices, float* dists) {
    GRAB_HIP(hipMemcpyAsync(indices, h->out_i.ptr, nq * (size_t)k * sizeof(int64_t), hipMemcpyDeviceToHost, h->stream));
    GRAB_HIP(hipMemcpyAsync(dists, h->out_d.ptr, nq * (size_t)k * sizeof(float), hipMemcpyDeviceToHost, h->stream));
    GRAB_HIP(hipStreamSynchronize(h->stream));
    return GRAB_OK;
}

void fill_empty(size_t nq, int k, int64_t* indices, float* dists) {
    // CagraIndexOpt reports an empty window / bucket like this (src/cagraIndexOpt.cu:479-485)
    for (size_t i = 0; i < nq * (size_t)k; ++i) {
        indices[i] = -1;
        dists[i] = -1.0f;
    }
}

int run_desc(grab_index* h, grab_search_desc& d) {
    d.kernel_ms = &h->last_kernel_ms;
    return search_ex_impl(&d, false);
}

void base_desc(grab_index* h, grab_search_desc* d, int wrapper, size_t nq, int k, uint32_t active_degree,
               const uint32_t* d_seeds, uint32_t n_provided) {
    fill_search_desc(d, wrapper, static_cast<const float*>(grab_vmm_data(h->d_data)), h->size, h->dim,
                     static_cast<const uint32_t*>(grab_vmm_data(h->d_graph)), h->degree, active_degree,
                     static_cast<const float*>(h->q.ptr), nq, (uint32_t)k, h->search_params, h->metric, d_seeds,
                     n_provided, next_mask(h), h->flags, static_cast<int64_t*>(h->out_i.ptr),
                     static_cast<float*>(h->out_d.ptr), h->stream);
}

// stratified sample of `want` entries of `ids` (all of them when there are fewer)
std::vector<uint32_t> sample_ids(grab_index* h, const std::vector<uint32_t>& ids, size_t want) {
    if (ids.size() <= want) return ids;
    std::vector<uint32_t> out(want);
    for (size_t i = 0; i < want; ++i) {
        const size_t b0 = i * ids.size() / want, b1 = (i + 1) * ids.size() / want;
        out[i] = ids[b0 + splitmix64(&h->rng) % (b1 - b0)];
    }
    return out;
}

// first row whose timestamp is not below t, rows in timestamp order: a search over every 256th timestamp (a table that
// stays in the cache) and one inside the stretch it names, instead of twenty steps across the whole array
size_t first_row_at(grab_index* h, uint64_t t) {
    const size_t n = h->size;
    if (h->ts_pivot_rows != n) {
        h->ts_pivots.clear();
        for (size_t i = 0; i < n; i += 256) h->ts_pivots.push_back(h->h_ts[i]);
        h->ts_pivot_rows = n;
    }
    // pivots[j] = ts[256 j]; the first pivot not below t bounds the stretch from above, the one before it from below
    const size_t j = (size_t)(std::lower_bound(h->ts_pivots.begin(), h->ts_pivots.end(), t) - h->ts_pivots.begin());
    const size_t lo = j == 0 ? 0 : (j - 1) * 256, hi = std::min(n, j * 256 + 1);
    return (size_t)(std::lower_bound(h->h_ts.begin() + lo, h->h_ts.begin() + hi, t) - h->h_ts.begin());
}

int ensure_ts_order(grab_index* h) {
    if (!h->ts_order_stale) return GRAB_OK;
    h->graph_ts_rows = 0;
    const size_t n = h->size;
    GRAB_REQUIRE(h->h_ts.size() >= n, "the index holds rows without timestamps");
    std::vector<uint32_t> order(n);
    std::iota(order.begin(), order.end(), 0u);
    h->ts_monotone = std::is_sorted(h->h_ts.begin(), h->h_ts.begin() + n);
    if (!h->ts_monotone)
        std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return h->h_ts[x] < h->h_ts[y]; });
    std::vector<uint64_t> sorted(n);
    for (size_t i = 0; i < n; ++i) sorted[i] = h->h_ts[order[i]];
    GRAB_TRY(upload(h, h->sorted_ts, sorted.data(), n * sizeof(uint64_t)));
    GRAB_TRY(upload(h, h->ids_by_ts, order.data(), n * sizeof(uint32_t)));
    GRAB_HIP(hipStreamSynchronize(h->stream));  // the host vectors go out of scope
    h->ts_order_stale = false;
    return GRAB_OK;
}

// (re)makes the entry-point layer over the current rows
// Timestamp-filtered searches that the wave-per-query kernel with the queue in registers will run (large batch,
// short queue, filter before the visited set) read the neighbours' timestamps from rows laid out like the graph.
// Everything that changes the graph or the timestamps marks the timestamp order stale, which drops these rows too.
int attach_neighbor_timestamps(grab_index* h, grab_search_desc& d, size_t nq) {
    if (!(h->flags & GRAB_FLAG_FILTER_FIRST) || (h->flags & GRAB_FLAG_STRICT_REFERENCE) || nq < 1024 || d.itopk > 64 ||
        d.hash_bitlen > 15)
        return GRAB_OK;
    GRAB_TRY(ensure_ts_order(h));  // a change of graph or timestamps since the rows were made drops them here
    if (h->graph_ts_rows != h->size) {
        GRAB_TRY(h->graph_ts.ensure(h->size * (size_t)h->degree * sizeof(uint64_t)));
        GRAB_TRY(grab_neighbor_timestamps(static_cast<const uint32_t*>(grab_vmm_data(h->d_graph)),
                                          static_cast<const uint64_t*>(grab_vmm_data(h->d_ts)), h->size, h->degree,
                                          static_cast<uint64_t*>(h->graph_ts.ptr), h->stream));
        h->graph_ts_rows = h->size;
    }
    d.d_graph_ts = static_cast<const uint64_t*>(h->graph_ts.ptr);
    return GRAB_OK;
}

int ensure_entry_layer(grab_index* h) {
    GRAB_TRY(ensure_ts_order(h));
    if (h->entry && h->entry_rows == h->size) return GRAB_OK;
    if (h->entry) grab_entry_layer_destroy(h->entry);
    h->entry = nullptr;
    GRAB_HIP(hipStreamSynchronize(h->stream));
    GRAB_TRY(grab_entry_layer_create(static_cast<const float*>(grab_vmm_data(h->d_data)), h->size, h->dim,
                                     h->ts_monotone ? nullptr : static_cast<const uint32_t*>(h->ids_by_ts.ptr),
                                     static_cast<const uint64_t*>(grab_vmm_data(h->d_ts)), nullptr, h->entry_samples, &h->entry));
    if (h->entry_groups > 0)
        GRAB_TRY(grab_entry_layer_build_groups(h->entry, std::min<uint32_t>(h->entry_groups, grab_entry_layer_size(h->entry)), 10,
                                               splitmix64(&h->rng)));
    h->entry_rows = h->size;
    return GRAB_OK;
}

// where one range search with entry-layer seeds finds its staged queries and leaves its results
struct RangeStage {
    const float* q;
    uint32_t* seeds;       // [nq, entry_seed_count]
    uint64_t *id_lo, *id_hi;  // [nq] each, used when the window becomes an interval of row ids
    uint32_t* probe;       // scratch of the coarse level, null = the layer's own
    int64_t* out_i;
    float* out_d;
    hipStream_t stream;
    uint64_t mask;         // rand_xor_mask of the search
    bool timed;            // kernel duration into last_kernel_ms (waits for the kernel)
};

bool window_is_id_interval(const grab_index* h, int per_query) { return h->ts_monotone && per_query; }

// seeds per query that the entry layer hands over: the listed rows, or the scored ones
uint32_t entry_seed_count(const grab_index* h, int per_query) {
    const bool listed = h->entry_list > 0 && h->entry_groups > 0 && window_is_id_interval(h, per_query);
    return listed ? std::min(h->entry_list, 64u) : std::min(h->entry_seeds, std::max(h->search_params.itopk_size, 64u));
}

// Range search seeded by the entry-point layer; windows are on the device (per query) or scalar.
int search_range_with_layer(grab_index* h, const RangeStage& g, size_t nq, int k, const uint64_t* d_ws, const uint64_t* d_we,
                            uint64_t ws, uint64_t we, int per_query) {
    const bool id_filter = window_is_id_interval(h, per_query);  // the window as an interval of row ids: no timestamp is read
    const bool listed = h->entry_list > 0 && h->entry_groups > 0 && id_filter;
    const uint32_t want = entry_seed_count(h, per_query);
    const bool grouped = h->entry_groups > 0 && want <= 64;
    const uint64_t* d_base_ts = static_cast<const uint64_t*>(grab_vmm_data(h->d_ts));
    if (grouped) {
        GRAB_TRY(entry_layer_select_grouped_async(h->entry, g.q, nq, h->metric, d_ws, d_we, ws, we, per_query,
                                                  id_filter ? d_base_ts : nullptr, h->size, g.id_lo, g.id_hi, h->entry_nprobe,
                                                  h->entry_min_rows, want, g.seeds, nullptr, g.stream, listed, g.probe));
    } else {
        GRAB_TRY(grab_entry_layer_select(h->entry, g.q, nq, h->metric, 1, d_ws, d_we, ws, we, per_query, nullptr, want, g.seeds,
                                         nullptr, g.stream));
    }
    grab_search_desc d;
    fill_search_desc(&d, GRAB_WRAP_RANGE, static_cast<const float*>(grab_vmm_data(h->d_data)), h->size, h->dim,
                     static_cast<const uint32_t*>(grab_vmm_data(h->d_graph)), h->degree, h->degree, g.q, nq, (uint32_t)k,
                     h->search_params, h->metric, g.seeds, want, g.mask, h->flags, g.out_i, g.out_d, g.stream);
    if (id_filter) {
        if (!grouped) GRAB_TRY(grab_windows_to_id_ranges(d_base_ts, h->size, d_ws, d_we, nq, g.id_lo, g.id_hi, g.stream));
        d.filter_kind = 3;
        d.d_win_start = g.id_lo;
        d.d_win_end = g.id_hi;
        d.per_query_window = 1;
    } else {
        d.filter_kind = 1;
        d.d_ts = static_cast<const uint64_t*>(grab_vmm_data(h->d_ts));
        d.d_win_start = d_ws;
        d.d_win_end = d_we;
        d.win_start = ws;
        d.win_end = we;
        d.per_query_window = per_query;
        GRAB_TRY(attach_neighbor_timestamps(h, d, nq));
    }
    if (g.timed) return run_desc(h, d);
    return search_ex_impl(&d, false);
}

// the handle's own staging (queries and result buffers by stage_queries), one call at a time on its stream
int own_stage(grab_index* h, size_t nq, int per_query, RangeStage* g) {
    GRAB_TRY(ensure_entry_layer(h));
    GRAB_TRY(h->seeds.ensure(nq * (size_t)entry_seed_count(h, per_query) * sizeof(uint32_t)));
    GRAB_TRY(h->id_lo.ensure(nq * sizeof(uint64_t)));
    GRAB_TRY(h->id_hi.ensure(nq * sizeof(uint64_t)));
    *g = RangeStage{static_cast<const float*>(h->q.ptr), static_cast<uint32_t*>(h->seeds.ptr), static_cast<uint64_t*>(h->id_lo.ptr),
                    static_cast<uint64_t*>(h->id_hi.ptr), nullptr, static_cast<int64_t*>(h->out_i.ptr),
                    static_cast<float*>(h->out_d.ptr), h->stream, next_mask(h), true};
    return GRAB_OK;
}

void pipe_helper_main(BatchPipe* p) {
    uint64_t epoch = 0;
    std::unique_lock<std::mutex> lock(p->mu);
    for (;;) {
        ++p->parked;
        p->cv.wait(lock, [&] { return p->quit || p->epoch != epoch; });
        --p->parked;
        if (p->quit) return;
        epoch = p->epoch;
        const size_t n = p->jobs.size();
        lock.unlock();
        for (;;) {
            const size_t j = p->next.fetch_add(1, std::memory_order_relaxed);
            if (j >= n) break;
            const BatchPipe::Copy& job = p->jobs[j];
            char* dst = job.dst;
            for (int i = 0; i < 3; ++i) {
                if (job.bytes[i]) std::memcpy(dst, job.src[i], job.bytes[i]);
                dst += job.bytes[i];
            }
            p->done_flag[j].store(1, std::memory_order_release);
        }
        lock.lock();
    }
}

// every helper is back at its wait: the job list may be rewritten
void pipe_wait_parked(BatchPipe& p) {
    for (;;) {
        {
            std::lock_guard<std::mutex> lock(p.mu);
            if (p.parked == BatchPipe::kHelpers) return;
        }
        std::this_thread::yield();
    }
}

void pipe_release(BatchPipe& p) {
    if (p.helper[0].joinable()) {
        {
            std::lock_guard<std::mutex> lock(p.mu);
            p.quit = true;
        }
        p.cv.notify_all();
        for (std::thread& t : p.helper)
            if (t.joinable()) t.join();
    }
    for (hipStream_t st : p.stream)
        if (st) (void)hipStreamSynchronize(st);
    for (ScratchBuf* b : {&p.in, &p.id_lo, &p.id_hi, &p.seeds, &p.probe}) b->release();
    if (p.h_in) (void)hipHostFree(p.h_in);
    if (p.h_out) (void)hipHostFree(p.h_out);
    for (hipEvent_t e : p.done) (void)hipEventDestroy(e);
    for (hipStream_t st : p.stream)
        if (st) (void)hipStreamDestroy(st);
}

int pipe_ready(grab_index* h, size_t nq, size_t chunks, size_t in_bytes, size_t out_bytes, uint32_t seeds_per_query) {
    BatchPipe& p = h->pipe;
    for (hipStream_t& st : p.stream)
        if (st == nullptr) GRAB_HIP(hipStreamCreate(&st));  // default priority, like the handle's stream
    while (p.done.size() < chunks) {
        hipEvent_t e = nullptr;
        GRAB_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        p.done.push_back(e);
    }
    auto grow = [](void*& ptr, size_t& have, size_t need) -> int {
        if (need <= have) return GRAB_OK;
        if (ptr) GRAB_HIP(hipHostFree(ptr));
        ptr = nullptr;
        have = 0;
        GRAB_HIP(hipHostMalloc(&ptr, need, hipHostMallocDefault));
        have = need;
        return GRAB_OK;
    };
    GRAB_TRY(grow(p.h_in, p.h_in_bytes, in_bytes));
    GRAB_TRY(grow(p.h_out, p.h_out_bytes, out_bytes));
    GRAB_TRY(p.in.ensure(in_bytes));
    GRAB_TRY(p.seeds.ensure(nq * (size_t)seeds_per_query * sizeof(uint32_t)));
    GRAB_TRY(p.id_lo.ensure(nq * sizeof(uint64_t)));
    GRAB_TRY(p.id_hi.ensure(nq * sizeof(uint64_t)));
    GRAB_TRY(p.probe.ensure(nq * (size_t)h->entry_nprobe * sizeof(uint32_t)));
    if (!p.helper[0].joinable())
        for (std::thread& t : p.helper) t = std::thread(pipe_helper_main, &p);
    return GRAB_OK;
}

// `bytes` of the caller's (pageable) memory into the pipe's page-locked staging, shared out between the calling thread
// and the helpers, and behind them two short arrays that the calling thread copies; returns when all of it is there.
void pipe_stage(BatchPipe& p, const void* src, size_t bytes, const void* tail0, const void* tail1, size_t tail_bytes) {
    constexpr size_t kParts = BatchPipe::kHelpers + 1;
    const char* from = static_cast<const char*>(src);
    char* to = static_cast<char*>(p.h_in);
    auto bound = [&](size_t part) { return part >= kParts ? bytes : (bytes * part / kParts) & ~(size_t)63; };
    pipe_wait_parked(p);
    {
        std::lock_guard<std::mutex> lock(p.mu);
        p.jobs.clear();
        for (size_t part = 1; part < kParts; ++part)
            p.jobs.push_back(BatchPipe::Copy{to + bound(part), {from + bound(part), nullptr, nullptr}, {bound(part + 1) - bound(part), 0, 0}});
        if (p.flags < p.jobs.size()) {
            p.done_flag.reset(new std::atomic<uint8_t>[p.jobs.size()]);
            p.flags = p.jobs.size();
        }
        for (size_t j = 0; j < p.jobs.size(); ++j) p.done_flag[j].store(0, std::memory_order_relaxed);
        p.next.store(0, std::memory_order_relaxed);
        ++p.epoch;
    }
    p.cv.notify_all();
    std::memcpy(to, from, bound(1));
    if (tail_bytes) {
        std::memcpy(to + bytes, tail0, tail_bytes);
        std::memcpy(to + bytes + tail_bytes, tail1, tail_bytes);
    }
    for (size_t j = 0; j < p.jobs.size(); ++j)
        while (p.done_flag[j].load(std::memory_order_acquire) == 0) std::this_thread::yield();
}

// A large batch with a window per query, cut into chunks that take turns on the pipe's streams: while one chunk's kernels
// run, the next chunk's queries are staged and copied in, and the chunk before's results are handed back.  The
// caller's memory is pageable, so its rows are first copied to page-locked staging by the CPU - a quarter of a chunk
// by the calling thread, the rest by three helper threads.  Every query's answer depends on that query alone and
// all chunks use the one rand_xor_mask that the undivided call would have drawn, so the results are those of that call.
int search_range_batch_chunked(grab_index* h, const float* queries, size_t nq, int k, const uint64_t* start_ts,
                               const uint64_t* end_ts, int64_t* indices, float* dists) {
    GRAB_TRY(ensure_entry_layer(h));
    GRAB_HIP(hipStreamSynchronize(h->stream));  // the layer, the timestamp order: all there before the chunks start
    const uint64_t mask = next_mask(h);
    BatchPipe& p = h->pipe;
    // equal chunks of at most chunk_queries queries
    // (an even number each, so that a chunk's slice of the result staging starts on an 8-byte boundary whatever k is)
    const size_t parts = (nq + h->chunk_queries - 1) / h->chunk_queries, chunk = ((nq + parts - 1) / parts + 1) & ~(size_t)1;
    const size_t chunks = (nq + chunk - 1) / chunk;
    const size_t row_q = h->dim * sizeof(float), row_in = row_q + 2 * sizeof(uint64_t);
    const size_t row_out = (size_t)k * (sizeof(int64_t) + sizeof(float));
    const uint32_t want = entry_seed_count(h, 1);
    GRAB_TRY(pipe_ready(h, nq, chunks, nq * row_in, nq * row_out, want));
    auto slice = [&](size_t c, size_t* off, size_t* m) {
        *off = c * chunk;
        *m = std::min(chunk, nq - *off);
    };
    // a chunk's rows are copied to the staging in kHelpers + 1 parts: the first (with the windows) by the calling thread,
    // the others by the helpers
    constexpr size_t kParts = BatchPipe::kHelpers + 1;
    auto copy_job = [&](size_t c, size_t part) {
        size_t off, m;
        slice(c, &off, &m);
        const size_t r0 = m * part / kParts, r1 = m * (part + 1) / kParts;
        char* dst = static_cast<char*>(p.h_in) + off * row_in;
        const char* q = reinterpret_cast<const char*>(queries + off * h->dim);
        if (part > 0) return BatchPipe::Copy{dst + r0 * row_q, {q + r0 * row_q, nullptr, nullptr}, {(r1 - r0) * row_q, 0, 0}};
        return BatchPipe::Copy{dst, {q, reinterpret_cast<const char*>(start_ts + off), reinterpret_cast<const char*>(end_ts + off)},
                               {r1 * row_q, m * sizeof(uint64_t), m * sizeof(uint64_t)}};
    };
    pipe_wait_parked(p);
    {
        std::lock_guard<std::mutex> lock(p.mu);
        p.jobs.clear();
        for (size_t c = 0; c < chunks; ++c)
            for (size_t part = 1; part < kParts; ++part) p.jobs.push_back(copy_job(c, part));
        if (p.flags < p.jobs.size()) {
            p.done_flag.reset(new std::atomic<uint8_t>[p.jobs.size()]);
            p.flags = p.jobs.size();
        }
        for (size_t j = 0; j < p.jobs.size(); ++j) p.done_flag[j].store(0, std::memory_order_relaxed);
        p.next.store(0, std::memory_order_relaxed);
        ++p.epoch;
    }
    p.cv.notify_all();
    auto chunk_staged = [&](size_t c) {
        for (size_t j = c * BatchPipe::kHelpers; j < (c + 1) * BatchPipe::kHelpers; ++j)
            while (p.done_flag[j].load(std::memory_order_acquire) == 0) std::this_thread::yield();
    };
    int rc = GRAB_OK;
    size_t queued = 0;
    for (size_t c = 0; c < chunks && rc == GRAB_OK; ++c) {
        size_t off, m;
        slice(c, &off, &m);
        char* hin = static_cast<char*>(p.h_in) + off * row_in;
        {
            const BatchPipe::Copy job = copy_job(c, 0);
            std::memcpy(job.dst, job.src[0], job.bytes[0]);
            std::memcpy(job.dst + m * row_q, job.src[1], job.bytes[1]);
            std::memcpy(job.dst + m * row_q + m * sizeof(uint64_t), job.src[2], job.bytes[2]);
            chunk_staged(c);
        }
        auto enqueue = [&]() -> int {
            hipStream_t st = p.stream[c % BatchPipe::kStreams];
            // Both hand-overs stay on the stream's compute queue: a copy kernel reads the page-locked staging, and the
            // search writes its results straight into page-locked memory.  (Copy-engine transfers between the kernels
            // of two streams cost tens of microseconds per hand-over from queue to engine and back.)
            char* din = static_cast<char*>(p.in.ptr) + off * row_in;
            // ... by 32 workgroups: the copy waits on the host link, and a grid that fills the device takes the wave slots
            // of the chunk before's kernels (centroid ranking beside a full-grid copy: 80 us instead of 13)
            GRAB_TRY(device_copy_async(din, hin, m * row_in, st, 32));
            const uint64_t* d_ws = reinterpret_cast<const uint64_t*>(din + m * row_q);
            char* hout = static_cast<char*>(p.h_out) + off * row_out;
            const RangeStage g{reinterpret_cast<const float*>(din), static_cast<uint32_t*>(p.seeds.ptr) + off * want,
                               static_cast<uint64_t*>(p.id_lo.ptr) + off, static_cast<uint64_t*>(p.id_hi.ptr) + off,
                               static_cast<uint32_t*>(p.probe.ptr) + off * h->entry_nprobe, reinterpret_cast<int64_t*>(hout),
                               reinterpret_cast<float*>(hout + m * (size_t)k * sizeof(int64_t)), st, mask, false};
            GRAB_TRY(search_range_with_layer(h, g, m, k, d_ws, d_ws + m, 0, 0, 1));
            GRAB_HIP(hipEventRecord(p.done[c], st));
            return GRAB_OK;
        };
        rc = enqueue();
        if (rc == GRAB_OK) queued = c + 1;
    }
    // results leave the staging chunk by chunk, as the chunks finish
    for (size_t c = 0; c < queued; ++c) {
        size_t off, m;
        slice(c, &off, &m);
        if (hipEventSynchronize(p.done[c]) != hipSuccess) {
            if (rc == GRAB_OK) {
                set_error("HIP error while waiting for a chunk of the batch");
                rc = GRAB_ERR_HIP;
            }
            continue;
        }
        if (rc != GRAB_OK) continue;
        const char* hout = static_cast<const char*>(p.h_out) + off * row_out;
        std::memcpy(indices + off * (size_t)k, hout, m * (size_t)k * sizeof(int64_t));
        std::memcpy(dists + off * (size_t)k, hout + m * (size_t)k * sizeof(int64_t), m * (size_t)k * sizeof(float));
    }
    // the helpers must be through with the caller's arrays before the call returns, whatever happened
    for (size_t c = 0; c < chunks; ++c) chunk_staged(c);
    if (rc != GRAB_OK)
        for (hipStream_t st : p.stream) (void)hipStreamSynchronize(st);
    h->last_kernel_ms = 0.0f;  // not measured: the chunks' kernels overlap
    return rc;
}

int require_built(const grab_index* h) {
    if (!h->built || h->size == 0) {
        set_error("the index has no graph yet: call build first");
        return GRAB_ERR_STATE;
    }
    return GRAB_OK;
}

}  // namespace

extern "C" {

int grab_index_create(uint32_t dim, uint32_t graph_degree, uint32_t local_degree, size_t vmm_max_bytes, grab_index** out) {
    GRAB_REQUIRE(out != nullptr, "null output pointer");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(graph_degree >= 1 && graph_degree <= GRAB_MAX_DEGREE / 2, "graph_degree must be in [1,%d]", GRAB_MAX_DEGREE / 2);
    GRAB_REQUIRE(local_degree <= graph_degree, "local_degree exceeds graph_degree");
    GRAB_REQUIRE(vmm_max_bytes >= (1u << 22), "vmm_max_bytes too small");
    auto* h = new grab_index();
    h->dim = dim;
    h->degree = graph_degree;
    h->local_degree = local_degree ? local_degree : graph_degree;
    // src/cagraIndex.cu:13-37
    h->build_params.graph_degree = graph_degree;
    h->build_params.intermediate_degree = std::max(128u, graph_degree * 2);
    h->search_params = {256, 6, 0, 50, 13};
    h->insert_params = {128, 6, 0, 50, 12};
    int rc = GRAB_OK;
    if (hipStreamCreate(&h->stream) != hipSuccess) {
        set_error("cannot create a HIP stream (is a GPU present?)");
        rc = GRAB_ERR_HIP;
    }
    if (rc == GRAB_OK) rc = grab_vmm_create(vmm_max_bytes / 2, &h->d_data);
    if (rc == GRAB_OK) rc = grab_vmm_create(vmm_max_bytes / 2, &h->d_graph);
    // room for one timestamp per row that the data buffer can hold (the reference reserves a
    // fixed 10M entries, src/cagraIndex.cu:18)
    if (rc == GRAB_OK) rc = grab_vmm_create(std::max<size_t>(vmm_max_bytes / 2 / (dim * 4) * 8, 1u << 21), &h->d_ts);
    if (rc != GRAB_OK) {
        grab_index_destroy(h);
        return rc;
    }
    *out = h;
    return GRAB_OK;
}

void grab_index_destroy(grab_index* h) {
    if (!h) return;
    if (h->stream) (void)hipStreamSynchronize(h->stream);
    for (ScratchBuf* b : {&h->q, &h->out_i, &h->out_d, &h->seeds, &h->win_s, &h->win_e, &h->masks, &h->ins_ws,
                          &h->sorted_ts, &h->ids_by_ts, &h->labels, &h->id_lo, &h->id_hi, &h->graph_ts})
        b->release();
    pipe_release(h->pipe);
    if (h->entry) grab_entry_layer_destroy(h->entry);
    grab_scan_base_destroy(h->scan);
    grab_vmm_destroy(h->d_data);
    grab_vmm_destroy(h->d_graph);
    grab_vmm_destroy(h->d_ts);
    if (h->side.stream) (void)hipStreamSynchronize(h->side.stream);
    if (h->side.fork) (void)hipEventDestroy(h->side.fork);
    if (h->side.join) (void)hipEventDestroy(h->side.join);
    if (h->side.stream) (void)hipStreamDestroy(h->side.stream);
    if (h->stream) (void)hipStreamDestroy(h->stream);
    delete h;
}

int grab_index_set_metric(grab_index* h, int metric) {
    GRAB_REQUIRE(h && (metric == GRAB_METRIC_L2 || metric == GRAB_METRIC_IP), "bad metric");
    h->metric = metric;
    return GRAB_OK;
}
int grab_index_set_seed(grab_index* h, uint64_t seed) {
    GRAB_REQUIRE(h != nullptr, "null index");
    h->rng = seed;
    return GRAB_OK;
}
int grab_index_get_rng_state(const grab_index* h, uint64_t* state) {
    GRAB_REQUIRE(h && state, "null pointer");
    *state = h->rng;
    return GRAB_OK;
}

int grab_index_get_query_params(const grab_index* h, grab_search_params* out) {
    GRAB_REQUIRE(h && out, "null pointer");
    *out = h->search_params;
    return GRAB_OK;
}

int grab_index_set_scan_below(grab_index* h, double fraction) {
    GRAB_REQUIRE(h != nullptr, "null index");
    GRAB_REQUIRE(fraction >= 0.0 && fraction <= 1.0, "the fraction must be in [0,1]");
    h->scan_below = fraction;
    return GRAB_OK;
}
int grab_index_set_flags(grab_index* h, uint32_t flags) {
    GRAB_REQUIRE(h != nullptr, "null index");
    h->flags = flags;
    return GRAB_OK;
}
// CagraIndexOpt::build, src/cagraIndexOpt.cu:133-221: buckets are the runs of equal consecutive
// timestamps; local graphs per bucket, remote edges in the slots [local_degree, degree)
int grab_index_build_partitioned(grab_index* h) {
    GRAB_REQUIRE(h != nullptr, "null index");
    const size_t n = h->h_data.size() / h->dim;
    if (n == 0) return GRAB_OK;
    GRAB_REQUIRE(h->h_ts.size() == n, "the time-partitioned build needs a timestamp for every row");
    GRAB_REQUIRE(h->local_degree >= 1 && h->local_degree <= h->degree, "local_degree must be in [1, graph_degree]");
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    std::vector<size_t> bucket_sizes;
    size_t count = 0;
    for (size_t i = 0; i < n; ++i) {
        if (i > 0 && h->h_ts[i] != h->h_ts[i - 1]) {
            bucket_sizes.push_back(count);
            count = 0;
        }
        ++count;
    }
    bucket_sizes.push_back(count);
    GRAB_TRY(grab_vmm_resize(h->d_data, n * h->dim * sizeof(float)));
    GRAB_TRY(grab_vmm_resize(h->d_graph, n * h->degree * sizeof(uint32_t)));
    GRAB_TRY(grab_vmm_resize(h->d_ts, n * sizeof(uint64_t)));
    float* d_data = static_cast<float*>(grab_vmm_data(h->d_data));
    uint32_t* d_graph = static_cast<uint32_t*>(grab_vmm_data(h->d_graph));
    uint64_t* d_ts = static_cast<uint64_t*>(grab_vmm_data(h->d_ts));
    GRAB_HIP(hipMemcpy(d_data, h->h_data.data(), n * h->dim * sizeof(float), hipMemcpyHostToDevice));
    GRAB_HIP(hipMemcpy(d_ts, h->h_ts.data(), n * sizeof(uint64_t), hipMemcpyHostToDevice));
    GRAB_TRY(grab_build_time_partitioned_graph(d_data, n, h->dim, d_graph, d_ts, bucket_sizes.data(), bucket_sizes.size(),
                                               h->degree, h->local_degree, h->metric, h->stream));
    h->h_graph.resize(n * h->degree);
    GRAB_HIP(hipMemcpy(h->h_graph.data(), d_graph, n * h->degree * sizeof(uint32_t), hipMemcpyDeviceToHost));
    h->size = n;
    h->built = true;
    h->host_graph_stale = false;
    h->ts_order_stale = true;
    h->entry_rows = 0;
    h->scan_rows = 0;
    h->ts_pivot_rows = 0;
    h->knn_s = h->opt_s = 0;
    h->total_s = std::chrono::duration<double>(clk::now() - t0).count();
    return GRAB_OK;
}

int grab_index_set_entry_layer(grab_index* h, uint32_t num_samples, uint32_t seeds_per_query) {
    GRAB_REQUIRE(h != nullptr, "null index");
    GRAB_REQUIRE(num_samples == 0 || (seeds_per_query >= 1 && seeds_per_query <= 256), "seeds_per_query must be in [1,256]");
    if (h->entry) grab_entry_layer_destroy(h->entry);
    h->entry = nullptr;
    h->entry_rows = 0;
    h->scan_rows = 0;
    h->ts_pivot_rows = 0;
    h->entry_samples = num_samples;
    h->entry_seeds = seeds_per_query;
    return GRAB_OK;
}

int grab_index_set_entry_groups(grab_index* h, uint32_t num_groups, uint32_t nprobe, uint32_t min_rows) {
    GRAB_REQUIRE(h != nullptr, "null index");
    GRAB_REQUIRE(num_groups == 0 || (nprobe >= 1 && nprobe <= 64), "nprobe must be in [1,64]");
    if (h->entry) grab_entry_layer_destroy(h->entry);
    h->entry = nullptr;
    h->entry_rows = 0;
    h->scan_rows = 0;
    h->ts_pivot_rows = 0;
    h->entry_groups = num_groups;
    h->entry_nprobe = nprobe;
    h->entry_min_rows = min_rows;
    return GRAB_OK;
}

int grab_index_debug_fail_insert(grab_index* h, int inner_step) {
    GRAB_REQUIRE(h != nullptr, "null index");
    h->fail_insert_at = inner_step;
    return GRAB_OK;
}

int grab_index_set_entry_list(grab_index* h, uint32_t max_rows) {
    GRAB_REQUIRE(h != nullptr, "null index");
    GRAB_REQUIRE(max_rows <= 64, "at most 64 listed rows per query");
    h->entry_list = max_rows;
    return GRAB_OK;
}

int grab_index_set_batch_chunk(grab_index* h, size_t queries_per_chunk) {
    GRAB_REQUIRE(h != nullptr, "null index");
    GRAB_REQUIRE(queries_per_chunk == 0 || queries_per_chunk >= 256, "a chunk holds at least 256 queries (0 = no chunks)");
    h->chunk_queries = queries_per_chunk;
    return GRAB_OK;
}

int grab_index_set_build_params(grab_index* h, uint32_t intermediate_degree, uint32_t graph_degree) {
    GRAB_REQUIRE(h != nullptr, "null index");
    GRAB_REQUIRE(graph_degree == h->degree, "graph_degree is fixed at construction (the reference's buffers are sized by it)");
    GRAB_REQUIRE(intermediate_degree >= graph_degree && intermediate_degree <= GRAB_MAX_DEGREE, "bad intermediate degree");
    h->build_params = {intermediate_degree, graph_degree};
    return GRAB_OK;
}
int grab_index_set_query_params(grab_index* h, uint32_t itopk, uint32_t sw, uint32_t min_it, uint32_t max_it, uint32_t bitlen) {
    GRAB_REQUIRE(h != nullptr, "null index");
    h->search_params = {itopk, sw, min_it, max_it, bitlen};
    return GRAB_OK;
}
int grab_index_set_insert_params(grab_index* h, uint32_t itopk, uint32_t sw, uint32_t min_it, uint32_t max_it, uint32_t bitlen) {
    GRAB_REQUIRE(h != nullptr, "null index");
    h->insert_params = {itopk, sw, min_it, max_it, bitlen};
    return GRAB_OK;
}

// CagraIndex::add, src/cagraIndex.cu:48-75: host accumulation, timestamps mirrored to the device
int grab_index_add(grab_index* h, size_t n, const float* vectors, const uint64_t* timestamps) {
    GRAB_REQUIRE(h != nullptr, "null index");
    if (n == 0) return GRAB_OK;
    GRAB_REQUIRE(vectors != nullptr, "null vectors");
    const size_t old = h->h_data.size() / h->dim;
    GRAB_REQUIRE(old + n < (1ull << 31), "index too large");
    h->h_data.insert(h->h_data.end(), vectors, vectors + n * h->dim);
    if (timestamps) {
        GRAB_REQUIRE(h->h_ts.size() == old, "timestamps must be given for every row or for none");
        for (size_t i = 0; i < n; ++i) {
            h->h_ts.push_back(timestamps[i]);
            h->ts_to_ids[timestamps[i]].push_back((uint32_t)(old + i));
        }
        GRAB_TRY(grab_vmm_resize(h->d_ts, h->h_ts.size() * sizeof(uint64_t)));
        GRAB_HIP(hipMemcpy(static_cast<uint64_t*>(grab_vmm_data(h->d_ts)) + old, timestamps, n * sizeof(uint64_t),
                           hipMemcpyHostToDevice));
        h->ts_order_stale = true;
        h->entry_rows = 0;  // the entry-point layer samples the rows present
        h->scan_rows = 0;
        h->ts_pivot_rows = 0;
    }
    h->built = false;  // rows added after a build are not in the graph until build() runs again
    return GRAB_OK;
}

int grab_index_set_labels(grab_index* h, size_t n, const uint8_t* labels) {
    GRAB_REQUIRE(h && labels, "null pointer");
    GRAB_REQUIRE(n == h->h_data.size() / h->dim, "one label per row");
    for (size_t i = 0; i < n; ++i) GRAB_REQUIRE(labels[i] < 64, "labels must be below 64");
    h->h_labels.assign(labels, labels + n);
    h->labels_stale = true;
    return GRAB_OK;
}

// CagraIndex::build, src/cagraIndex.cu:80-124
int grab_index_build(grab_index* h) {
    GRAB_REQUIRE(h != nullptr, "null index");
    const size_t n = h->h_data.size() / h->dim;
    if (n == 0) return GRAB_OK;
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    GRAB_TRY(grab_vmm_resize(h->d_data, n * h->dim * sizeof(float)));
    GRAB_TRY(grab_vmm_resize(h->d_graph, n * h->degree * sizeof(uint32_t)));
    float* d_data = static_cast<float*>(grab_vmm_data(h->d_data));
    uint32_t* d_graph = static_cast<uint32_t*>(grab_vmm_data(h->d_graph));
    GRAB_HIP(hipMemcpy(d_data, h->h_data.data(), n * h->dim * sizeof(float), hipMemcpyHostToDevice));
    const auto t1 = clk::now();
    {
        DeviceScratch knn;
        GRAB_HIP(knn.alloc(n * h->build_params.intermediate_degree * sizeof(uint32_t)));
        GRAB_TRY(grab_generate_knn_graph(d_data, n, h->dim, h->build_params.intermediate_degree, h->metric,
                                         knn.as<uint32_t>(), nullptr, h->stream));
        const auto t2 = clk::now();
        GRAB_TRY(grab_build_graph(d_data, n, knn.as<uint32_t>(), h->build_params, d_graph, h->stream));
        const auto t3 = clk::now();
        h->knn_s = std::chrono::duration<double>(t2 - t1).count();
        h->opt_s = std::chrono::duration<double>(t3 - t2).count();
    }
    h->h_graph.resize(n * h->degree);
    GRAB_HIP(hipMemcpy(h->h_graph.data(), d_graph, n * h->degree * sizeof(uint32_t), hipMemcpyDeviceToHost));
    h->size = n;
    h->built = true;
    h->host_graph_stale = false;
    h->ts_order_stale = true;
    h->entry_rows = 0;  // the entry-point layer samples the rows present
    h->scan_rows = 0;
    h->ts_pivot_rows = 0;
    h->total_s = std::chrono::duration<double>(clk::now() - t0).count();
    return GRAB_OK;
}

namespace {
// test hook (grab_index_debug_fail_insert): fails the insert before inner step `step`, once
int injected_failure(grab_index* h, size_t step) {
    if (h->fail_insert_at < 0 || (size_t)h->fail_insert_at != step) return GRAB_OK;
    h->fail_insert_at = -1;
    set_error("insert: failure injected before inner step %zu (grab_index_debug_fail_insert)", step);
    return GRAB_ERR_STATE;
}

// a failed insert: the host copies drop the rows from `old` on (their timestamps, n of them, were recorded under these keys)
void forget_rows_from(grab_index* h, size_t old, const uint64_t* timestamps, size_t n) {
    h->h_data.resize(old * h->dim);
    h->h_graph.resize(old * h->degree);
    if (timestamps == nullptr) return;
    h->h_ts.resize(old);
    for (size_t i = 0; i < n; ++i) {
        auto it = h->ts_to_ids.find(timestamps[i]);
        if (it == h->ts_to_ids.end()) continue;
        while (!it->second.empty() && it->second.back() >= old) it->second.pop_back();
        if (it->second.empty()) h->ts_to_ids.erase(it);
    }
}
}  // namespace

// CagraIndex::insert, src/cagraIndex.cu:129-183
int grab_index_insert(grab_index* h, size_t n, const float* vectors, const uint64_t* timestamps) {
    GRAB_REQUIRE(h != nullptr, "null index");
    if (n == 0) return GRAB_OK;
    GRAB_REQUIRE(vectors != nullptr, "null vectors");
    if (h->size == 0 || !h->built) {  // empty index: add + build (:134-138)
        GRAB_TRY(grab_index_add(h, n, vectors, timestamps));
        return grab_index_build(h);
    }
    const size_t old = h->size, total = old + n;
    GRAB_REQUIRE(total < (1ull << 31), "index too large");
    GRAB_REQUIRE((timestamps != nullptr) == (h->h_ts.size() == old) || h->h_ts.empty(),
                 "timestamps must be given for every row or for none");
    GRAB_TRY(grab_vmm_resize(h->d_data, total * h->dim * sizeof(float)));
    GRAB_TRY(grab_vmm_resize(h->d_graph, total * h->degree * sizeof(uint32_t)));
    if (timestamps && h->h_ts.size() == old) GRAB_TRY(grab_vmm_resize(h->d_ts, total * sizeof(uint64_t)));
    const bool with_ts = timestamps && h->h_ts.size() == old;
    h->h_data.insert(h->h_data.end(), vectors, vectors + n * h->dim);
    h->h_graph.resize(total * h->degree, GRAB_INVALID_ID);
    // the reference drops the timestamps of inserted rows (src/cagraIndex.cu:129-183 never
    // touches h_timestamps_ / ts_to_ids_ / d_ts_vmm_); they are recorded here so that a range
    // query after an insert sees the new rows
    if (with_ts) {
        for (size_t i = 0; i < n; ++i) {
            h->h_ts.push_back(timestamps[i]);
            h->ts_to_ids[timestamps[i]].push_back((uint32_t)(old + i));
        }
    }
    auto device_work = [&]() -> int {
        float* d_data = static_cast<float*>(grab_vmm_data(h->d_data));
        uint32_t* d_graph = static_cast<uint32_t*>(grab_vmm_data(h->d_graph));
        GRAB_HIP(hipMemcpyAsync(d_data + old * h->dim, vectors, n * h->dim * sizeof(float), hipMemcpyHostToDevice, h->stream));
        if (with_ts)
            GRAB_HIP(hipMemcpyAsync(static_cast<uint64_t*>(grab_vmm_data(h->d_ts)) + old, timestamps, n * sizeof(uint64_t),
                                    hipMemcpyHostToDevice, h->stream));
        GRAB_TRY(h->ins_ws.ensure(insert_workspace_bytes(64, h->degree)));
        const size_t batch = 64;  // :165
        for (size_t off = 0; off < n; off += batch) {
            const size_t cur = std::min(batch, n - off);
            GRAB_TRY(injected_failure(h, off / batch));
            GRAB_TRY(insert_impl(d_data, h->dim, old + off, cur, d_data + (old + off) * h->dim, d_graph, h->degree,
                                 h->insert_params, h->metric, &h->rng, h->flags, (h->flags & GRAB_FLAG_STRICT_REFERENCE) ? 1 : 0,
                                 h->ins_ws.ptr, h->stream));
        }
        GRAB_HIP(hipStreamSynchronize(h->stream));
        return GRAB_OK;
    };
    const uint64_t rng_before = h->rng;
    const int rc = device_work();
    if (rc != GRAB_OK) {
        // nothing may still read the caller's buffers, and the host copies, the row count and the generator go back to
        // what they were: searches see the old rows and draw the masks they would have drawn.  (h->size is unchanged.
        // Old rows of the device graph may hold edges to ids of the failed batch already: the search kernels skip ids
        // beyond the row count, and once later inserts reuse those ids the edges lead to the rows that then carry them.)
        (void)hipStreamSynchronize(h->stream);
        forget_rows_from(h, old, with_ts ? timestamps : nullptr, n);
        h->rng = rng_before;
        h->host_graph_stale = true;
        return rc;
    }
    if (with_ts) {
        h->ts_order_stale = true;
        h->entry_rows = 0;  // the entry-point layer samples the rows present
        h->scan_rows = 0;
        h->ts_pivot_rows = 0;
    }
    h->size = total;
    h->host_graph_stale = true;
    h->labels_stale = true;
    return GRAB_OK;
}

// CagraIndexOpt::insert, src/cagraIndexOpt.cu:557-652
int grab_index_insert_partitioned(grab_index* h, size_t n, const float* vectors, const uint64_t* timestamps) {
    GRAB_REQUIRE(h != nullptr, "null index");
    if (n == 0) return GRAB_OK;
    GRAB_REQUIRE(vectors && timestamps, "null vectors or timestamps");
    GRAB_REQUIRE(h->local_degree >= 1 && h->local_degree < h->degree, "the index has no local/remote split");
    GRAB_TRY(require_built(h));
    GRAB_REQUIRE(h->h_ts.size() == h->size, "the index holds rows without timestamps");
    const uint64_t target_ts = timestamps[0];  // :561
    const size_t old = h->size, total = old + n;
    GRAB_REQUIRE(total < (1ull << 31), "index too large");
    GRAB_TRY(grab_vmm_resize(h->d_data, total * h->dim * sizeof(float)));
    GRAB_TRY(grab_vmm_resize(h->d_graph, total * h->degree * sizeof(uint32_t)));
    GRAB_TRY(grab_vmm_resize(h->d_ts, total * sizeof(uint64_t)));
    h->h_data.insert(h->h_data.end(), vectors, vectors + n * h->dim);
    h->h_graph.resize(total * h->degree, GRAB_INVALID_ID);
    for (size_t i = 0; i < n; ++i) {
        h->h_ts.push_back(timestamps[i]);
        h->ts_to_ids[timestamps[i]].push_back((uint32_t)(old + i));
    }
    auto device_work = [&]() -> int {
        float* d_data = static_cast<float*>(grab_vmm_data(h->d_data));
        uint32_t* d_graph = static_cast<uint32_t*>(grab_vmm_data(h->d_graph));
        uint64_t* d_ts = static_cast<uint64_t*>(grab_vmm_data(h->d_ts));
        GRAB_HIP(hipMemcpyAsync(d_data + old * h->dim, vectors, n * h->dim * sizeof(float), hipMemcpyHostToDevice, h->stream));
        GRAB_HIP(hipMemcpyAsync(d_ts + old, timestamps, n * sizeof(uint64_t), hipMemcpyHostToDevice, h->stream));
        h->ts_order_stale = true;
        h->labels_stale = true;
        h->entry_rows = 0;
        h->scan_rows = 0;
        h->ts_pivot_rows = 0;
        h->host_graph_stale = true;
        h->size = total;  // the rows are in place; their adjacency rows are filled step by step below

        const uint32_t n_seeds = std::max(32u, h->search_params.itopk_size);  // :576, read before the overwrite
        h->search_params = grab_search_params{128, 4, 0, 100, 14};           // :581-587
        const size_t batch = 32;                                             // :575
        GRAB_TRY(h->ins_ws.ensure(insert_partitioned_workspace_bytes(batch, h->search_params.itopk_size, h->degree)));
        const std::vector<uint32_t>& bucket = h->ts_to_ids[target_ts];
        // The seeds of every step are drawn up front and uploaded once, so that the steps follow each other on the stream
        // without a host round trip.  The generator is consumed in the order of a step-by-step run: one draw for a
        // step's sample (when the bucket is larger than the seed list), then the two masks of its searches.
        std::vector<uint32_t> seeds_host(n * n_seeds, GRAB_INVALID_ID);
        std::vector<uint8_t> sampled((n + batch - 1) / batch, 0);
        {
            uint64_t rng = h->rng;
            size_t done = old;
            for (size_t off = 0, step = 0; off < n; off += batch, ++step) {
                const size_t cur = std::min(batch, n - off);
                uint32_t* first = seeds_host.data() + off * n_seeds;
                // old rows of the bucket: the id list ascends, so they are a prefix (:599-608)
                const size_t n_old = std::lower_bound(bucket.begin(), bucket.end(), (uint32_t)done) - bucket.begin();
                if (n_old <= n_seeds) {
                    std::copy(bucket.begin(), bucket.begin() + n_old, first);
                } else {  // std::sample with a std::random_device seed in the reference (:611-620)
                    std::mt19937 gen((uint32_t)splitmix64(&rng));
                    std::sample(bucket.begin(), bucket.begin() + n_old, first, n_seeds, gen);
                    sampled[step] = 1;
                }
                for (size_t i = 1; i < cur; ++i) std::copy(first, first + n_seeds, first + i * n_seeds);
                (void)splitmix64(&rng);  // the masks of the step's two searches
                (void)splitmix64(&rng);
                done += cur;
            }
        }
        GRAB_TRY(h->seeds.ensure(seeds_host.size() * sizeof(uint32_t)));
        GRAB_HIP(hipMemcpyAsync(h->seeds.ptr, seeds_host.data(), seeds_host.size() * sizeof(uint32_t), hipMemcpyHostToDevice, h->stream));
        GRAB_HIP(hipStreamSynchronize(h->stream));  // seeds_host may go out of scope on an error below
        if (h->side.stream == nullptr) {
            GRAB_HIP(hipStreamCreate(&h->side.stream));
            GRAB_HIP(hipEventCreateWithFlags(&h->side.fork, hipEventDisableTiming));
            GRAB_HIP(hipEventCreateWithFlags(&h->side.join, hipEventDisableTiming));
        }
        size_t done = old;
        for (size_t off = 0, step = 0; off < n; off += batch, ++step) {
            const size_t cur = std::min(batch, n - off);
            if (sampled[step]) (void)splitmix64(&h->rng);
            GRAB_TRY(injected_failure(h, step));
            GRAB_TRY(insert_partitioned_impl(d_data, d_graph, d_ts, static_cast<const uint32_t*>(h->seeds.ptr) + off * n_seeds, done, cur,
                                             target_ts, h->dim, h->degree, h->local_degree, h->search_params, n_seeds, h->metric,
                                             &h->rng, h->flags, h->ins_ws.ptr, h->stream, &h->side));
            done += cur;
        }
        GRAB_HIP(hipStreamSynchronize(h->stream));
        return GRAB_OK;
    };
    const uint64_t rng_before = h->rng;
    const grab_search_params params_before = h->search_params;
    const int rc = device_work();
    if (rc != GRAB_OK) {
        // nothing may still read the caller's buffers; host copies, row count, generator and query parameters go back to
        // what they were (the flags that mark derived tables stale stay set: the tables are remade on demand).  As after
        // a failed CagraIndex::insert, old rows of the device graph may hold edges to ids of the failed batch.
        (void)hipStreamSynchronize(h->stream);
        if (h->side.stream != nullptr) (void)hipStreamSynchronize(h->side.stream);
        forget_rows_from(h, old, timestamps, n);
        h->size = old;
        h->rng = rng_before;
        h->search_params = params_before;
    }
    return rc;
}

// CagraIndex::query, src/cagraIndex.cu:188-235
int grab_index_search(grab_index* h, const float* queries, size_t nq, int k, int64_t* indices, float* dists,
                      const uint32_t* seeds, size_t seeds_per_query) {
    GRAB_REQUIRE(h && indices && dists, "null pointer");
    if (h->h_data.empty()) return GRAB_OK;  // :196
    GRAB_TRY(require_built(h));
    if (nq == 0) return GRAB_OK;
    GRAB_TRY(stage_queries(h, queries, nq, k));
    const uint32_t* d_seeds = nullptr;
    if (seeds && seeds_per_query > 0) {
        GRAB_TRY(upload(h, h->seeds, seeds, nq * seeds_per_query * sizeof(uint32_t)));
        d_seeds = static_cast<const uint32_t*>(h->seeds.ptr);
    }
    grab_search_desc d;
    base_desc(h, &d, GRAB_WRAP_SEARCH, nq, k, h->degree, d_seeds, (uint32_t)seeds_per_query);
    GRAB_TRY(run_desc(h, d));
    return fetch_results(h, nq, k, indices, dists);
}

// CagraIndex::query_range, src/cagraIndex.cu:237-347
int grab_index_search_range(grab_index* h, const float* queries, size_t nq, int k, float range_radius,
                            uint64_t start_ts, uint64_t end_ts, int64_t* indices, float* dists, const uint32_t* seeds,
                            size_t seeds_per_query) {
    GRAB_REQUIRE(h && indices && dists, "null pointer");
    if (h->h_data.empty()) return GRAB_OK;  // :248
    if (range_radius >= 0.99f) return grab_index_search(h, queries, nq, k, indices, dists, seeds, seeds_per_query);  // :323-338
    GRAB_TRY(require_built(h));
    GRAB_REQUIRE(h->h_ts.size() >= h->size, "the index holds rows without timestamps");
    if (nq == 0) return GRAB_OK;
    if (h->entry_samples > 0) {
        GRAB_TRY(stage_queries(h, queries, nq, k));
        RangeStage g;
        GRAB_TRY(own_stage(h, nq, 0, &g));
        GRAB_TRY(search_range_with_layer(h, g, nq, k, nullptr, nullptr, start_ts, end_ts, 0));
        return fetch_results(h, nq, k, indices, dists);
    }
    // one seed set for the batch, itopk_size of the ids inside the window (:268-295); the
    // map is entered at the window's lower bound instead of being walked from the start
    const size_t want = h->search_params.itopk_size;
    std::vector<uint32_t> in_window;
    for (auto it = h->ts_to_ids.lower_bound(start_ts); it != h->ts_to_ids.end() && it->first < end_ts; ++it)
        for (uint32_t id : it->second)
            if (id < h->size) in_window.push_back(id);
    if (in_window.empty()) {
        fill_empty(nq, k, indices, dists);
        return GRAB_OK;
    }
    std::vector<uint32_t> picked = sample_ids(h, in_window, want);
    // the reference pads a short seed list with zeros, i.e. with node 0 (:291); by default the
    // padding is an invalid id instead, which the kernel replaces by a random row
    const uint32_t pad = (h->flags & GRAB_FLAG_STRICT_REFERENCE) ? 0u : GRAB_INVALID_ID;
    std::vector<uint32_t> all(nq * want, pad);
    for (size_t i = 0; i < nq; ++i) std::copy(picked.begin(), picked.end(), all.begin() + i * want);
    GRAB_TRY(stage_queries(h, queries, nq, k));
    GRAB_TRY(upload(h, h->seeds, all.data(), all.size() * sizeof(uint32_t)));
    grab_search_desc d;
    base_desc(h, &d, GRAB_WRAP_RANGE, nq, k, h->degree, static_cast<const uint32_t*>(h->seeds.ptr), (uint32_t)want);
    d.filter_kind = 1;
    d.d_ts = static_cast<const uint64_t*>(grab_vmm_data(h->d_ts));
    d.win_start = start_ts;
    d.win_end = end_ts;
    GRAB_TRY(attach_neighbor_timestamps(h, d, nq));
    GRAB_TRY(run_desc(h, d));
    return fetch_results(h, nq, k, indices, dists);
}

int grab_index_search_range_batch(grab_index* h, const float* queries, size_t nq, int k, const uint64_t* start_ts,
                                  const uint64_t* end_ts, int64_t* indices, float* dists) {
    GRAB_REQUIRE(h && indices && dists && start_ts && end_ts, "null pointer");
    if (h->h_data.empty()) return GRAB_OK;
    GRAB_TRY(require_built(h));
    if (nq == 0) return GRAB_OK;
    GRAB_REQUIRE(queries != nullptr && k >= 1, "null queries, or k not positive");
    GRAB_TRY(ensure_ts_order(h));
    if (h->scan_below > 0.0 && h->ts_monotone && k <= 128) {
        // narrow windows are scanned, the others searched: the batch is cut in two by the width of the windows (in rows)
        const size_t n = h->size;
        const double most = h->scan_below * (double)n;
        std::vector<uint32_t> narrow, wide;
        for (size_t i = 0; i < nq; ++i) {
            const size_t lo = first_row_at(h, start_ts[i]), hi = first_row_at(h, end_ts[i]);
            ((hi > lo ? (double)(hi - lo) : 0.0) <= most ? narrow : wide).push_back((uint32_t)i);
        }
        if (!narrow.empty()) {
            if (wide.empty()) return grab_index_scan_range_batch(h, queries, nq, k, start_ts, end_ts, indices, dists);
            const double keep = h->scan_below;
            h->scan_below = 0.0;  // the two halves are calls of this function and of the scan
            int rc = GRAB_OK;
            for (int part = 0; part < 2 && rc == GRAB_OK; ++part) {
                const std::vector<uint32_t>& which = part == 0 ? narrow : wide;
                const size_t m = which.size();
                std::vector<float> q(m * h->dim), d(m * (size_t)k);
                std::vector<uint64_t> s0(m), s1(m);
                std::vector<int64_t> ids(m * (size_t)k);
                for (size_t j = 0; j < m; ++j) {
                    std::copy(queries + (size_t)which[j] * h->dim, queries + (size_t)(which[j] + 1) * h->dim, q.begin() + j * h->dim);
                    s0[j] = start_ts[which[j]];
                    s1[j] = end_ts[which[j]];
                }
                rc = part == 0 ? grab_index_scan_range_batch(h, q.data(), m, k, s0.data(), s1.data(), ids.data(), d.data())
                               : grab_index_search_range_batch(h, q.data(), m, k, s0.data(), s1.data(), ids.data(), d.data());
                for (size_t j = 0; j < m && rc == GRAB_OK; ++j) {
                    std::copy(ids.begin() + j * k, ids.begin() + (j + 1) * k, indices + (size_t)which[j] * k);
                    std::copy(d.begin() + j * k, d.begin() + (j + 1) * k, dists + (size_t)which[j] * k);
                }
            }
            h->scan_below = keep;
            return rc;
        }
    }
    // the coarse level's walk answers from scratch that a lane can own: such batches are cut over two lanes
    if (h->entry_samples > 0 && h->entry_groups > 0 && h->entry_groups <= 1024 && h->ts_monotone && h->chunk_queries >= 256 &&
        nq > h->chunk_queries && std::min(h->entry_seeds, std::max(h->search_params.itopk_size, 64u)) <= 64)
        return search_range_batch_chunked(h, queries, nq, k, start_ts, end_ts, indices, dists);
    GRAB_TRY(stage_queries(h, queries, nq, k));
    GRAB_TRY(upload(h, h->win_s, start_ts, nq * sizeof(uint64_t)));
    GRAB_TRY(upload(h, h->win_e, end_ts, nq * sizeof(uint64_t)));
    if (h->entry_samples > 0) {
        RangeStage g;
        GRAB_TRY(own_stage(h, nq, 1, &g));
        GRAB_TRY(search_range_with_layer(h, g, nq, k, static_cast<const uint64_t*>(h->win_s.ptr),
                                         static_cast<const uint64_t*>(h->win_e.ptr), 0, 0, 1));
        return fetch_results(h, nq, k, indices, dists);
    }
    const uint32_t want = h->search_params.itopk_size;
    GRAB_TRY(h->seeds.ensure(nq * (size_t)want * sizeof(uint32_t)));
    const uint64_t seed = splitmix64(&h->rng);
    GRAB_TRY(sample_window_seeds_async(static_cast<const uint64_t*>(h->sorted_ts.ptr),
                                       static_cast<const uint32_t*>(h->ids_by_ts.ptr), h->size,
                                       static_cast<const uint64_t*>(h->win_s.ptr), static_cast<const uint64_t*>(h->win_e.ptr),
                                       0, 0, 1, nq, want, seed, static_cast<uint32_t*>(h->seeds.ptr), h->stream));
    grab_search_desc d;
    base_desc(h, &d, GRAB_WRAP_RANGE, nq, k, h->degree, static_cast<const uint32_t*>(h->seeds.ptr), want);
    d.filter_kind = 1;
    d.d_ts = static_cast<const uint64_t*>(grab_vmm_data(h->d_ts));
    d.d_win_start = static_cast<const uint64_t*>(h->win_s.ptr);
    d.d_win_end = static_cast<const uint64_t*>(h->win_e.ptr);
    d.per_query_window = 1;
    GRAB_TRY(attach_neighbor_timestamps(h, d, nq));
    GRAB_TRY(run_desc(h, d));
    return fetch_results(h, nq, k, indices, dists);
}

// Exact answers for per-query windows: with rows in timestamp order a window is an interval of row ids, and the
// intervals are scanned on the matrix cores (grab_scan_base_window_topk); in any other order every row is scanned
// with the window test.  Empty windows are reported like query_range_batch reports them.
int grab_index_scan_range_batch(grab_index* h, const float* queries, size_t nq, int k, const uint64_t* start_ts,
                                const uint64_t* end_ts, int64_t* indices, float* dists) {
    GRAB_REQUIRE(h && indices && dists && start_ts && end_ts, "null pointer");
    if (h->h_data.empty()) return GRAB_OK;
    if (nq == 0) return GRAB_OK;
    GRAB_REQUIRE(queries != nullptr && k >= 1 && k <= 128, "null queries, or k outside [1,128]");
    GRAB_REQUIRE(h->h_ts.size() >= h->size, "the index holds rows without timestamps");
    const size_t n = h->size;
    const float* d_data = static_cast<const float*>(grab_vmm_data(h->d_data));
    GRAB_TRY(ensure_ts_order(h));  // whether the timestamps ascend with the row id is found once per change of the rows
    if (h->ts_monotone) {
        if (h->scan == nullptr || h->scan_rows != n) {
            grab_scan_base_destroy(h->scan);
            h->scan = nullptr;
            GRAB_TRY(grab_scan_base_create(d_data, n, h->dim, h->metric, &h->scan));
            h->scan_rows = n;
        }
        // Queries and windows cross through page-locked staging (the pipe's, filled by the calling thread and its helpers)
        // and a copy kernel; a kernel turns the windows into intervals of row ids and writes them where the host reads
        // them (20,000 searches of a million timestamps take the host half a millisecond); the results come back
        // through page-locked memory that the re-scoring writes itself.
        const size_t q_bytes = nq * h->dim * sizeof(float), w_bytes = nq * sizeof(uint64_t);
        const size_t ids_bytes = nq * (size_t)k * sizeof(int64_t), dist_bytes = (nq * (size_t)k * sizeof(float) + 7) & ~(size_t)7;
        BatchPipe& p = h->pipe;
        GRAB_TRY(pipe_ready(h, nq, 1, q_bytes + 2 * w_bytes, ids_bytes + dist_bytes + 2 * w_bytes, 1));
        GRAB_TRY(h->q.ensure(q_bytes + 2 * w_bytes));
        pipe_stage(p, queries, q_bytes, start_ts, end_ts, w_bytes);
        GRAB_TRY(device_copy_async(h->q.ptr, p.h_in, q_bytes + 2 * w_bytes, h->stream, 32));
        const uint64_t* d_ws = reinterpret_cast<const uint64_t*>(static_cast<const char*>(h->q.ptr) + q_bytes);
        int64_t* out_i = static_cast<int64_t*>(p.h_out);
        float* out_d = reinterpret_cast<float*>(static_cast<char*>(p.h_out) + ids_bytes);
        uint64_t* lo = reinterpret_cast<uint64_t*>(static_cast<char*>(p.h_out) + ids_bytes + dist_bytes);
        GRAB_TRY(grab_windows_to_id_ranges(static_cast<const uint64_t*>(grab_vmm_data(h->d_ts)), n, d_ws, d_ws + nq, nq, lo, lo + nq, h->stream));
        GRAB_HIP(hipStreamSynchronize(h->stream));
        GRAB_TRY(grab_scan_base_window_topk(h->scan, static_cast<const float*>(h->q.ptr), nq, (uint32_t)k, lo, lo + nq, out_i, out_d, nullptr,
                                            h->stream));  // returns with the stream drained
        std::memcpy(indices, out_i, ids_bytes);
        for (size_t i = 0; i < nq * (size_t)k; ++i) dists[i] = out_i[i] < 0 ? -1.0f : out_d[i];  // :479-485 of cagraIndexOpt.cu
        return GRAB_OK;
    } else {
        GRAB_TRY(stage_queries(h, queries, nq, k));
        GRAB_TRY(upload(h, h->win_s, start_ts, nq * sizeof(uint64_t)));
        GRAB_TRY(upload(h, h->win_e, end_ts, nq * sizeof(uint64_t)));
        GRAB_TRY(grab_bruteforce_topk(d_data, n, h->dim, static_cast<const float*>(h->q.ptr), nq, (uint32_t)k, h->metric, 1,
                                      static_cast<const uint64_t*>(grab_vmm_data(h->d_ts)), static_cast<const uint64_t*>(h->win_s.ptr),
                                      static_cast<const uint64_t*>(h->win_e.ptr), 0, 0, 1, nullptr, nullptr,
                                      static_cast<int64_t*>(h->out_i.ptr), static_cast<float*>(h->out_d.ptr), nullptr, h->stream));
    }
    GRAB_TRY(fetch_results(h, nq, k, indices, dists));
    for (size_t i = 0; i < nq * (size_t)k; ++i)
        if (indices[i] < 0) dists[i] = -1.0f;  // the way an empty window or a short one is reported (src/cagraIndexOpt.cu:479-485)
    return GRAB_OK;
}

// CagraIndexOpt::query_local, src/cagraIndexOpt.cu:301-420
int grab_index_search_bucket(grab_index* h, const float* queries, size_t nq, int k, uint64_t target_ts, int64_t* indices,
                             float* dists) {
    GRAB_REQUIRE(h && indices && dists, "null pointer");
    if (h->h_data.empty()) return GRAB_OK;
    GRAB_TRY(require_built(h));
    if (nq == 0) return GRAB_OK;
    const size_t want = std::max(32u, h->search_params.itopk_size);  // :312
    auto it = h->ts_to_ids.find(target_ts);
    std::vector<uint32_t> bucket;
    if (it != h->ts_to_ids.end())
        for (uint32_t id : it->second)
            if (id < h->size) bucket.push_back(id);
    if (bucket.empty()) {
        fill_empty(nq, k, indices, dists);
        return GRAB_OK;
    }
    std::vector<uint32_t> picked = sample_ids(h, bucket, want);
    const size_t per_q = picked.size();
    std::vector<uint32_t> all(nq * per_q);
    for (size_t i = 0; i < nq; ++i) std::copy(picked.begin(), picked.end(), all.begin() + i * per_q);
    GRAB_TRY(stage_queries(h, queries, nq, k));
    GRAB_TRY(upload(h, h->seeds, all.data(), all.size() * sizeof(uint32_t)));
    grab_search_desc d;
    base_desc(h, &d, GRAB_WRAP_BUCKET, nq, k, h->local_degree, static_cast<const uint32_t*>(h->seeds.ptr), (uint32_t)per_q);
    GRAB_TRY(run_desc(h, d));
    return fetch_results(h, nq, k, indices, dists);
}

int grab_index_search_mask(grab_index* h, const float* queries, size_t nq, int k, const uint64_t* masks, int64_t* indices,
                           float* dists) {
    GRAB_REQUIRE(h && indices && dists && masks, "null pointer");
    if (h->h_data.empty()) return GRAB_OK;
    GRAB_TRY(require_built(h));
    GRAB_REQUIRE(h->h_labels.size() >= h->size, "labels are missing: call grab_index_set_labels");
    if (nq == 0) return GRAB_OK;
    if (h->labels_stale) {
        GRAB_TRY(upload(h, h->labels, h->h_labels.data(), h->size));
        h->label_ids.assign(64, {});
        for (size_t i = 0; i < h->size; ++i) h->label_ids[h->h_labels[i]].push_back((uint32_t)i);
        h->labels_stale = false;
    }
    // seeds: round-robin over the query's allowed labels, one random row of the label each
    const uint32_t want = h->search_params.itopk_size;
    std::vector<uint32_t> all(nq * (size_t)want, GRAB_INVALID_ID);
    bool any = false;
    for (size_t qi = 0; qi < nq; ++qi) {
        uint32_t allowed[64], na = 0;
        for (uint32_t b = 0; b < 64; ++b)
            if (((masks[qi] >> b) & 1ull) && !h->label_ids[b].empty()) allowed[na++] = b;
        if (na == 0) continue;
        any = true;
        for (uint32_t i = 0; i < want; ++i) {
            const auto& ids = h->label_ids[allowed[i % na]];
            all[qi * want + i] = ids[splitmix64(&h->rng) % ids.size()];
        }
    }
    if (!any) {
        fill_empty(nq, k, indices, dists);
        return GRAB_OK;
    }
    GRAB_TRY(stage_queries(h, queries, nq, k));
    GRAB_TRY(upload(h, h->seeds, all.data(), all.size() * sizeof(uint32_t)));
    GRAB_TRY(upload(h, h->masks, masks, nq * sizeof(uint64_t)));
    grab_search_desc d;
    base_desc(h, &d, GRAB_WRAP_RANGE, nq, k, h->degree, static_cast<const uint32_t*>(h->seeds.ptr), want);
    d.filter_kind = 2;
    d.d_labels = static_cast<const uint8_t*>(h->labels.ptr);
    d.d_masks = static_cast<const uint64_t*>(h->masks.ptr);
    GRAB_TRY(run_desc(h, d));
    return fetch_results(h, nq, k, indices, dists);
}

size_t grab_index_size(const grab_index* h) { return h ? h->h_data.size() / h->dim : 0; }  // cagraIndex.hpp:96
const float* grab_index_get_data(const grab_index* h) { return h ? h->h_data.data() : nullptr; }

const uint32_t* grab_index_get_graph(grab_index* h) {
    if (!h || h->size == 0) return nullptr;
    if (h->host_graph_stale) {
        h->h_graph.resize(h->size * h->degree);
        if (hipMemcpy(h->h_graph.data(), grab_vmm_data(h->d_graph), h->size * h->degree * sizeof(uint32_t),
                      hipMemcpyDeviceToHost) != hipSuccess)
            return nullptr;
        h->host_graph_stale = false;
    }
    return h->h_graph.data();
}

size_t grab_index_ids_by_timestamp(const grab_index* h, uint64_t ts, uint32_t* out, size_t cap) {
    if (!h) return 0;
    auto it = h->ts_to_ids.find(ts);
    if (it == h->ts_to_ids.end()) return 0;
    if (out)
        for (size_t i = 0; i < it->second.size() && i < cap; ++i) out[i] = it->second[i];
    return it->second.size();
}

// CagraIndexOpt::sample_seeds_by_time, src/cagraIndexOpt.cu:95-131: ids with min_ts <= timestamp <=
// max_ts (inclusive), collection cut off once more than 100*num are gathered, then std::sample of num
// with a std::mt19937 seeded 1234 (one generator per index here, one per process in the reference)
size_t grab_index_sample_seeds_by_time(grab_index* h, uint64_t min_ts, uint64_t max_ts, size_t num, uint32_t* out, size_t cap) {
    if (!h || num == 0) return 0;
    std::vector<uint32_t> candidates;
    const auto it_end = h->ts_to_ids.upper_bound(max_ts);
    for (auto it = h->ts_to_ids.lower_bound(min_ts); it != it_end; ++it) {
        candidates.insert(candidates.end(), it->second.begin(), it->second.end());
        if (candidates.size() > num * 100) break;
    }
    if (candidates.empty()) return 0;
    std::vector<uint32_t> result;
    result.reserve(num);
    std::sample(candidates.begin(), candidates.end(), std::back_inserter(result), num, h->seed_rng);
    if (out)
        for (size_t i = 0; i < result.size() && i < cap; ++i) out[i] = result[i];
    return result.size();
}

int grab_index_mapped_bytes(const grab_index* h, size_t* data, size_t* graph, size_t* ts) {
    GRAB_REQUIRE(h != nullptr, "null index");
    if (data) *data = grab_vmm_size(h->d_data);
    if (graph) *graph = grab_vmm_size(h->d_graph);
    if (ts) *ts = grab_vmm_size(h->d_ts);
    return GRAB_OK;
}

int grab_index_device_ptrs(grab_index* h, const float** d_data, const uint32_t** d_graph, const uint64_t** d_ts) {
    GRAB_REQUIRE(h != nullptr, "null index");
    if (d_data) *d_data = static_cast<const float*>(grab_vmm_data(h->d_data));
    if (d_graph) *d_graph = static_cast<const uint32_t*>(grab_vmm_data(h->d_graph));
    if (d_ts) *d_ts = static_cast<const uint64_t*>(grab_vmm_data(h->d_ts));
    return GRAB_OK;
}

float grab_index_last_kernel_ms(const grab_index* h) { return h ? h->last_kernel_ms : 0.0f; }

int grab_index_last_build_seconds(const grab_index* h, double* knn, double* optimize, double* total) {
    GRAB_REQUIRE(h != nullptr, "null index");
    if (knn) *knn = h->knn_s;
    if (optimize) *optimize = h->opt_s;
    if (total) *total = h->total_s;
    return GRAB_OK;
}

// CagraIndex::save, src/cagraIndex.cu:352-369: dim u32, degree u32, size size_t, data, graph
int grab_index_save(grab_index* h, const char* path) {
    GRAB_REQUIRE(h && path, "null pointer");
    std::ofstream out(path, std::ios::binary);
    if (!out) {
        set_error("Cannot open file for save");
        return GRAB_ERR_IO;
    }
    const size_t n = h->size;
    const uint32_t* graph = n ? grab_index_get_graph(h) : nullptr;
    if (n && !graph) {
        set_error("cannot read the graph back from the device");
        return GRAB_ERR_HIP;
    }
    out.write(reinterpret_cast<const char*>(&h->dim), sizeof(h->dim));
    out.write(reinterpret_cast<const char*>(&h->degree), sizeof(h->degree));
    out.write(reinterpret_cast<const char*>(&n), sizeof(n));
    if (n > 0) {
        out.write(reinterpret_cast<const char*>(h->h_data.data()), n * h->dim * sizeof(float));
        out.write(reinterpret_cast<const char*>(graph), n * h->degree * sizeof(uint32_t));
    }
    if (!out) {
        set_error("write failed");
        return GRAB_ERR_IO;
    }
    return GRAB_OK;
}

// CagraIndex::load, src/cagraIndex.cu:371-395.  The file holds no timestamps.
int grab_index_load(grab_index* h, const char* path) {
    GRAB_REQUIRE(h && path, "null pointer");
    std::ifstream in(path, std::ios::binary);
    if (!in) {
        set_error("Cannot open file for load");
        return GRAB_ERR_IO;
    }
    uint32_t dim = 0, degree = 0;
    size_t n = 0;
    in.read(reinterpret_cast<char*>(&dim), sizeof(dim));
    in.read(reinterpret_cast<char*>(&degree), sizeof(degree));
    in.read(reinterpret_cast<char*>(&n), sizeof(n));
    if (!in || dim < 4 || dim % 4 != 0 || degree < 1 || degree > GRAB_MAX_DEGREE / 2 || n >= (1ull << 31)) {
        set_error("not an index file (dim %u, degree %u, size %zu)", dim, degree, n);
        return GRAB_ERR_IO;
    }
    std::vector<float> data(n * dim);
    std::vector<uint32_t> graph(n * degree);
    if (n > 0) {
        in.read(reinterpret_cast<char*>(data.data()), data.size() * sizeof(float));
        in.read(reinterpret_cast<char*>(graph.data()), graph.size() * sizeof(uint32_t));
        if (!in) {
            set_error("index file is truncated");
            return GRAB_ERR_IO;
        }
    }
    h->dim = dim;
    h->degree = degree;
    if (h->local_degree > degree) h->local_degree = degree;
    h->build_params.graph_degree = degree;
    h->build_params.intermediate_degree = std::max(h->build_params.intermediate_degree, degree);
    h->h_data.swap(data);
    h->h_graph.swap(graph);
    h->h_ts.clear();
    h->ts_to_ids.clear();
    h->h_labels.clear();
    h->size = n;
    h->built = n > 0;
    h->host_graph_stale = false;
    h->ts_order_stale = true;
    h->entry_rows = 0;  // the entry-point layer samples the rows present
    h->scan_rows = 0;
    h->ts_pivot_rows = 0;
    h->labels_stale = true;
    if (n > 0) {
        GRAB_TRY(grab_vmm_resize(h->d_data, n * dim * sizeof(float)));
        GRAB_TRY(grab_vmm_resize(h->d_graph, n * degree * sizeof(uint32_t)));
        GRAB_HIP(hipMemcpy(grab_vmm_data(h->d_data), h->h_data.data(), n * dim * sizeof(float), hipMemcpyHostToDevice));
        GRAB_HIP(hipMemcpy(grab_vmm_data(h->d_graph), h->h_graph.data(), n * degree * sizeof(uint32_t), hipMemcpyHostToDevice));
    }
    return GRAB_OK;
}

// CagraIndexOpt::save, src/cagraIndexOpt.cu:725-789: "MCAG", version 1, dim u32, degree u32,
// local_degree u64, size u64, timestamps (count u64 + u64 each), the timestamp -> ids map in key
// order (count u64; per key: ts u64, count u64, ids u32 each), data (count u64 + f32 each), graph
// (count u64 + u32 each).  size_t is 8 bytes on both sides.
int grab_index_save_mcag(grab_index* h, const char* path) {
    GRAB_REQUIRE(h && path, "null pointer");
    std::ofstream out(path, std::ios::binary);
    if (!out) {
        set_error("Failed to open file for writing");
        return GRAB_ERR_IO;
    }
    const uint64_t n = h->size;
    const uint32_t* graph = n ? grab_index_get_graph(h) : nullptr;
    if (n && !graph) {
        set_error("cannot read the graph back from the device");
        return GRAB_ERR_HIP;
    }
    auto put = [&](const void* p, size_t bytes) { out.write(static_cast<const char*>(p), (std::streamsize)bytes); };
    auto put64 = [&](uint64_t v) { put(&v, 8); };
    const uint32_t version = 1;
    put("MCAG", 4);
    put(&version, 4);
    put(&h->dim, 4);
    put(&h->degree, 4);
    put64(h->local_degree);
    put64(n);
    const uint64_t nts = std::min<uint64_t>(h->h_ts.size(), n);
    put64(nts);
    put(h->h_ts.data(), nts * 8);
    put64(h->ts_to_ids.size());
    for (const auto& e : h->ts_to_ids) {
        put64(e.first);
        put64(e.second.size());
        put(e.second.data(), e.second.size() * 4);
    }
    put64(n * h->dim);
    put(h->h_data.data(), n * h->dim * sizeof(float));
    put64(n * h->degree);
    if (n) put(graph, n * h->degree * sizeof(uint32_t));
    if (!out) {
        set_error("write failed");
        return GRAB_ERR_IO;
    }
    return GRAB_OK;
}

// CagraIndexOpt::load, src/cagraIndexOpt.cu:794-896
int grab_index_load_mcag(grab_index* h, const char* path) {
    GRAB_REQUIRE(h && path, "null pointer");
    std::ifstream in(path, std::ios::binary);
    if (!in) {
        set_error("Failed to open file for reading");
        return GRAB_ERR_IO;
    }
    auto get = [&](void* p, size_t bytes) { in.read(static_cast<char*>(p), (std::streamsize)bytes); };
    auto get64 = [&]() {
        uint64_t v = 0;
        get(&v, 8);
        return v;
    };
    char magic[4] = {0, 0, 0, 0};
    uint32_t version = 0, dim = 0, degree = 0;
    get(magic, 4);
    if (!in || std::memcmp(magic, "MCAG", 4) != 0) {
        set_error("Invalid file format: Magic number mismatch");
        return GRAB_ERR_IO;
    }
    get(&version, 4);
    if (!in || version != 1) {
        set_error("Unsupported version: %u", version);
        return GRAB_ERR_IO;
    }
    get(&dim, 4);
    get(&degree, 4);
    const uint64_t local_degree = get64(), n = get64();
    if (!in || dim < 4 || dim % 4 != 0 || degree < 1 || degree > GRAB_MAX_DEGREE || n >= (1ull << 31)) {
        set_error("not an index file (dim %u, degree %u, size %llu)", dim, degree, (unsigned long long)n);
        return GRAB_ERR_IO;
    }
    const uint64_t nts = get64();
    if (!in || nts > n + (1ull << 20)) {
        set_error("index file is damaged (timestamp count)");
        return GRAB_ERR_IO;
    }
    std::vector<uint64_t> ts(nts);
    get(ts.data(), nts * 8);
    std::map<uint64_t, std::vector<uint32_t>> inv;
    const uint64_t nb = get64();
    for (uint64_t b = 0; b < nb && in; ++b) {
        const uint64_t key = get64(), cnt = get64();
        if (!in || cnt > n) {
            set_error("index file is damaged (bucket size)");
            return GRAB_ERR_IO;
        }
        std::vector<uint32_t> ids(cnt);
        get(ids.data(), cnt * 4);
        inv[key] = std::move(ids);
    }
    const uint64_t nd = get64();
    if (!in || nd != n * dim) {
        set_error("index file is damaged (data size)");
        return GRAB_ERR_IO;
    }
    std::vector<float> data(nd);
    get(data.data(), nd * sizeof(float));
    const uint64_t ng = get64();
    if (!in || ng != n * degree) {
        set_error("index file is damaged (graph size)");
        return GRAB_ERR_IO;
    }
    std::vector<uint32_t> graph(ng);
    get(graph.data(), ng * sizeof(uint32_t));
    if (!in) {
        set_error("index file is truncated");
        return GRAB_ERR_IO;
    }
    h->dim = dim;
    h->degree = degree;
    h->local_degree = (uint32_t)std::min<uint64_t>(local_degree, degree);
    h->build_params.graph_degree = degree;
    h->build_params.intermediate_degree = std::max(h->build_params.intermediate_degree, degree);
    h->h_data.swap(data);
    h->h_graph.swap(graph);
    h->h_ts.swap(ts);
    h->ts_to_ids.swap(inv);
    h->h_labels.clear();
    h->size = n;
    h->built = n > 0;
    h->host_graph_stale = false;
    h->ts_order_stale = true;
    h->entry_rows = 0;
    h->scan_rows = 0;
    h->ts_pivot_rows = 0;
    h->labels_stale = true;
    if (n > 0) {
        GRAB_TRY(grab_vmm_resize(h->d_data, n * dim * sizeof(float)));
        GRAB_TRY(grab_vmm_resize(h->d_graph, n * degree * sizeof(uint32_t)));
        GRAB_HIP(hipMemcpy(grab_vmm_data(h->d_data), h->h_data.data(), n * dim * sizeof(float), hipMemcpyHostToDevice));
        GRAB_HIP(hipMemcpy(grab_vmm_data(h->d_graph), h->h_graph.data(), n * degree * sizeof(uint32_t), hipMemcpyHostToDevice));
        if (h->h_ts.size() >= n) {
            GRAB_TRY(grab_vmm_resize(h->d_ts, n * sizeof(uint64_t)));
            GRAB_HIP(hipMemcpy(grab_vmm_data(h->d_ts), h->h_ts.data(), n * sizeof(uint64_t), hipMemcpyHostToDevice));
        }
    }
    return GRAB_OK;
}

}  // extern "C"
