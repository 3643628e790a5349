// Host side of the search entry points: the reference wrappers' clamping rules, argument
// checks that keep a bad call from reaching the GPU, and the kernel launch.
#include <algorithm>
#include <cstring>

#include "entry_layer.hpp"
#include "search_internal.hpp"

static_assert(grab::kStaticTableSlots == GRAB_STATIC_TABLE_SLOTS, "header and library disagree on the static array");

namespace grab {

namespace {
thread_local std::string g_error;
thread_local ScratchArena* g_scratch_arena = nullptr;
}

ScratchArena*& scratch_arena() { return g_scratch_arena; }

void set_error(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
}
const char* get_error() { return g_error.c_str(); }

}  // namespace grab

using namespace grab;

namespace grab {

// sync == false leaves the kernel running on the stream (used by the insert path, which
// chains further kernels behind it); a per-call visited-set allocation forces a sync.
int search_ex_impl(const grab_search_desc* d, bool sync, bool static_tables) {
    GRAB_REQUIRE(d != nullptr, "null descriptor");
    // the reference throws "Graph is null!" (src/index/cagra.cu:858-860)
    GRAB_REQUIRE(d->d_graph != nullptr, "Graph is null!");
    GRAB_REQUIRE(d->d_dataset && d->d_queries && d->d_out_indices && d->d_out_dists, "null data/query/output pointer");
    GRAB_REQUIRE(d->num_dataset > 0 && d->num_dataset < (1ull << 31), "num_dataset must be in [1, 2^31)");
    GRAB_REQUIRE(d->dim >= 4 && d->dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", d->dim);
    GRAB_REQUIRE(d->graph_degree >= 1 && d->graph_degree <= GRAB_MAX_DEGREE, "graph_degree %u out of range", d->graph_degree);
    GRAB_REQUIRE(d->active_degree <= d->graph_degree, "active_degree exceeds graph_degree");
    GRAB_REQUIRE(d->k >= 1 && d->k <= d->itopk, "k must be in [1, itopk]");
    GRAB_REQUIRE(d->itopk <= 4096, "itopk %u too large (max 4096)", d->itopk);
    GRAB_REQUIRE(d->search_width >= 1 && d->search_width <= 1024 &&
                     (uint64_t)d->search_width * d->graph_degree <= 8192, "search_width*degree too large");
    GRAB_REQUIRE(d->n_seeds <= d->itopk, "n_seeds exceeds itopk");
    GRAB_REQUIRE(d->hash_bitlen >= 4 && d->hash_bitlen <= 24, "hash_bitlen %u out of range [4,24]", d->hash_bitlen);
    GRAB_REQUIRE(d->metric == GRAB_METRIC_L2 || d->metric == GRAB_METRIC_IP, "bad metric");
    GRAB_REQUIRE(d->num_queries < (1ull << 31), "too many queries");
    if (d->filter_kind == 1) {
        GRAB_REQUIRE(d->d_ts != nullptr, "range filter needs timestamps");
        GRAB_REQUIRE(!d->per_query_window || (d->d_win_start && d->d_win_end), "per-query windows missing");
    } else if (d->filter_kind == 2) {
        GRAB_REQUIRE(d->d_labels && d->d_masks, "mask filter needs labels and masks");
    } else if (d->filter_kind == 3) {
        GRAB_REQUIRE(!d->per_query_window || (d->d_win_start && d->d_win_end), "per-query id ranges missing");
    } else {
        GRAB_REQUIRE(d->filter_kind == 0, "bad filter kind");
    }
    GRAB_REQUIRE(d->n_provided == 0 || d->d_seeds != nullptr, "n_provided > 0 with null seeds");
    const grab_entry_layer* el = d->entry_layer;
    if (el != nullptr) {
        GRAB_REQUIRE(el->num_groups > 0, "entry_layer: the layer has no groups (grab_entry_layer_build_groups)");
        GRAB_REQUIRE(el->base_in_ts_order, "entry_layer: the layer was not made over a base whose timestamps ascend with the row id");
        GRAB_REQUIRE(d->filter_kind == 3 && d->d_ts != nullptr, "entry_layer: needs filter_kind 3 and the base's timestamps in d_ts");
        GRAB_REQUIRE(d->d_entry_groups != nullptr && d->entry_nprobe >= 1 && d->entry_nprobe <= 64,
                     "entry_layer: d_entry_groups missing or entry_nprobe outside [1,64]");
        GRAB_REQUIRE(d->n_seeds >= 1 && d->n_seeds <= 64, "entry_layer: n_seeds must be in [1,64]");
        GRAB_REQUIRE(el->dim == d->dim && el->num_base <= d->num_dataset, "entry_layer: made over another base");
        GRAB_REQUIRE(d->d_rank == nullptr, "entry_layer: the layer's intervals are row ids, d_rank must be NULL");
    }
    if (d->num_queries == 0) return GRAB_OK;

    hipStream_t stream = static_cast<hipStream_t>(d->stream);
    SearchArgs a{};
    a.data = d->d_dataset;
    a.graph = d->d_graph;
    a.queries = d->d_queries;
    a.seeds = d->n_provided ? d->d_seeds : nullptr;
    a.ts = d->d_ts;
    a.graph_ts = d->filter_kind == dev::kFilterRange ? d->d_graph_ts : nullptr;
    a.rank_of_id = d->filter_kind == dev::kFilterIdRange ? d->d_rank : nullptr;
    a.graph_rank = a.rank_of_id != nullptr ? d->d_graph_rank : nullptr;
    a.win_start_arr = d->d_win_start;
    a.win_end_arr = d->d_win_end;
    a.labels = d->d_labels;
    a.masks = d->d_masks;
    a.out_ids = d->d_out_indices;
    a.out_dists = d->d_out_dists;
    a.counters = d->d_counters;
    a.n = d->num_dataset;
    a.rand_xor_mask = d->rand_xor_mask;
    a.win_start = d->win_start;
    a.win_end = d->win_end;
    a.dim = d->dim;
    a.degree = d->graph_degree;
    a.active_degree = d->active_degree;
    a.nq = (uint32_t)d->num_queries;
    a.k = d->k;
    a.itopk = d->itopk;
    a.search_width = d->search_width;
    a.max_iterations = d->max_iterations;
    a.hash_bitlen = d->hash_bitlen;
    a.n_seeds = d->n_seeds;
    a.n_provided = d->n_provided;
    a.flags = d->flags;
    a.cmax = std::max(d->search_width * d->graph_degree, std::max(d->n_seeds, 1u));
    a.per_query_window = d->per_query_window;

    // one wave per query when that fills the device (many queries, a few KB of LDS each),
    // else one workgroup per query
    // Its survivor/candidate lists may be shorter than one iteration's worth of neighbours (the
    // kernel scores and merges early when they fill up): an eighth of the visited set's slots, at
    // least 128 (two full visits of 64 ids, so that the few survivors of a selective filter never
    // force an early merge), so that a small table is not dwarfed by lists that are never filled.
    uint32_t wave_cmax = a.cmax, wave_ccap = a.cmax;
    if (!(d->flags & GRAB_FLAG_STRICT_REFERENCE)) {
        wave_cmax = std::min(a.cmax, std::max(128u, (1u << a.hash_bitlen) / 8u));
        wave_ccap = std::min(wave_cmax, std::max(64u, wave_cmax / 2));  // only keys that beat the worst entry are listed
    }
    const bool wave_single = a.itopk <= 64 && wave_ccap <= 128;  // one queue buffer, merged in place
    // queue in registers: no queue, candidate or parent list in LDS
    const bool wave_reg = a.itopk <= 256 && a.search_width <= 64 && !(d->flags & GRAB_FLAG_STRICT_REFERENCE);
    // the usual shape gets a kernel instance with that shape compiled in; its survivor list holds a whole iteration
    const bool wave_fixed = wave_reg && a.itopk <= 64 && a.degree == 64 && a.active_degree == 64 && a.search_width <= 4 &&
                            a.n_seeds <= 64 && d->filter_kind != 0 && (d->flags & GRAB_FLAG_FILTER_FIRST);
    if (wave_fixed) wave_cmax = 256;
    const SearchWaveLdsLayout wlay =
        wave_reg ? search_wave_lds_layout(0, a.dim == 128 ? 0 : a.dim, wave_cmax, 0, true, 0, a.hash_bitlen)
                 : search_wave_lds_layout(a.itopk, a.dim == 128 ? 0 : a.dim, wave_cmax, wave_ccap, wave_single, a.search_width,
                                          a.hash_bitlen);
    GRAB_REQUIRE(!((d->flags & GRAB_FLAG_WAVE_PER_QUERY) && (d->flags & GRAB_FLAG_BLOCK_PER_QUERY)),
                 "GRAB_FLAG_WAVE_PER_QUERY and GRAB_FLAG_BLOCK_PER_QUERY exclude each other");
    // A wave per query pays while enough waves fit a CU to hide the latency of the row reads: with 20 KB of LDS a
    // wave, eight do.  Beyond that (a visited set of 8192 slots or more) the workgroup per query, whose waves share
    // one table, is the faster one - by a few percent at 128 dimensions, two to three times at 256 to 768.
    bool use_wave = a.hash_bitlen <= 15 && wlay.total <= 20 * 1024 && a.nq >= 1024;
    if (d->flags & GRAB_FLAG_BLOCK_PER_QUERY) use_wave = false;
    if (d->flags & GRAB_FLAG_WAVE_PER_QUERY) {
        GRAB_REQUIRE(a.hash_bitlen < 20 && wlay.total <= kMaxLdsBytes, "wave-per-query search: queue and visited set (%u bytes) do not fit LDS", wlay.total);
        use_wave = true;
    }

    // visited set: LDS when it fits next to the queue, otherwise one table per query in
    // device memory (the reference switches at hash_bitlen >= 14, src/index/search.cu:188-194)
    DeviceScratch ghash;
    // A small batch splits its merges over the waves when the partial counts fit LDS beside everything else; they
    // never push the visited set to device memory or the queue out of LDS - such shapes take the plain merge.
    const bool small = a.nq <= kSmallBatchQueries;
    SearchLdsLayout lay = search_lds_layout(a.itopk, a.dim, a.cmax, a.search_width, a.hash_bitlen, true, small);
    a.split_merge = small ? 1 : 0;
    if (small && (a.hash_bitlen >= 20 || lay.total > kMaxLdsBytes)) {
        const SearchLdsLayout plain = search_lds_layout(a.itopk, a.dim, a.cmax, a.search_width, a.hash_bitlen, true, false);
        const bool table_fits_without = a.hash_bitlen < 20 && plain.total <= kMaxLdsBytes;
        const bool queue_fits_with = search_lds_layout(a.itopk, a.dim, a.cmax, a.search_width, 0, false, true).total <= kMaxLdsBytes;
        if (table_fits_without || !queue_fits_with) {
            a.split_merge = 0;
            lay = plain;
        }
    }
    if (use_wave) {
        lay.total = wlay.total;
        a.cmax = wave_cmax;
        a.ccap = wave_ccap;
        a.single_queue = wave_single ? 1 : 0;
        a.reg_queue = wave_reg ? 1 : 0;
        a.fixed_shape = wave_fixed ? 1 : 0;
    } else if (a.hash_bitlen >= 20 || lay.total > kMaxLdsBytes) {
        lay = search_lds_layout(a.itopk, a.dim, a.cmax, a.search_width, 0, false, a.split_merge != 0);
        GRAB_REQUIRE(lay.total <= kMaxLdsBytes, "queue does not fit LDS (itopk %u)", a.itopk);
        const size_t slots = (size_t)a.nq << a.hash_bitlen;
        if (static_tables) {
            GRAB_REQUIRE(slots <= kStaticTableSlots,
                         "grab_search_ex_static: %u queries x 2^%u visited-set slots exceed the %zu slots (%zu MiB) of the "
                         "static array; use fewer queries per call, a smaller hash_bitlen, or grab_search_ex",
                         a.nq, a.hash_bitlen, kStaticTableSlots, kStaticTableSlots * sizeof(uint32_t) >> 20);
            GRAB_TRY(static_visited_sets(&a.global_hash));
        } else {
            GRAB_HIP(ghash.alloc(slots * sizeof(uint32_t)));
            a.global_hash = ghash.as<uint32_t>();
        }
    }

    if (el != nullptr) {
        GRAB_REQUIRE(use_wave && wave_reg, "entry_layer: only the wave-per-query kernel with the queue in registers lists its own "
                                          "seeds (itopk <= 256, search_width <= 64, no strict flag, a visited set that fits LDS, "
                                          "1024 queries or more unless GRAB_FLAG_WAVE_PER_QUERY is set)");
        a.entry.groups = d->d_entry_groups;
        a.entry.tbl = el->group_tbl_id.as<uint32_t>();
        a.entry.ids = el->group_ids.as<uint32_t>();
        a.entry.piv = el->pivots.as<uint64_t>();
        for (uint32_t i = 0; i < 6; ++i) {
            a.entry.piv_off[i] = el->piv_off[i];
            a.entry.piv_cnt[i] = el->piv_cnt[i];
        }
        a.entry.nlev = el->piv_levels;
        a.entry.nprobe = d->entry_nprobe;
        a.entry.min_rows = d->entry_min_rows;
        a.entry.n_base = (uint32_t)el->num_base;
        a.entry.stretch = (uint32_t)((el->num_base + kIdStretches - 1) / kIdStretches);
    }

    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (d->kernel_ms) {
        GRAB_REQUIRE(!static_tables, "grab_search_ex_static: kernel_ms must be NULL (timing creates events)");
        hipError_t e = hipEventCreate(&e0);
        if (e == hipSuccess) e = hipEventCreate(&e1);
        if (e == hipSuccess) e = hipEventRecord(e0, stream);
        if (e != hipSuccess) {
            if (e0) (void)hipEventDestroy(e0);
            if (e1) (void)hipEventDestroy(e1);
            set_error("HIP error %s while setting up the timing of the search kernel", hipGetErrorString(e));
            return GRAB_ERR_HIP;
        }
    }
    // an id interval that comes with a table of places is tested on the places
    const int filter = (d->filter_kind == dev::kFilterIdRange && a.rank_of_id != nullptr) ? dev::kFilterRank : d->filter_kind;
    int rc = use_wave ? launch_search_wave(a, d->metric, filter, lay.total, stream)
                      : launch_search(a, d->metric, filter, lay.total, stream);
    if (d->kernel_ms && rc == GRAB_OK) {
        hipError_t e = hipEventRecord(e1, stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        if (e == hipSuccess) e = hipEventElapsedTime(d->kernel_ms, e0, e1);
        if (e != hipSuccess) {
            set_error("HIP error %s while timing the search kernel", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    // a table from hipMalloc is freed on return, so the kernel must have finished - also when the launch
    // reported an error after queueing work
    if (!static_tables && (sync || ghash.ptr != nullptr)) {
        hipError_t e = hipStreamSynchronize(stream);
        if (rc == GRAB_OK && e != hipSuccess) {
            set_error("HIP error %s while waiting for the search kernel", hipGetErrorString(e));
            rc = GRAB_ERR_HIP;
        }
    }
    return rc;
}

void fill_search_desc(grab_search_desc* d, int wrapper, const float* d_dataset, size_t n, uint32_t dim,
                      const uint32_t* d_graph, uint32_t degree, uint32_t active_degree, const float* d_queries,
                      size_t nq, uint32_t k, grab_search_params p, int metric, const uint32_t* d_seeds,
                      uint32_t n_provided, uint64_t mask, uint32_t flags, int64_t* d_out_indices,
                      float* d_out_dists, void* stream) {
    std::memset(d, 0, sizeof(*d));
    d->d_dataset = d_dataset;
    d->d_graph = d_graph;
    d->num_dataset = n;
    d->dim = dim;
    d->graph_degree = degree;
    d->active_degree = active_degree;
    d->metric = metric;
    d->d_queries = d_queries;
    d->num_queries = nq;
    d->k = k;
    uint32_t cap;
    grab_search_plan(wrapper, k, p.itopk_size, p.search_width, degree, d_seeds ? n_provided : 0, &d->itopk,
                     &d->n_seeds, &cap);
    d->search_width = p.search_width;
    d->max_iterations = p.max_iterations;
    d->hash_bitlen = p.hash_bitlen;
    d->d_seeds = d_seeds;
    d->n_provided = d_seeds ? n_provided : 0;
    d->rand_xor_mask = mask;
    d->flags = flags;
    d->d_out_indices = d_out_indices;
    d->d_out_dists = d_out_dists;
    d->stream = stream;
}

}  // namespace grab

extern "C" {

const char* grab_last_error(void) { return grab::get_error(); }

int grab_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

uint32_t grab_next_power_of_2(uint32_t n) {
    if (n == 0) return 1;
    n--;
    n |= n >> 1;
    n |= n >> 2;
    n |= n >> 4;
    n |= n >> 8;
    n |= n >> 16;
    return n + 1;
}

uint32_t grab_queue_capacity(uint32_t itopk, uint32_t search_width, uint32_t degree) {
    return std::max(256u, grab_next_power_of_2(itopk + search_width * degree));
}

size_t grab_reference_smem_bytes(uint32_t itopk, uint32_t dim, uint32_t search_width, uint32_t degree,
                                 uint32_t hash_bitlen) {
    auto up16 = [](size_t x) { return (x + 15) & ~(size_t)15; };
    size_t smem = up16((size_t)dim * 4);
    smem += up16(((size_t)1 << hash_bitlen) * 4);
    smem += up16((size_t)grab_queue_capacity(itopk, search_width, degree) * 8);
    smem += up16((size_t)search_width * 4);
    smem += 256;
    if (hash_bitlen >= 14) smem -= ((size_t)1 << hash_bitlen) * 4;
    return smem;
}

size_t grab_search_lds_bytes(uint32_t itopk, uint32_t dim, uint32_t search_width, uint32_t degree,
                             uint32_t n_seeds, uint32_t hash_bitlen) {
    const uint32_t cmax = std::max(search_width * degree, std::max(n_seeds, 1u));
    SearchLdsLayout with_hash = search_lds_layout(itopk, dim, cmax, search_width, hash_bitlen, true, false);
    if (hash_bitlen < 20 && with_hash.total <= kMaxLdsBytes) return with_hash.total;
    return search_lds_layout(itopk, dim, cmax, search_width, 0, false, false).total;
}

void grab_search_plan(int wrapper, uint32_t k, uint32_t itopk_param, uint32_t search_width,
                      uint32_t degree, uint32_t n_provided, uint32_t* itopk_eff, uint32_t* n_seeds,
                      uint32_t* queue_capacity) {
    uint32_t itopk = std::max(k, itopk_param);
    const uint32_t floor_itopk = wrapper == GRAB_WRAP_BUCKET ? 128u : 64u;
    if (itopk < floor_itopk) itopk = floor_itopk;
    uint32_t seeds;
    switch (wrapper) {
        case GRAB_WRAP_SEARCH: seeds = itopk_param / 4; break;
        case GRAB_WRAP_SEARCH_OPT: seeds = std::min(std::max(32u, n_provided), itopk); break;
        default: seeds = std::min(n_provided, itopk); break;
    }
    if (itopk_eff) *itopk_eff = itopk;
    if (n_seeds) *n_seeds = seeds;
    if (queue_capacity) *queue_capacity = grab_queue_capacity(itopk, search_width, degree);
}

int grab_search_ex(const grab_search_desc* d) { return grab::search_ex_impl(d, true); }
int grab_search_ex_async(const grab_search_desc* d) { return grab::search_ex_impl(d, false); }
int grab_search_ex_static(const grab_search_desc* d) { return grab::search_ex_impl(d, false, true); }

static int search_wrapped(int wrapper, const float* d_dataset, size_t n, uint32_t dim, const uint32_t* d_graph,
                          uint32_t degree, uint32_t active_degree, const float* d_queries, int64_t nq,
                          int64_t k, grab_search_params p, int filter_kind, const uint64_t* d_ts,
                          uint64_t ws, uint64_t we, int64_t* d_out_indices, float* d_out_dists,
                          const uint32_t* d_seeds, uint32_t n_provided, uint64_t mask, uint32_t flags,
                          void* stream) {
    GRAB_REQUIRE(nq >= 0 && k >= 1, "bad num_queries / k");
    grab_search_desc d;
    fill_search_desc(&d, wrapper, d_dataset, n, dim, d_graph, degree, active_degree, d_queries, (size_t)nq,
                     (uint32_t)k, p, GRAB_METRIC_L2, d_seeds, n_provided, mask, flags, d_out_indices, d_out_dists,
                     stream);
    d.filter_kind = filter_kind;
    d.d_ts = d_ts;
    d.win_start = ws;
    d.win_end = we;
    return grab_search_ex(&d);
}

int grab_search(const float* d_dataset, size_t num_dataset, uint32_t dim, const uint32_t* d_graph,
                uint32_t graph_degree, const float* d_queries, int64_t num_queries, int64_t k,
                grab_search_params params, int64_t* d_out_indices, float* d_out_dists,
                const uint32_t* d_seeds, uint32_t num_seeds_per_query, uint64_t rand_xor_mask,
                uint32_t flags, void* stream) {
    return search_wrapped(GRAB_WRAP_SEARCH, d_dataset, num_dataset, dim, d_graph, graph_degree, graph_degree,
                          d_queries, num_queries, k, params, 0, nullptr, 0, 0, d_out_indices, d_out_dists,
                          d_seeds, num_seeds_per_query, rand_xor_mask, flags, stream);
}

int grab_search_opt(const float* d_dataset, uint32_t dim, size_t num_dataset, const uint32_t* d_graph,
                    uint32_t graph_degree, const float* d_queries, int64_t num_queries, int64_t k,
                    grab_search_params params, int64_t* d_out_indices, float* d_out_dists,
                    const uint32_t* d_seeds, uint32_t num_seeds_per_query, uint64_t rand_xor_mask,
                    uint32_t flags, void* stream) {
    return search_wrapped(GRAB_WRAP_SEARCH_OPT, d_dataset, num_dataset, dim, d_graph, graph_degree,
                          graph_degree, d_queries, num_queries, k, params, 0, nullptr, 0, 0, d_out_indices,
                          d_out_dists, d_seeds, num_seeds_per_query, rand_xor_mask, flags, stream);
}

int grab_search_bucket(const float* d_dataset, uint32_t dim, size_t num_dataset, const uint32_t* d_graph,
                       uint32_t total_degree, uint32_t local_degree, const float* d_queries,
                       int64_t num_queries, int64_t k, grab_search_params params, int64_t* d_out_indices,
                       float* d_out_dists, const uint32_t* d_seeds, uint32_t num_seeds_per_query,
                       uint64_t rand_xor_mask, uint32_t flags, void* stream) {
    return search_wrapped(GRAB_WRAP_BUCKET, d_dataset, num_dataset, dim, d_graph, total_degree, local_degree,
                          d_queries, num_queries, k, params, 0, nullptr, 0, 0, d_out_indices, d_out_dists,
                          d_seeds, num_seeds_per_query, rand_xor_mask, flags, stream);
}

int grab_search_range(const float* d_dataset, uint32_t dim, size_t num_dataset, const uint32_t* d_graph,
                      const uint64_t* d_ts, uint32_t total_degree, uint32_t local_degree,
                      const float* d_queries, int64_t num_queries, int64_t k, uint64_t start_bucket,
                      uint64_t end_bucket, grab_search_params params, int64_t* d_out_indices,
                      float* d_out_dists, const uint32_t* d_seeds, uint32_t num_seeds_per_query,
                      uint64_t rand_xor_mask, uint32_t flags, void* stream) {
    // the range kernel of the reference is called with graph_stride for both widths
    // (src/index/search.cu:759-761), so local_degree has no effect there either
    (void)local_degree;
    return search_wrapped(GRAB_WRAP_RANGE, d_dataset, num_dataset, dim, d_graph, total_degree, total_degree,
                          d_queries, num_queries, k, params, 1, d_ts, start_bucket, end_bucket,
                          d_out_indices, d_out_dists, d_seeds, num_seeds_per_query, rand_xor_mask, flags,
                          stream);
}

}  // extern "C"
