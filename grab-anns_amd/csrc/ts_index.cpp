// Two-level index over per-timestamp CAGRA indices: timestamp::TimeStampIndex of the reference
// (src/timeStampIndex.cuh:47-63, src/timeStampIndex.cu:36-419).  A map of timestamp -> CagraIndex
// ("bucket"), global <-> (bucket, local) id maps, and a "virtual" CagraIndex over k-means centroids
// of every bucket, each centroid carrying entry points into its bucket.  A query searches the
// virtual layer, lets the hits vote for buckets, searches the most voted buckets from the hits'
// entry points and merges.  The reference clusters with faiss::Clustering on a GPU flat index;
// FAISS is not available here, so grab_kmeans restates plain Lloyd iterations on the exact
// nearest-centroid assignment of this library.
#include <algorithm>
#include <cmath>
#include <map>
#include <memory>
#include <vector>

#include "common.hpp"
#include "topk_gemm.hpp"

using namespace grab;

extern "C" {

// Lloyd k-means.  Initial centroids: k distinct rows drawn with splitmix64(seed) (partial
// Fisher-Yates).  Every iteration assigns each row to its nearest centroid (exact squared L2, lower
// centroid id on ties; on the GPU) and moves each centroid to the mean of its rows, summed in
// double in row order on the host; a centroid without rows stays where it is.
int grab_kmeans(const float* h_data, size_t n, uint32_t dim, uint32_t k, uint32_t niter, uint64_t seed, float* h_centroids,
                int64_t* h_assign) {
    GRAB_REQUIRE(h_data && h_centroids, "null pointer");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(k >= 1 && k <= n && n < (1ull << 31), "k must be in [1, n]");
    std::vector<uint32_t> perm(n);
    for (size_t i = 0; i < n; ++i) perm[i] = (uint32_t)i;
    uint64_t state = seed;
    for (uint32_t c = 0; c < k; ++c) {
        const size_t j = c + (size_t)(splitmix64(&state) % (n - c));
        std::swap(perm[c], perm[j]);
        std::copy(h_data + (size_t)perm[c] * dim, h_data + (size_t)(perm[c] + 1) * dim, h_centroids + (size_t)c * dim);
    }
    DeviceScratch d_data, d_cent, d_ids, d_dist;
    GRAB_HIP(d_data.alloc(n * dim * sizeof(float)));
    GRAB_HIP(d_cent.alloc((size_t)k * dim * sizeof(float)));
    GRAB_HIP(d_ids.alloc(n * sizeof(int64_t)));
    GRAB_HIP(d_dist.alloc(n * sizeof(float)));
    GRAB_HIP(hipMemcpy(d_data.ptr, h_data, n * dim * sizeof(float), hipMemcpyHostToDevice));
    std::vector<int64_t> assign(n);
    std::vector<double> sums((size_t)k * dim);
    std::vector<uint32_t> counts(k);
    for (uint32_t it = 0; it <= niter; ++it) {  // the last round only assigns
        GRAB_HIP(hipMemcpy(d_cent.ptr, h_centroids, (size_t)k * dim * sizeof(float), hipMemcpyHostToDevice));
        TopkProblem p;
        p.A = d_data.as<float>();
        p.B = d_cent.as<float>();
        p.M = n;
        p.N = k;
        p.dim = dim;
        p.k = 1;
        p.metric = GRAB_METRIC_L2;
        p.out_i64 = d_ids.as<int64_t>();
        p.out_dist = d_dist.as<float>();
        GRAB_TRY(exact_topk(p, nullptr, nullptr));
        GRAB_HIP(hipMemcpy(assign.data(), d_ids.ptr, n * sizeof(int64_t), hipMemcpyDeviceToHost));
        if (it == niter) break;
        std::fill(sums.begin(), sums.end(), 0.0);
        std::fill(counts.begin(), counts.end(), 0u);
        for (size_t i = 0; i < n; ++i) {
            const size_t c = (size_t)assign[i];
            counts[c]++;
            const float* r = h_data + i * dim;
            double* s = sums.data() + c * dim;
            for (uint32_t d = 0; d < dim; ++d) s[d] += (double)r[d];
        }
        for (uint32_t c = 0; c < k; ++c) {
            if (counts[c] == 0) continue;
            for (uint32_t d = 0; d < dim; ++d) h_centroids[(size_t)c * dim + d] = (float)(sums[(size_t)c * dim + d] / (double)counts[c]);
        }
    }
    if (h_assign) std::copy(assign.begin(), assign.end(), h_assign);
    return GRAB_OK;
}

}  // extern "C"

struct grab_tsindex {
    uint32_t dim = 0, degree = 0;
    size_t cluster_ratio = 0, vmm_max_bytes = 0;
    uint64_t global_count = 0, seed = 0x9E3779B97F4A7C15ull;
    struct Bucket {
        grab_index* index = nullptr;
        std::vector<uint64_t> local_to_global;
        size_t num_dirty = 0;
    };
    std::map<uint64_t, Bucket> buckets;
    struct Location {
        uint64_t ts;
        size_t local;
    };
    std::vector<Location> id_to_location;
    grab_index* virtual_index = nullptr;
    struct VirtualPoint {
        uint64_t target_ts;
        std::vector<uint32_t> entry_points;
    };
    std::vector<VirtualPoint> virtual_meta;
};

extern "C" {

int grab_tsindex_create(uint32_t dim, uint32_t graph_degree, size_t cluster_ratio, size_t vmm_max_bytes_per_bucket,
                        grab_tsindex** out) {
    GRAB_REQUIRE(out != nullptr, "null pointer");
    GRAB_REQUIRE(dim >= 4 && dim % 4 == 0, "unsupported dimension %u (must be a multiple of 4)", dim);
    GRAB_REQUIRE(graph_degree >= 1 && graph_degree <= GRAB_MAX_DEGREE / 2, "graph_degree %u out of range", graph_degree);
    auto* t = new grab_tsindex();
    t->dim = dim;
    t->degree = graph_degree;
    t->cluster_ratio = cluster_ratio;
    t->vmm_max_bytes = vmm_max_bytes_per_bucket ? vmm_max_bytes_per_bucket : (size_t)20 << 30;
    *out = t;
    return GRAB_OK;
}

void grab_tsindex_destroy(grab_tsindex* t) {
    if (!t) return;
    for (auto& kv : t->buckets) grab_index_destroy(kv.second.index);
    grab_index_destroy(t->virtual_index);
    delete t;
}

size_t grab_tsindex_size(const grab_tsindex* t) { return t ? (size_t)t->global_count : 0; }
size_t grab_tsindex_num_buckets(const grab_tsindex* t) { return t ? t->buckets.size() : 0; }
size_t grab_tsindex_num_virtual_points(const grab_tsindex* t) { return t ? t->virtual_meta.size() : 0; }

int grab_tsindex_set_seed(grab_tsindex* t, uint64_t seed) {
    GRAB_REQUIRE(t != nullptr, "null index");
    t->seed = seed;
    return GRAB_OK;
}

// TimeStampIndex::insert, src/timeStampIndex.cu:65-139: rows are grouped by timestamp, every group goes
// into its bucket's CagraIndex::insert, global ids are assigned in arrival order
int grab_tsindex_insert(grab_tsindex* t, const float* vectors, const uint64_t* timestamps, size_t n, uint64_t* out_start_id) {
    GRAB_REQUIRE(t && (n == 0 || (vectors && timestamps)), "null pointer");
    const uint64_t start = t->global_count;
    if (out_start_id) *out_start_id = start;
    if (n == 0) return GRAB_OK;
    struct Group {
        std::vector<float> vecs;
        std::vector<uint64_t> gids;
    };
    std::map<uint64_t, Group> groups;
    for (size_t i = 0; i < n; ++i) {
        Group& g = groups[timestamps[i]];
        g.vecs.insert(g.vecs.end(), vectors + i * t->dim, vectors + (i + 1) * t->dim);
        g.gids.push_back(start + i);
    }
    t->id_to_location.resize(start + n);
    for (auto& kv : groups) {
        grab_tsindex::Bucket& b = t->buckets[kv.first];
        if (b.index == nullptr) {
            GRAB_TRY(grab_index_create(t->dim, t->degree, 0, t->vmm_max_bytes, &b.index));
            GRAB_TRY(grab_index_set_seed(b.index, t->seed ^ kv.first));
        }
        const size_t first_local = grab_index_size(b.index), count = kv.second.gids.size();
        GRAB_TRY(grab_index_insert(b.index, count, kv.second.vecs.data(), nullptr));
        for (size_t j = 0; j < count; ++j) {
            t->id_to_location[kv.second.gids[j]] = {kv.first, first_local + j};
            b.local_to_global.push_back(kv.second.gids[j]);
        }
        b.num_dirty += count;
    }
    t->global_count = start + n;
    return GRAB_OK;
}

// TimeStampIndex::build_virtual_index, src/timeStampIndex.cu:141-238: per bucket 16*sqrt(n) centroids
// (30 Lloyd iterations), 5 entry points per centroid found by searching the bucket with the centroid,
// then one CagraIndex over all centroids
int grab_tsindex_build_virtual_index(grab_tsindex* t) {
    GRAB_REQUIRE(t != nullptr, "null index");
    if (t->buckets.empty()) return GRAB_OK;
    std::vector<float> all_centroids;
    std::vector<grab_tsindex::VirtualPoint> meta;
    const int entries_per_centroid = 5;
    for (auto& kv : t->buckets) {
        grab_index* b = kv.second.index;
        const size_t n = grab_index_size(b);
        if (n == 0) continue;
        const float* h_data = grab_index_get_data(b);
        uint32_t k = 16u * (uint32_t)std::max(1, (int)std::sqrt((double)n));
        k = (uint32_t)std::min<size_t>(k, n);  // the reference lets FAISS reject k > n
        std::vector<float> cent((size_t)k * t->dim);
        GRAB_TRY(grab_kmeans(h_data, n, t->dim, k, 30, t->seed ^ (kv.first * 0x100000001B3ull), cent.data(), nullptr));
        const int want = (int)std::min<size_t>(entries_per_centroid, n);
        std::vector<int64_t> idx((size_t)k * want);
        std::vector<float> dist((size_t)k * want);
        GRAB_TRY(grab_index_search(b, cent.data(), k, want, idx.data(), dist.data(), nullptr, 0));
        for (uint32_t c = 0; c < k; ++c) {
            all_centroids.insert(all_centroids.end(), cent.begin() + (size_t)c * t->dim, cent.begin() + (size_t)(c + 1) * t->dim);
            grab_tsindex::VirtualPoint vp;
            vp.target_ts = kv.first;
            for (int e = 0; e < want; ++e) {
                const int64_t id = idx[(size_t)c * want + e];
                if (id >= 0 && (size_t)id < n) vp.entry_points.push_back((uint32_t)id);
            }
            meta.push_back(std::move(vp));
        }
        kv.second.num_dirty = 0;
    }
    grab_index_destroy(t->virtual_index);
    t->virtual_index = nullptr;
    t->virtual_meta.clear();
    if (all_centroids.empty()) return GRAB_OK;
    GRAB_TRY(grab_index_create(t->dim, t->degree, 0, t->vmm_max_bytes, &t->virtual_index));
    GRAB_TRY(grab_index_set_seed(t->virtual_index, t->seed));
    GRAB_TRY(grab_index_add(t->virtual_index, all_centroids.size() / t->dim, all_centroids.data(), nullptr));
    GRAB_TRY(grab_index_build(t->virtual_index));
    t->virtual_meta = std::move(meta);
    return GRAB_OK;
}

// TimeStampIndex::query, src/timeStampIndex.cu:240-419: one query; -1 / -1.0f for slots without a result
int grab_tsindex_query(grab_tsindex* t, const float* query, size_t topk, int64_t* out_indices, float* out_dists,
                       int probe_buckets) {
    GRAB_REQUIRE(t && query && out_indices && out_dists, "null pointer");
    GRAB_REQUIRE(topk >= 1 && probe_buckets >= 1, "topk and probe_buckets must be positive");
    auto fill_empty = [&]() {
        for (size_t i = 0; i < topk; ++i) {
            out_indices[i] = -1;
            out_dists[i] = -1.0f;
        }
    };
    if (t->virtual_index == nullptr || t->buckets.empty()) {
        fill_empty();
        return GRAB_OK;
    }
    // level 1: ten virtual points per bucket to probe vote for their buckets (:262-293)
    size_t vk = (size_t)probe_buckets * 10;
    vk = std::min(vk, t->virtual_meta.size());
    std::vector<int64_t> v_idx(vk);
    std::vector<float> v_dist(vk);
    GRAB_TRY(grab_index_search(t->virtual_index, query, 1, (int)vk, v_idx.data(), v_dist.data(), nullptr, 0));
    struct Votes {
        int count = 0;
        size_t first_rank = 0;
        std::vector<uint32_t> seeds;
    };
    std::map<uint64_t, Votes> votes;
    for (size_t i = 0; i < vk; ++i) {
        const int64_t v = v_idx[i];
        if (v < 0 || (size_t)v >= t->virtual_meta.size()) continue;
        const auto& m = t->virtual_meta[(size_t)v];
        Votes& c = votes[m.target_ts];
        if (c.count == 0) c.first_rank = i;
        c.count++;
        c.seeds.insert(c.seeds.end(), m.entry_points.begin(), m.entry_points.end());
    }
    // most votes first; the reference leaves equal counts to std::sort, here the bucket whose first
    // vote came from the nearer virtual point goes first
    std::vector<std::pair<uint64_t, const Votes*>> ranked;
    for (auto& kv : votes) ranked.push_back({kv.first, &kv.second});
    std::sort(ranked.begin(), ranked.end(), [](const auto& a, const auto& b) {
        return a.second->count != b.second->count ? a.second->count > b.second->count : a.second->first_rank < b.second->first_rank;
    });
    const size_t nb = std::min((size_t)probe_buckets, ranked.size());
    // level 2: the chosen buckets, seeded with the entry points of the virtual points that voted (:330-390)
    std::vector<std::pair<float, int64_t>> all;
    std::vector<int64_t> b_idx(topk);
    std::vector<float> b_dist(topk);
    for (size_t i = 0; i < nb; ++i) {
        auto it = t->buckets.find(ranked[i].first);
        if (it == t->buckets.end()) continue;
        const grab_tsindex::Bucket& b = it->second;
        const std::vector<uint32_t>& seeds = ranked[i].second->seeds;
        const int k = (int)std::min(topk, grab_index_size(b.index));
        if (k == 0) continue;
        GRAB_TRY(grab_index_search(b.index, query, 1, k, b_idx.data(), b_dist.data(), seeds.empty() ? nullptr : seeds.data(),
                                   seeds.size()));
        for (int r = 0; r < k; ++r) {
            const int64_t lid = b_idx[r];
            if (lid >= 0 && (size_t)lid < b.local_to_global.size()) all.push_back({b_dist[r], (int64_t)b.local_to_global[(size_t)lid]});
        }
    }
    std::sort(all.begin(), all.end());  // by (distance, global id); the reference compares distances only
    for (size_t r = 0; r < topk; ++r) {
        out_indices[r] = r < all.size() ? all[r].second : -1;
        out_dists[r] = r < all.size() ? all[r].first : -1.0f;
    }
    return GRAB_OK;
}

// read-only views of the two levels, for callers that want to inspect or re-derive a query's routing: the
// handles stay owned by the index and are valid until the next insert / build_virtual_index / destroy
grab_index* grab_tsindex_virtual_index(grab_tsindex* t) { return t ? t->virtual_index : nullptr; }

grab_index* grab_tsindex_bucket_index(grab_tsindex* t, uint64_t ts) {
    if (!t) return nullptr;
    auto it = t->buckets.find(ts);
    return it == t->buckets.end() ? nullptr : it->second.index;
}

size_t grab_tsindex_bucket_timestamps(const grab_tsindex* t, uint64_t* out, size_t cap) {
    if (!t) return 0;
    size_t i = 0;
    for (auto& kv : t->buckets) {
        if (out && i < cap) out[i] = kv.first;
        ++i;
    }
    return i;
}

int grab_tsindex_virtual_point(const grab_tsindex* t, size_t i, uint64_t* out_ts, uint32_t* out_entry_points, size_t cap,
                               size_t* out_count) {
    GRAB_REQUIRE(t != nullptr, "null index");
    GRAB_REQUIRE(i < t->virtual_meta.size(), "virtual point out of range");
    const auto& m = t->virtual_meta[i];
    if (out_ts) *out_ts = m.target_ts;
    if (out_count) *out_count = m.entry_points.size();
    if (out_entry_points)
        for (size_t e = 0; e < m.entry_points.size() && e < cap; ++e) out_entry_points[e] = m.entry_points[e];
    return GRAB_OK;
}

// global id -> (timestamp, id inside the bucket)
int grab_tsindex_locate(const grab_tsindex* t, uint64_t global_id, uint64_t* out_ts, size_t* out_local) {
    GRAB_REQUIRE(t != nullptr, "null index");
    GRAB_REQUIRE(global_id < t->global_count, "global id out of range");
    if (out_ts) *out_ts = t->id_to_location[global_id].ts;
    if (out_local) *out_local = t->id_to_location[global_id].local;
    return GRAB_OK;
}

}  // extern "C"
