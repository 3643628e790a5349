// CPU baseline: a plain HNSW index (Malkov & Yashunin, "Efficient and robust approximate nearest
// neighbor search using Hierarchical Navigable Small World graphs", Algorithms 1-5) with the
// parameters the benchmark configurations name for FAISS IndexHNSWFlat (M = 32, efConstruction =
// 200, efSearch = 128).  FAISS is not installed here, so the published algorithm is restated.
// BENCHMARK / TEST INFRASTRUCTURE ONLY: timed beside the GPU path by bench.py, never part of it.
//
// Filtered queries post-filter, the way an index without filter support is used: search with a
// growing ef until k results pass the filter or the whole index was asked for.
// Build: g++ -O3 -mavx2 -mfma -fopenmp -shared -fPIC hnsw_baseline.cpp -o libhnsw_baseline.so
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <mutex>
#include <queue>
#include <random>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

struct Spin {
    std::atomic_flag f = ATOMIC_FLAG_INIT;
    void lock() {
        while (f.test_and_set(std::memory_order_acquire)) {
        }
    }
    void unlock() { f.clear(std::memory_order_release); }
};

typedef std::pair<float, uint32_t> Cand;  // (distance, id)

struct Hnsw {
    uint32_t dim, M, M0, efc;
    double mult;
    std::vector<float> data;                       // rows are copied in: the index owns them
    std::vector<int> level;                        // top layer of each node
    std::vector<std::vector<uint32_t>> links0;     // layer 0: count + M0 ids per node, flat per node
    std::vector<std::vector<std::vector<uint32_t>>> upper;  // [node][layer-1] -> ids
    std::vector<Spin> locks;
    std::mutex global;
    int max_level = -1;
    uint32_t entry = 0;
    size_t n = 0;
    std::mt19937_64 rng;

    const float* row(uint32_t i) const { return data.data() + (size_t)i * dim; }
    float dist(const float* a, const float* b) const {
        float s = 0.0f;
        for (uint32_t i = 0; i < dim; ++i) {
            const float d = a[i] - b[i];
            s += d * d;
        }
        return s;
    }
    std::vector<uint32_t>& links(uint32_t node, int layer) { return layer == 0 ? links0[node] : upper[node][layer - 1]; }
};

struct Visited {
    std::vector<uint32_t> tag;
    uint32_t cur = 0;
    void reset(size_t n) {
        if (tag.size() < n) tag.assign(n, 0), cur = 0;
        if (++cur == 0) {
            std::fill(tag.begin(), tag.end(), 0);
            cur = 1;
        }
    }
    bool test_and_set(uint32_t i) {
        if (tag[i] == cur) return true;
        tag[i] = cur;
        return false;
    }
};

// Algorithm 2: ef nearest elements of one layer, starting from `ep`
std::vector<Cand> search_layer(Hnsw& h, const float* q, const std::vector<Cand>& ep, uint32_t ef, int layer, Visited& vis,
                               bool locked) {
    std::priority_queue<Cand> best;                                        // farthest on top
    std::priority_queue<Cand, std::vector<Cand>, std::greater<Cand>> open;  // nearest on top
    for (const Cand& c : ep) {
        vis.test_and_set(c.second);
        best.push(c);
        open.push(c);
    }
    std::vector<uint32_t> nb;
    while (!open.empty()) {
        const Cand c = open.top();
        if (c.first > best.top().first && best.size() >= ef) break;
        open.pop();
        if (locked) {
            h.locks[c.second].lock();
            nb = h.links(c.second, layer);
            h.locks[c.second].unlock();
        } else {
            nb = h.links(c.second, layer);
        }
        for (uint32_t e : nb) {
            if (vis.test_and_set(e)) continue;
            const float d = h.dist(q, h.row(e));
            if (best.size() < ef || d < best.top().first) {
                open.push({d, e});
                best.push({d, e});
                if (best.size() > ef) best.pop();
            }
        }
    }
    std::vector<Cand> out(best.size());
    for (size_t i = out.size(); i-- > 0;) {
        out[i] = best.top();
        best.pop();
    }
    return out;  // ascending
}

// Algorithm 4: neighbour selection heuristic (no extension, no pruned-connection keeping)
std::vector<uint32_t> select_heuristic(Hnsw& h, const std::vector<Cand>& cand_sorted, uint32_t m) {
    std::vector<uint32_t> out;
    for (const Cand& c : cand_sorted) {
        if (out.size() >= m) break;
        bool good = true;
        for (uint32_t r : out)
            if (h.dist(h.row(c.second), h.row(r)) < c.first) {
                good = false;
                break;
            }
        if (good) out.push_back(c.second);
    }
    return out;
}

void insert_one(Hnsw& h, uint32_t id, Visited& vis) {
    const float* q = h.row(id);
    const int lvl = h.level[id];
    std::unique_lock<std::mutex> g(h.global);
    const int top = h.max_level;
    uint32_t ep = h.entry;
    if (top < 0) {
        h.max_level = lvl;
        h.entry = id;
        return;
    }
    if (lvl <= top) g.unlock();  // only a new top layer keeps the global lock
    vis.reset(h.n);
    float epd = h.dist(q, h.row(ep));
    for (int l = top; l > lvl; --l) {  // greedy descent
        bool moved = true;
        while (moved) {
            moved = false;
            h.locks[ep].lock();
            std::vector<uint32_t> nb = h.links(ep, l);
            h.locks[ep].unlock();
            for (uint32_t e : nb) {
                const float d = h.dist(q, h.row(e));
                if (d < epd) {
                    epd = d;
                    ep = e;
                    moved = true;
                }
            }
        }
    }
    std::vector<Cand> eps{{epd, ep}};
    for (int l = std::min(lvl, top); l >= 0; --l) {
        vis.reset(h.n);
        std::vector<Cand> w = search_layer(h, q, eps, h.efc, l, vis, true);
        const uint32_t mmax = l == 0 ? h.M0 : h.M;
        std::vector<uint32_t> sel = select_heuristic(h, w, h.M);
        h.locks[id].lock();
        h.links(id, l) = sel;
        h.locks[id].unlock();
        for (uint32_t e : sel) {
            h.locks[e].lock();
            std::vector<uint32_t>& le = h.links(e, l);
            if (le.size() < mmax) {
                le.push_back(id);
            } else {  // shrink with the same heuristic
                std::vector<Cand> c;
                c.reserve(le.size() + 1);
                c.push_back({h.dist(h.row(e), q), id});
                for (uint32_t x : le) c.push_back({h.dist(h.row(e), h.row(x)), x});
                std::sort(c.begin(), c.end());
                le = select_heuristic(h, c, mmax);
            }
            h.locks[e].unlock();
        }
        eps = w;
    }
    if (lvl > top) {
        h.max_level = lvl;
        h.entry = id;
    }
}

std::vector<Cand> knn(Hnsw& h, const float* q, uint32_t ef, Visited& vis) {
    if (h.max_level < 0) return {};
    uint32_t ep = h.entry;
    float epd = h.dist(q, h.row(ep));
    for (int l = h.max_level; l > 0; --l) {
        bool moved = true;
        while (moved) {
            moved = false;
            for (uint32_t e : h.links(ep, l)) {
                const float d = h.dist(q, h.row(e));
                if (d < epd) {
                    epd = d;
                    ep = e;
                    moved = true;
                }
            }
        }
    }
    vis.reset(h.n);
    return search_layer(h, q, {{epd, ep}}, ef, 0, vis, false);
}

int nthreads(int t) {
#ifdef _OPENMP
    return t > 0 ? t : omp_get_max_threads();
#else
    (void)t;
    return 1;
#endif
}

}  // namespace

extern "C" {

void* hnsw_create(uint32_t dim, uint32_t M, uint32_t ef_construction, uint64_t seed) {
    Hnsw* h = new Hnsw();
    h->dim = dim;
    h->M = M;
    h->M0 = 2 * M;
    h->efc = ef_construction;
    h->mult = 1.0 / std::log((double)M);
    h->rng.seed(seed);
    return h;
}

void hnsw_destroy(void* p) { delete static_cast<Hnsw*>(p); }

size_t hnsw_size(void* p) { return static_cast<Hnsw*>(p)->n; }

// appends `count` rows (ids continue from the current size); insertion is parallel over rows
void hnsw_add(void* p, size_t count, const float* rows, int threads) {
    Hnsw& h = *static_cast<Hnsw*>(p);
    const size_t old = h.n, total = old + count;
    h.data.insert(h.data.end(), rows, rows + count * h.dim);
    h.level.resize(total);
    h.links0.resize(total);
    h.upper.resize(total);
    {
        std::vector<Spin> nl(total);
        h.locks.swap(nl);
    }
    std::uniform_real_distribution<double> u(0.0, 1.0);
    for (size_t i = old; i < total; ++i) {
        const int l = (int)(-std::log(1.0 - u(h.rng)) * h.mult);
        h.level[i] = l;
        h.links0[i].reserve(h.M0 + 1);
        h.upper[i].resize(l);
    }
    h.n = total;
    size_t first = old;
    if (old == 0 && count > 0) {  // the first node alone, so that there is an entry point
        Visited v;
        insert_one(h, 0, v);
        first = 1;
    }
#pragma omp parallel num_threads(nthreads(threads))
    {
        Visited vis;
#pragma omp for schedule(dynamic, 64)
        for (long long i = (long long)first; i < (long long)total; ++i) insert_one(h, (uint32_t)i, vis);
    }
}

void hnsw_search(void* p, const float* queries, size_t nq, uint32_t k, uint32_t ef, int64_t* out_ids, float* out_dists,
                 int threads) {
    Hnsw& h = *static_cast<Hnsw*>(p);
#pragma omp parallel num_threads(nthreads(threads))
    {
        Visited vis;
#pragma omp for schedule(dynamic, 16)
        for (long long qi = 0; qi < (long long)nq; ++qi) {
            std::vector<Cand> r = knn(h, queries + (size_t)qi * h.dim, std::max(ef, k), vis);
            for (uint32_t j = 0; j < k; ++j) {
                out_ids[qi * k + j] = j < r.size() ? (int64_t)r[j].second : -1;
                out_dists[qi * k + j] = j < r.size() ? r[j].first : 3.40282e38f;
            }
        }
    }
}

// timestamps[id] in [start,end) per query; ef doubles until k results pass or ef covers the index
void hnsw_search_range(void* p, const float* queries, size_t nq, uint32_t k, uint32_t ef, const uint64_t* timestamps,
                       const uint64_t* win_start, const uint64_t* win_end, int64_t* out_ids, float* out_dists,
                       uint64_t* distance_evals_unused, int threads) {
    (void)distance_evals_unused;
    Hnsw& h = *static_cast<Hnsw*>(p);
#pragma omp parallel num_threads(nthreads(threads))
    {
        Visited vis;
#pragma omp for schedule(dynamic, 16)
        for (long long qi = 0; qi < (long long)nq; ++qi) {
            uint32_t e = std::max(ef, k);
            std::vector<Cand> keep;
            for (;;) {
                std::vector<Cand> r = knn(h, queries + (size_t)qi * h.dim, e, vis);
                keep.clear();
                for (const Cand& c : r) {
                    const uint64_t t = timestamps[c.second];
                    if (t >= win_start[qi] && t < win_end[qi]) keep.push_back(c);
                    if (keep.size() == k) break;
                }
                if (keep.size() >= k || e >= h.n) break;
                e = (uint32_t)std::min<size_t>((size_t)e * 2, h.n);
            }
            for (uint32_t j = 0; j < k; ++j) {
                out_ids[qi * k + j] = j < keep.size() ? (int64_t)keep[j].second : -1;
                out_dists[qi * k + j] = j < keep.size() ? keep[j].first : 3.40282e38f;
            }
        }
    }
}

}  // extern "C"
