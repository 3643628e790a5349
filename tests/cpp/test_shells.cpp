// Exercises the C++ class shells the way the reference's own drivers use its classes
// (tests/test_cagra_index.cu, tests/test_cagra_insert.cu, tests/test_cagra_auto.cu): build, query,
// insert, range query with the bound-error check, save/load; recall against exact brute force.
// Usage: test_shells            full run, needs a GPU
//        test_shells --no-gpu   only checks that construction fails loudly without a GPU
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <set>
#include <vector>

#include "cagraIndex.hpp"
#include "cagraIndexOpt.hpp"
#include "timeStampIndex.hpp"
#include "vmm_allocator.hpp"

static float l2(const float* a, const float* b, int dim) {  // tests/test_cagra_auto.cu:48-50
    float r = 0;
    for (int i = 0; i < dim; ++i) {
        float d = a[i] - b[i];
        r += d * d;
    }
    return r;
}

static std::vector<std::vector<int64_t>> ground_truth(const std::vector<float>& data, const std::vector<uint64_t>& ts,
                                                      size_t n, const std::vector<float>& q, size_t nq, int dim, int k,
                                                      uint64_t s, uint64_t e) {
    std::vector<std::vector<int64_t>> gt(nq);
    for (size_t i = 0; i < nq; ++i) {
        std::vector<std::pair<float, int64_t>> c;
        for (size_t j = 0; j < n; ++j)
            if (ts[j] >= s && ts[j] < e) c.push_back({l2(&q[i * dim], &data[j * dim], dim), (int64_t)j});
        size_t keep = std::min<size_t>(k, c.size());
        std::partial_sort(c.begin(), c.begin() + keep, c.end());
        for (size_t r = 0; r < keep; ++r) gt[i].push_back(c[r].second);
    }
    return gt;
}

static double recall(const std::vector<int64_t>& ids, const std::vector<std::vector<int64_t>>& gt, size_t nq, int k) {
    size_t hit = 0, tot = 0;
    for (size_t i = 0; i < nq; ++i) {
        std::set<int64_t> g(gt[i].begin(), gt[i].end());
        if (g.empty()) continue;
        for (int r = 0; r < k; ++r) hit += g.count(ids[i * k + r]);
        tot += g.size();
    }
    return tot ? (double)hit / tot : 0.0;
}

#define REQUIRE(cond)                                                        \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::printf("FAILED: %s (line %d)\n", #cond, __LINE__);          \
            return 1;                                                        \
        }                                                                    \
    } while (0)

int main(int argc, char** argv) {
    if (argc > 1 && std::strcmp(argv[1], "--no-gpu") == 0) {
        if (grab_device_count() > 0) {
            std::printf("SKIPPED: a GPU is present\n");
            return 0;
        }
        try {
            cagra::CagraIndex idx(128, 32, 1ull << 28);
        } catch (const std::runtime_error& e) {
            std::printf("PASSED: construction without a GPU throws: %s\n", e.what());
            return 0;
        }
        std::printf("FAILED: construction without a GPU did not throw\n");
        return 1;
    }

    const int dim = 128, k = 10;
    const size_t n0 = 6000, n_ins = 1000, nq = 200, n = n0 + n_ins;
    std::mt19937 gen(42);
    std::uniform_real_distribution<float> dis(-1.0f, 1.0f);  // tests/test_cagra_build.cu:69-74
    std::vector<float> data(n * dim), q(nq * dim);
    for (auto& x : data) x = dis(gen);
    for (auto& x : q) x = dis(gen);
    std::vector<uint64_t> ts(n);
    for (size_t i = 0; i < n; ++i) ts[i] = i / 500;  // ts[i] = i / bucket_size (tests/test_cagra_opt_search_range.cu:444-446)

    cagra::CagraIndex idx(dim, 32, 1ull << 30);
    idx.setSeed(7);
    std::vector<int64_t> ids(nq * k, -7);
    std::vector<float> dist(nq * k);
    idx.query(q.data(), nq, k, ids.data(), dist.data());  // empty index: silent return
    REQUIRE(ids[0] == -7);
    idx.add(n0, data.data(), ts.data());
    REQUIRE(idx.size() == n0);
    idx.build();
    idx.query(q.data(), nq, k, ids.data(), dist.data());
    auto gt = ground_truth(data, ts, n0, q, nq, dim, k, 0, ~0ull);
    double r = recall(ids, gt, nq, k);
    std::printf("recall@%d after build: %.4f\n", k, r);
    REQUIRE(r > 0.90);
    for (size_t i = 0; i < nq; ++i)
        for (int j = 1; j < k; ++j) REQUIRE(dist[i * k + j] >= dist[i * k + j - 1]);

    idx.insert(n_ins, data.data() + n0 * dim, ts.data() + n0);
    REQUIRE(idx.size() == n);
    idx.query(q.data(), nq, k, ids.data(), dist.data());
    gt = ground_truth(data, ts, n, q, nq, dim, k, 0, ~0ull);
    r = recall(ids, gt, nq, k);
    std::printf("recall@%d after insert: %.4f\n", k, r);
    REQUIRE(r > 0.90);  // tests/test_cagra_insert.cu:284

    idx.query_range(q.data(), nq, k, 0.2f, 3, 9, ids.data(), dist.data());
    size_t bound_errors = 0;  // tests/test_cagra_opt_search_range.cu:254-261
    for (auto id : ids)
        if (id != -1 && (ts[id] < 3 || ts[id] >= 9)) ++bound_errors;
    gt = ground_truth(data, ts, n, q, nq, dim, k, 3, 9);
    r = recall(ids, gt, nq, k);
    std::printf("range recall@%d: %.4f, bound errors %zu\n", k, r, bound_errors);
    REQUIRE(bound_errors == 0 && r > 0.90);

    {   // per-query windows: the exact scan equals the brute force, and query_range_batch takes it up for narrow windows
        std::vector<uint64_t> ws(nq), we(nq);
        for (size_t i = 0; i < nq; ++i) {
            ws[i] = i % 12;
            we[i] = ws[i] + (i % 2 ? 1 : 6);  // one bucket of 500 rows, or six
        }
        idx.scan_range_batch(q.data(), nq, k, ws.data(), we.data(), ids.data(), dist.data());
        size_t wrong = 0;
        for (size_t i = 0; i < nq; ++i) {
            auto g = ground_truth(data, ts, n, std::vector<float>(q.begin() + i * dim, q.begin() + (i + 1) * dim), 1, dim, k, ws[i], we[i]);
            for (int j = 0; j < k; ++j) wrong += ids[i * k + j] != g[0][j];
        }
        std::printf("exact window scan: %zu ids differ from the brute force\n", wrong);
        REQUIRE(wrong == 0);
        std::vector<int64_t> auto_ids(nq * k);
        std::vector<float> auto_dist(nq * k);
        idx.setScanBelow(0.1);  // 700 rows: the one-bucket windows
        idx.query_range_batch(q.data(), nq, k, ws.data(), we.data(), auto_ids.data(), auto_dist.data());
        idx.setScanBelow(0.0);
        for (size_t i = 1; i < nq; i += 2)
            for (int j = 0; j < k; ++j) REQUIRE(auto_ids[i * k + j] == ids[i * k + j]);
    }

    idx.save("/tmp/grab_shell_test.bin");
    cagra::CagraIndex idx2(dim, 32, 1ull << 30);
    idx2.load("/tmp/grab_shell_test.bin");
    REQUIRE(idx2.size() == n);
    idx.setSeed(5);
    idx2.setSeed(5);
    std::vector<int64_t> ids2(nq * k);
    std::vector<float> dist2(nq * k);
    idx.query(q.data(), nq, k, ids.data(), dist.data());
    idx2.query(q.data(), nq, k, ids2.data(), dist2.data());
    REQUIRE(ids == ids2 && dist == dist2);
    bool threw = false;
    try {
        idx2.load("/tmp/does_not_exist.bin");
    } catch (const std::runtime_error&) {
        threw = true;
    }
    REQUIRE(threw);

    // CagraIndexOpt surface: bucket search returns only rows of the bucket
    cagra::CagraIndexOpt opt(dim, 32, 32, 1ull << 30);
    opt.add(n0, data.data(), ts.data());
    opt.build();
    opt.query_local(q.data(), nq, k, 4, ids.data(), dist.data());
    // seeds are inside the bucket; the traversal itself is unfiltered in the reference too, so
    // only non-emptiness and ordering are required here
    REQUIRE(ids[0] >= 0);
    opt.query_range(q.data(), nq, k, 100, 200, ids.data(), dist.data());  // empty range
    REQUIRE(ids[0] == -1 && dist[0] == -1.0f);
    REQUIRE(opt.get_ids_by_timestamp(2).size() == 500);
    {  // MCAG file: a second index loaded from it answers the same
        const std::string mcag = "/tmp/grab_shell_test.mcag";
        opt.save(mcag);
        cagra::CagraIndexOpt opt2(dim, 32, 32, 1ull << 30);
        opt2.load(mcag);
        REQUIRE(opt2.size() == opt.size());
        REQUIRE(std::memcmp(opt2.get_graph(), opt.get_graph(), opt.size() * 32 * sizeof(uint32_t)) == 0);
        REQUIRE(opt2.get_ids_by_timestamp(2).size() == 500);
        std::vector<uint32_t> sd = opt2.sample_seeds_by_time(1, 2, 16);  // inclusive upper bound
        REQUIRE(sd.size() == 16);
        for (uint32_t v : sd) REQUIRE(ts[v] >= 1 && ts[v] <= 2);
        std::remove(mcag.c_str());
    }

    {  // CagraIndexOpt::insert: rows added to bucket 2 afterwards are found by a search inside the bucket
        cagra::CagraIndexOpt split(dim, 32, 24, 1ull << 30);
        split.add(n0, data.data(), ts.data());
        split.build();
        std::vector<uint64_t> two(n_ins, 2);
        split.insert(n_ins, data.data() + n0 * dim, two.data());
        REQUIRE(split.size() == n0 + n_ins);
        REQUIRE(split.get_ids_by_timestamp(2).size() == 500 + n_ins);
        size_t found = 0;
        for (size_t i = 0; i < nq && i < n_ins; ++i) {  // the inserted row itself is its own nearest neighbour
            split.query_local(data.data() + (n0 + i) * dim, 1, k, 2, ids.data(), dist.data());
            found += ids[0] == (int64_t)(n0 + i);
        }
        std::printf("inserted rows found first by a bucket search: %zu of %zu\n", found, std::min(nq, n_ins));
        REQUIRE(found * 10 >= std::min(nq, n_ins) * 9);
    }

    // DeviceBufferVMM contract
    cagra::DeviceBufferVMM buf(64ull << 20);
    buf.resize(1000);
    void* p = buf.data();
    buf.resize(30ull << 20);
    REQUIRE(buf.data() == p && buf.size() >= (30ull << 20));
    threw = false;
    try {
        buf.resize(1ull << 40);
    } catch (const std::runtime_error& e) {
        threw = std::strstr(e.what(), "VMM OOM") != nullptr;
    }
    REQUIRE(threw);
    {  // timestamp::TimeStampIndex: rows of two timestamps, a query next to a row finds that row first
        timestamp::TimeStampIndex tsi(dim, 32);
        std::vector<uint64_t> two(n0);
        for (size_t i = 0; i < n0; ++i) two[i] = 100 + (i % 2);
        REQUIRE(tsi.insert(data.data(), two.data(), n0) == 0);
        REQUIRE(tsi.size() == n0);
        tsi.build_virtual_index();
        std::vector<int64_t> ti(k);
        std::vector<float> td(k);
        tsi.query(data.data() + 17 * dim, k, ti.data(), td.data(), 2);
        REQUIRE(ti[0] == 17 && td[0] == 0.0f);
    }
    std::printf("PASSED\n");
    return 0;
}
