"""Pins the CPU oracle against things it did not write itself: the reference's compiled
smem_cal.cuh, fixtures made with the recipes of the reference's own tests, closed forms,
float64, and independent pure-Python restatements on tiny inputs.  No GPU."""
import itertools
import json
import os

import numpy as np
import pytest

import datasets

HERE = os.path.dirname(os.path.abspath(__file__))


# ---------------------------------------------------------------- closed forms (smem_cal.cuh)
def test_next_power_of_2_and_capacity(oracle):
    for n, e in [(0, 1), (1, 1), (2, 2), (3, 4), (10, 16), (300, 512), (512, 512), (513, 1024), (2 ** 31, 2 ** 31)]:
        assert oracle.lib.orc_next_power_of_2(n) == e
    # (itopk, width, degree) -> capacity, cases worked out from src/index/smem_cal.cuh:43-46
    assert oracle.lib.orc_queue_capacity(64, 4, 64) == 512
    assert oracle.lib.orc_queue_capacity(256, 6, 64) == 1024
    assert oracle.lib.orc_queue_capacity(128, 4, 32) == 256
    assert oracle.lib.orc_queue_capacity(64, 1, 32) == 256  # floor of BLOCK_SIZE
    # 512 + 32768 + 4096 + 16 + 256 at dim 128, hash 13, capacity 512
    assert oracle.lib.orc_smem_bytes(64, 128, 4, 64, 13) == 37648


def test_closed_forms_against_compiled_reference_header(oracle):
    ref = oracle.ref_smem()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent when the oracle was built)")
    rng = np.random.default_rng(0)
    for n in list(range(0, 70)) + rng.integers(0, 2 ** 31, 200).tolist():
        assert oracle.lib.orc_next_power_of_2(int(n)) == ref.ref_next_power_of_2(int(n))
    for itopk, dim, sw, deg, bl in itertools.product([32, 64, 100, 256, 512], [96, 128, 768, 1024], [1, 4, 6], [32, 64, 128],
                                                     [10, 12, 13, 14, 15]):
        assert oracle.lib.orc_smem_bytes(itopk, dim, sw, deg, bl) == ref.ref_calculate_and_check_smem(itopk, dim, sw, deg, bl)


def test_search_plan_rules(oracle):
    # cagra::search: itopk = max(k, itopk, 64); seeds = raw itopk / 4 (src/index/cagra.cu:862-887)
    assert oracle.search_plan(oracle.WRAP_SEARCH, 10, 32, 4, 64) == (64, 8, 512)
    assert oracle.search_plan(oracle.WRAP_SEARCH, 10, 256, 6, 64) == (256, 64, 1024)
    assert oracle.search_plan(oracle.WRAP_SEARCH, 128, 128, 6, 64) == (128, 32, 512)
    assert oracle.search_plan(oracle.WRAP_SEARCH, 300, 64, 4, 64)[0] == 300
    # search_opt: seeds = min(max(32, provided), itopk) (src/index/cagra_opt.cu:1158-1160)
    assert oracle.search_plan(oracle.WRAP_SEARCH_OPT, 10, 64, 4, 32, 0)[:2] == (64, 32)
    assert oracle.search_plan(oracle.WRAP_SEARCH_OPT, 10, 64, 4, 32, 500)[:2] == (64, 64)
    # bucket: itopk >= 128 (:1243); range: itopk >= 64; seeds = min(provided, itopk)
    assert oracle.search_plan(oracle.WRAP_BUCKET, 10, 32, 4, 32, 200)[:2] == (128, 128)
    assert oracle.search_plan(oracle.WRAP_RANGE, 10, 32, 4, 64, 32)[:2] == (64, 32)
    assert oracle.search_plan(oracle.WRAP_RANGE, 10, 256, 4, 64, 0)[:2] == (256, 0)


def test_library_plan_and_closed_forms_match_oracle(oracle, grab):
    # host-only entry points of the product library (no GPU needed)
    for w, k, it, sw, deg, npv in itertools.product(range(4), [1, 10, 100], [16, 64, 200], [1, 4], [32, 64], [0, 17, 300]):
        assert grab.search_plan(w, k, it, sw, deg, npv) == oracle.search_plan(w, k, it, sw, deg, npv)
    for itopk, dim, sw, deg, bl in itertools.product([64, 256], [128, 768], [4, 6], [32, 64], [12, 13, 14]):
        assert grab.lib.grab_reference_smem_bytes(itopk, dim, sw, deg, bl) == oracle.lib.orc_smem_bytes(itopk, dim, sw, deg, bl)
        assert grab.lib.grab_queue_capacity(itopk, sw, deg) == oracle.lib.orc_queue_capacity(itopk, sw, deg)


# ---------------------------------------------------------------- sorting
def _fixtures():
    with open(os.path.join(HERE, "golden", "sort_fixtures.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("idx", range(7))
def test_bitonic_network_and_pair_sort_on_reference_recipes(oracle, idx):
    fx = _fixtures()[idx]
    keys = np.array(fx["key_bits"], np.uint32).view(np.float32)
    vals = np.arange(fx["n"], dtype=np.uint32)
    ek = np.array(fx["sorted_key_bits"], np.uint32)
    ev = np.array(fx["sorted_vals"], np.uint32)
    k, v = oracle.bitonic_network(keys, vals, 32, fx["n"] // 32)  # the reference's 32-lane network
    assert np.array_equal(k.view(np.uint32), ek)
    same_key_as_next = np.r_[ek[1:] == ek[:-1], False] | np.r_[False, ek[1:] == ek[:-1]]
    assert np.array_equal(v[~same_key_as_next], ev[~same_key_as_next])  # equal keys may come in any order there
    k, v = oracle.sort_pairs(keys, vals)
    assert np.array_equal(k.view(np.uint32), ek) and np.array_equal(v, ev)


def test_bitonic_network_zero_one_principle(oracle):
    # a comparator network sorts everything iff it sorts every 0/1 input: all 2^16 inputs, 4 lanes x 4
    vals = np.arange(16, dtype=np.uint32)
    for bits in range(1 << 16):
        keys = np.array([(bits >> i) & 1 for i in range(16)], np.float32)
        k, _ = oracle.bitonic_network(keys, vals, 4, 4)
        assert (np.diff(k) >= 0).all(), bits
    for bits in range(0, 1 << 16, 7):  # descending variant
        keys = np.array([(bits >> i) & 1 for i in range(16)], np.float32)
        k, _ = oracle.bitonic_network(keys, vals, 8, 2, asc=False)
        assert (np.diff(k) <= 0).all(), bits


def test_sort_special_inputs(oracle):
    for keys in (np.full(128, 5.0, np.float32), np.arange(128, 0, -1, dtype=np.float32), np.arange(128, dtype=np.float32),
                 np.r_[np.arange(60, dtype=np.float32), np.full(68, 3.40282e38, np.float32)]):
        vals = np.arange(128, dtype=np.uint32)[::-1].copy()
        k, v = oracle.sort_pairs(keys, vals)
        order = np.lexsort((vals, keys))
        assert np.array_equal(k, keys[order]) and np.array_equal(v, vals[order])
        k2, _ = oracle.bitonic_network(keys, vals, 32, 4)
        assert np.array_equal(k2, np.sort(keys))


# ---------------------------------------------------------------- visited set
def _py_hash_insert(table, bitlen, key):
    size = 1 << bitlen
    idx = (key ^ (key >> bitlen)) & (size - 1)
    for _ in range(size):
        if table[idx] == 0xFFFFFFFF:
            table[idx] = key
            return 1
        if table[idx] == key:
            return 0
        idx = (idx + 1) & (size - 1)
    return 0


@pytest.mark.parametrize("bitlen,n_unique,dup", [(10, 500, 0.4), (8, 200, 0.0), (8, 256, 0.0)])
def test_hash_reference_cases(oracle, bitlen, n_unique, dup):
    # tests/test_hashmap.cu:171-187
    keys = np.r_[np.arange(1, n_unique + 1), np.arange(1, int(n_unique * dup) + 1)].astype(np.uint32)
    res, table = oracle.hash_insert_many(bitlen, keys)
    assert int(res.sum()) == n_unique
    assert int((table != 0xFFFFFFFF).sum()) == n_unique
    py = [0xFFFFFFFF] * (1 << bitlen)
    exp = [_py_hash_insert(py, bitlen, int(k)) for k in keys]
    assert res.tolist() == exp and table.tolist() == py


def test_hash_full_and_random(oracle):
    rng = np.random.default_rng(1)
    keys = rng.integers(0, 2 ** 31, 700).astype(np.uint32)
    res, table = oracle.hash_insert_many(9, keys)  # 512 slots, > 512 distinct keys: the table fills up
    py = [0xFFFFFFFF] * 512
    exp = [_py_hash_insert(py, 9, int(k)) for k in keys]
    assert res.tolist() == exp and table.tolist() == py
    assert int(res.sum()) == 512 and (table != 0xFFFFFFFF).all()


# ---------------------------------------------------------------- distances
@pytest.mark.parametrize("dim", [4, 32, 96, 128, 768, 1024, 2048])
def test_distances_against_float64(oracle, dim):
    rng = np.random.default_rng(dim)
    for _ in range(20):
        a, b = rng.standard_normal(dim).astype(np.float32), rng.standard_normal(dim).astype(np.float32)
        ref = float(((a.astype(np.float64) - b.astype(np.float64)) ** 2).sum())
        for kind in ("canon", "natural", "ref_warp"):
            assert abs(oracle.l2(kind, a, b) - ref) <= 1e-5 * ref  # tolerance of the north star: 1e-5 relative
        dot = float((a.astype(np.float64) * b.astype(np.float64)).sum())
        mag = float(np.abs(a.astype(np.float64) * b.astype(np.float64)).sum())
        assert abs(oracle.l2("ip", a, b) + dot) <= 1e-5 * mag


def test_distances_exact_cases(oracle):
    rng = np.random.default_rng(0)
    for dim in (96, 128, 256):
        a = rng.integers(0, 256, dim).astype(np.float32)
        b = rng.integers(0, 256, dim).astype(np.float32)
        exact = int(((a.astype(np.int64) - b.astype(np.int64)) ** 2).sum())
        assert exact < 2 ** 24
        for kind in ("canon", "natural", "ref_warp"):  # integer inputs: every order gives the exact value
            assert oracle.l2(kind, a, b) == float(exact)
        assert oracle.l2("canon", a, a) == 0.0
        assert oracle.l2("ip", a, b) == -float((a.astype(np.int64) * b.astype(np.int64)).sum())
    u = datasets.unit_rows(2, 128, 5)
    d = oracle.l2("canon", u[0], u[1])
    assert abs(d - (2 + 2 * oracle.l2("ip", u[0], u[1]))) < 1e-5  # |a-b|^2 = 2 - 2ab on unit vectors
    # a dropped chunk or a wrong lane assignment shows up on one-hot inputs
    for pos in range(0, 128, 5):
        e = np.zeros(128, np.float32)
        e[pos] = 3.0
        assert oracle.l2("canon", e, np.zeros(128, np.float32)) == 9.0
        assert oracle.l2("ip", e, e) == -9.0


# ---------------------------------------------------------------- exact filtered top-k
def test_bruteforce_topk_vs_numpy(oracle):
    data = datasets.mixture(3000, 128, 5, 1, 2)  # integer data: many exact ties
    data[100:110] = data[50]                      # duplicated rows: ties must go to the lower id
    q = datasets.mixture(40, 128, 5, 1, 3)
    q[0] = data[50]
    ts = np.arange(3000, dtype=np.uint64)
    ws, we = datasets.windows(3000, 40, 0.2, 4)
    ids, dist = oracle.bruteforce_topk(data, q, 10)
    for i in range(40):
        d = ((q[i][None].astype(np.float64) - data.astype(np.float64)) ** 2).sum(1)
        order = np.lexsort((np.arange(3000), d))[:10]
        assert np.array_equal(ids[i], order) and np.array_equal(dist[i].astype(np.float64), d[order])
    assert ids[0].tolist()[:4] == [50, 100, 101, 102]
    ids, dist = oracle.bruteforce_topk(data, q, 10, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws, win_end=we)
    for i in range(40):
        d = ((q[i][None].astype(np.float64) - data.astype(np.float64)) ** 2).sum(1)
        inside = np.nonzero((ts >= ws[i]) & (ts < we[i]))[0]
        order = inside[np.lexsort((inside, d[inside]))][:10]
        assert np.array_equal(ids[i], order)
    # fewer than k rows pass: -1 padding
    ids, dist = oracle.bruteforce_topk(data, q[:2], 10, filter_kind=oracle.FILTER_RANGE, ts=ts, win=(7, 10))
    assert (ids[:, :3] >= 7).all() and (ids[:, 3:] == -1).all() and (dist[:, 3:] == np.float32(3.40282e38)).all()


# ---------------------------------------------------------------- graph build
def test_knn_graph_points_on_a_line(oracle):
    # recipe of tests/test_knn_build.cu:32-38 at reduced size: all components equal to i*0.001
    n, dim, k = 1500, 64, 10
    data = np.repeat((np.arange(n, dtype=np.float32) * np.float32(0.001))[:, None], dim, axis=1)
    g = oracle.knn_graph(data, k)
    assert not (g == np.arange(n, dtype=np.uint32)[:, None]).any()  # no self loops (:58-75)
    hit = 0
    for i in range(n):
        ideal = sorted(range(max(0, i - k), min(n, i + k + 1)), key=lambda j: (abs(j - i), j))[1:k + 1]
        hit += len(set(ideal) & set(g[i].tolist())) / k
    assert hit / n > 0.99  # :111


def test_knn_graph_order_self_and_padding(oracle):
    data = datasets.mixture(300, 32, 3, 1, 2)
    data[10] = data[3]
    g = oracle.knn_graph(data, 16)
    for i in range(300):
        d = ((data[i][None].astype(np.float64) - data.astype(np.float64)) ** 2).sum(1)
        order = [j for j in np.lexsort((np.arange(300), d)) if j != i][:16]
        assert g[i].tolist() == order
    small = oracle.knn_graph(data[:5], 8)
    assert (small[:, 4:] == 0xFFFFFFFF).all() and (small[:, :4] != 0xFFFFFFFF).all()


def _py_detour(knn):
    """kern_prune as written (src/index/cagra.cu:244-275), one node at a time."""
    n, deg = knn.shape
    out = np.zeros((n, deg), np.int64)
    for a in range(n):
        for kad in range(deg - 1):
            d = int(knn[a, kad])
            if d == 0xFFFFFFFF:
                continue
            for kdb in range(deg):
                cand = knn[d, kdb]
                for kab in range(kad + 1, deg):
                    if knn[a, kab] == cand:
                        out[a, kab] += 1
                        break
    return np.minimum(out, 255).astype(np.uint8)


def test_detour_counts_and_prune(oracle):
    rng = np.random.default_rng(2)
    data = rng.standard_normal((60, 8)).astype(np.float32)
    knn = oracle.knn_graph(data, 16)
    cnt = oracle.detour_counts(knn)
    assert np.array_equal(cnt, _py_detour(knn))
    pruned = oracle.prune(knn, 8)
    for i in range(60):
        order = sorted(range(16), key=lambda p: (cnt[i, p], p))[:8]  # stable sort by count (:381-391)
        assert pruned[i].tolist() == knn[i, order].tolist()
    # rows with repeated ids and padding behave like the literal loops
    g = rng.integers(0, 30, (30, 12)).astype(np.uint32)
    g[::4, 9:] = 0xFFFFFFFF
    assert np.array_equal(oracle.detour_counts(g), _py_detour(g))


def test_detour_closed_forms(oracle):
    # complete graph on d+1 nodes with rows in ascending id order: B = row[k] is reached through every D before it
    d = 12
    knn = np.array([[j for j in range(d + 1) if j != i] for i in range(d + 1)], np.uint32)
    cnt = oracle.detour_counts(knn)
    for i in range(d + 1):
        assert cnt[i].tolist() == list(range(d))
    # no 2-hop path lands in the row: all counts 0 and pruning keeps the first out_degree entries
    n = 40
    ring = np.array([[(i + 1 + 2 * j) % n for j in range(6)] for i in range(n)], np.uint32)
    assert not _py_detour(ring).any()
    assert np.array_equal(oracle.prune(ring, 3), ring[:, :3])


def _py_reverse(g):
    n, deg = g.shape
    rev = np.full((n, deg), 0xFFFFFFFF, np.uint32)
    cnt = np.zeros(n, np.uint32)
    for k in range(deg):           # column by column (src/index/cagra.cu:496-517)
        for src in range(n):       # ascending source = sequential execution of kern_make_rev_graph
            dst = int(g[src, k])
            if dst >= n:
                continue
            if cnt[dst] < deg:
                rev[dst, cnt[dst]] = src
            cnt[dst] += 1
    return rev, cnt


def _py_merge(g, rev, cnt):
    """optimize_merge_graphs as written (src/index/cagra.cu:574-650)."""
    n, deg = g.shape
    out = g.copy()
    for j in range(n):
        nb = []
        cf = cr = 0
        rc = min(int(cnt[j]), deg)
        while len(nb) < deg:
            added = False
            while cf < deg:
                c = int(g[j, cf]); cf += 1
                if c == j or c in nb:
                    continue
                nb.append(c); added = True
                break
            if len(nb) >= deg:
                break
            while cr < rc:
                c = int(rev[j, cr]); cr += 1
                if c >= n or c == j or c in nb:
                    continue
                nb.append(c); added = True
                break
            if not added:
                break
        out[j, :len(nb)] = nb
    return out


def test_reverse_and_merge(oracle):
    rng = np.random.default_rng(3)
    g = rng.integers(0, 50, (50, 8)).astype(np.uint32)
    g[:, 0] = 7                   # a hub: more in-edges than slots
    g[::5, 6:] = 0xFFFFFFFF
    rev, cnt = oracle.reverse_graph(g)
    erev, ecnt = _py_reverse(g)
    assert np.array_equal(rev, erev) and np.array_equal(cnt, ecnt)
    indeg = np.bincount(g[g < 50].astype(np.int64), minlength=50)
    assert np.array_equal(cnt, indeg)           # counts keep running past the row width (:437)
    assert cnt[7] >= 50 and (rev[7] != 0xFFFFFFFF).all()
    assert np.array_equal(oracle.merge_graphs(g, rev, cnt), _py_merge(g, rev, cnt))
    data = rng.standard_normal((80, 8)).astype(np.float32)
    knn = oracle.knn_graph(data, 16)
    pr = oracle.prune(knn, 8)
    rv, c = oracle.reverse_graph(pr)
    assert np.array_equal(oracle.optimize(knn, 8), _py_merge(pr, rv, c))


# ---------------------------------------------------------------- beam search
@pytest.fixture(scope="module")
def small(oracle):
    data = datasets.gaussian(2000, 64, 1)
    return data, oracle.optimize(oracle.knn_graph(data, 64), 32)


def test_search_invariants(oracle, small):
    data, graph = small
    q = datasets.gaussian(60, 64, 2)
    ts = np.arange(2000, dtype=np.uint64)
    seeds = np.tile(np.arange(500, 564, dtype=np.uint32), (60, 1))
    ids, dist, ctr = oracle.search(data, graph, q, 10, 64, 4, 50, 13, 64, 5, seeds=seeds, filter_kind=oracle.FILTER_RANGE,
                                   ts=ts, win=(400, 1200))
    assert (np.diff(dist, axis=1) >= 0).all()                      # ascending
    v = ids[ids >= 0]
    assert ((v >= 400) & (v < 1200)).all()                         # bound errors == 0
    for r in ids:
        assert len(set(r[r >= 0].tolist())) == (r >= 0).sum()      # no duplicate ids
    for i in range(60):                                            # reported distances are the canonical ones
        ok = ids[i] >= 0
        assert np.array_equal(dist[i][ok], oracle.distance_many(q[i], data, ids[i][ok].astype(np.uint32)))
    gt, _ = oracle.bruteforce_topk(data, q, 10, filter_kind=oracle.FILTER_RANGE, ts=ts, win=(400, 1200))
    assert datasets.recall(ids, gt) > 0.9
    assert (ctr[:, 1] == 64).all() and (ctr[:, 2] <= 4 * ctr[:, 0]).all() and (ctr[:, 4] <= ctr[:, 3]).all()


def test_search_exhaustive_equals_exact(oracle):
    data = datasets.gaussian(300, 64, 3)
    graph = oracle.optimize(oracle.knn_graph(data, 64), 32)
    q = datasets.gaussian(20, 64, 4)
    ids, dist, _ = oracle.search(data, graph, q, 10, 512, 8, 200, 13, 128, 9)
    gt, gd = oracle.bruteforce_topk(data, q, 10)
    assert np.array_equal(ids, gt) and np.array_equal(dist, gd)


def test_search_strict_reference_quirks(oracle, small):
    data, graph = small
    q = datasets.gaussian(10, 64, 5)
    ts = np.arange(2000, dtype=np.uint64)
    seeds = np.tile(np.array([1000, 1000, 5, 1001] * 8, np.uint32), (10, 1))
    sid, _, _ = oracle.search(data, graph, q, 10, 64, 4, 0, 13, 32, 1, seeds=seeds, filter_kind=oracle.FILTER_RANGE, ts=ts,
                              win=(990, 1400), flags=oracle.FLAG_STRICT)
    fid, _, _ = oracle.search(data, graph, q, 10, 64, 4, 0, 13, 32, 1, seeds=seeds, filter_kind=oracle.FILTER_RANGE, ts=ts,
                              win=(990, 1400))
    # zero iterations: the result is the sorted seed list.  Literal mode keeps duplicates and the
    # out-of-window seed 5 (compute_distance.cuh:237-266); the default drops both and pads with -1.
    for r in sid:
        assert sorted(r.tolist()).count(1000) >= 2 or sorted(r.tolist()).count(1001) >= 2 or 5 in r
    for r in fid:
        assert sorted(r[r >= 0].tolist()) == [1000, 1001] and (r[2:] == -1).all()
    # an unfilled slot is 2147483647 in literal mode (search.cu:351)
    one = np.array([[1000]], np.uint32)
    sid, sd, _ = oracle.search(data, graph, q[:1], 4, 64, 4, 0, 13, 1, 1, seeds=one, flags=oracle.FLAG_STRICT)
    assert sid[0].tolist() == [1000, 0x7FFFFFFF, 0x7FFFFFFF, 0x7FFFFFFF] and sd[0, 1] == np.float32(3.40282e38)


def test_random_seed_formula(oracle, small):
    data, graph = small
    q = datasets.gaussian(1, 64, 6)
    mask = 0xDEADBEEF
    ids, _, ctr = oracle.search(data, graph, q, 8, 64, 4, 0, 13, 8, mask)
    exp = {(mask * (i + 1)) % 2000 for i in range(8)}  # compute_distance.cuh:176
    assert set(ids[0][ids[0] >= 0].tolist()) == exp


# ---------------------------------------------------------------- seed sampling, rng, insert
def test_window_seed_sampler_properties(oracle):
    ts = np.sort(np.random.default_rng(1).integers(0, 300, 4000)).astype(np.uint64)
    order = np.arange(4000, dtype=np.uint32)
    ws = np.array([0, 50, 299, 120, 400], np.uint64)
    we = np.array([300, 60, 300, 120, 500], np.uint64)
    s = oracle.sample_window_seeds(ts, order, 32, 7, win_start=ws, win_end=we)
    for i in range(5):
        inside = np.nonzero((ts >= ws[i]) & (ts < we[i]))[0]
        v = s[i][s[i] != 0xFFFFFFFF]
        assert set(v.tolist()) <= set(inside.tolist())
        assert len(set(v.tolist())) == v.size == min(32, inside.size)  # distinct, all of a small window


def test_splitmix64_known_answers(oracle):
    # first outputs of SplitMix64 seeded with 1234567 (Vigna's reference implementation)
    state = 1234567
    out = []
    for _ in range(3):
        v, state = oracle.splitmix64(state)
        out.append(v)
    assert out == [6457827717110365317, 3203168211198807973, 9817491932198370423]


def test_insert_invariants_and_lcg(oracle):
    n0, n_new, deg = 1500, 100, 16
    data = datasets.gaussian(n0 + n_new, 64, 8)
    graph = np.full((n0 + n_new, deg), 0xFFFFFFFF, np.uint32)
    graph[:n0] = oracle.optimize(oracle.knn_graph(data[:n0], 32), deg)
    before = graph.copy()
    after, _ = oracle.insert_batch(data, n0, n_new, graph, 128, 6, 50, 12, 99)
    new_rows = after[n0:]
    assert ((new_rows < n0)).all()                         # new rows hold old ids only, all slots filled here
    for i in range(n_new):                                 # ... and they are the true nearest found, ascending
        d = oracle.distance_many(data[n0 + i], data, new_rows[i])
        assert (np.diff(d) >= 0).all()
    assert (after[:n0] != 0xFFFFFFFF).all()                # old rows stay full
    changed = np.nonzero((after[:n0] != before[:n0]).any(axis=1))[0]
    assert changed.size > 0
    for t in changed:                                      # only new ids were written into old rows
        diff = after[t] != before[t]
        assert (after[t][diff] >= n0).all()
    counts = np.bincount(after[:n0][after[:n0] >= n0].astype(np.int64) - n0, minlength=n_new)
    assert (counts <= 2 * deg).all()                       # a new id enters at most search_k old rows
    # slot choice: LCG of insert.cu:319-365 for a target that received exactly one request at a known position
    # (closed form re-derived here, independent of the C++ code)
    gt, _ = oracle.bruteforce_topk(data[:n0 + n_new], data[n0:n0 + n_new], 10)
    assert datasets.recall(after[n0:, :10].astype(np.int64), np.where(gt >= n0, -1, gt)) > 0.5
    # striped mode (insert.cu:100-117): with search_k = 32 and a 64-slot network, output slot p takes sorted
    # rank 2p, so the new row holds every second result and ranks past 31 are padding
    striped, _ = oracle.insert_batch(data, n0, n_new, graph, 128, 6, 50, 12, 99, striped_sort=1)
    full = oracle.search(data[:n0], graph[:n0], data[n0:], 32, 128, 6, 50, 12, 32, oracle.splitmix64(99)[0] & 0xFFFFFFFF)[0]
    assert np.array_equal(after[n0:n0 + 64], full[:64, :16].astype(np.uint32))   # default: the first deg results
    assert np.array_equal(striped[n0:n0 + 64], full[:64, 0:32:2].astype(np.uint32))


def test_insert_lcg_closed_form(oracle):
    # one new row, search_k = 2*deg results; recompute every slot decision in Python
    n0, deg = 200, 8
    data = datasets.gaussian(n0 + 1, 32, 11)
    graph = np.full((n0 + 1, deg), 0xFFFFFFFF, np.uint32)
    graph[:n0] = oracle.optimize(oracle.knn_graph(data[:n0], 16), deg)
    after, _ = oracle.insert_batch(data, n0, 1, graph, 128, 6, 50, 12, 3)
    # every old node that now holds the new id was one of the 16 search results; sort them as the kernel does
    targets = sorted(int(t) for t in np.nonzero((after[:n0] == n0).any(axis=1))[0])
    M = (1 << 64) - 1
    found = oracle.search(data[:n0], graph[:n0], data[n0:], 16, 128, 6, 50, 12, 32, oracle.splitmix64(3)[0] & 0xFFFFFFFF)[0][0]
    req = sorted(int(t) for t in found if 0 <= t < n0)
    assert set(targets) <= set(req)
    for pos, t in enumerate(req):
        rng = (t * 0x9e3779b97f4a7c15 + pos) & M
        rng = (rng * 6364136223846793005 + 1) & M
        r1 = rng >> 32
        rng = (rng * 6364136223846793005 + 1) & M
        r2 = rng >> 32
        slot = (r2 % (deg // 2)) if r1 % 10 == 0 else deg // 2 + (r2 % (deg - deg // 2))
        assert after[t, slot] == n0
        others = np.delete(after[t], slot)
        assert np.array_equal(others, np.delete(graph[t], slot))


# ---- time-partitioned graph: remote edges and reverse injection ----
def _py_wang(seed):
    seed &= 0xFFFFFFFF
    seed = (seed ^ 61) ^ (seed >> 16)
    seed = (seed * 9) & 0xFFFFFFFF
    seed ^= seed >> 4
    seed = (seed * 0x27D4EB2D) & 0xFFFFFFFF
    seed ^= seed >> 15
    return seed


def _py_remote_edges(cand, ts, graph, total, local):
    """The rule of update_remote_edges_kernel (src/index/cagra_opt.cu:209-303), written from its description:
    candidates nearest first; first up to a third of the remote slots from other buckets within +-20 % of the
    bucket range, then farther buckets, then any other bucket; a candidate is used once."""
    n = len(ts)
    g = graph.copy()
    buckets = int(ts[-1]) + 1
    span = max(1, buckets // 5)
    slots = total - local
    for i in range(n):
        lo, hi = max(0, int(ts[i]) - span), min(buckets - 1, int(ts[i]) + span)
        usable = [(k, int(c)) for k, c in enumerate(cand[i]) if c != i and c != 0xFFFFFFFF and ts[c] != ts[i]]
        near = [(k, c) for k, c in usable if lo <= ts[c] <= hi][:slots // 3]
        taken = {k for k, _ in near}
        far = [(k, c) for k, c in usable if not (lo <= ts[c] <= hi)][:slots - len(near)]
        taken |= {k for k, _ in far}
        rest = [(k, c) for k, c in usable if k not in taken][:slots - len(near) - len(far)]
        out = [c for _, c in near] + [c for _, c in far] + [c for _, c in rest]
        g[i, local:local + len(out)] = out
    return g


def _py_inject(graph, total, local):
    n = graph.shape[0]
    g = graph.copy()
    rev = [[] for _ in range(n)]
    for src in range(n):
        for k in range(local, total):
            d = int(g[src, k])
            if d != 0xFFFFFFFF and d < n:
                rev[d].append(src)
    remote = total - local
    strong = remote // 2
    weak = remote - strong
    for i in range(n):
        rng = _py_wang(i)
        for c in rev[i][:32]:
            if c in g[i].tolist():
                continue
            cur = g[i, local:]
            empty = [w for w in range(strong, remote) if cur[w] == 0xFFFFFFFF]
            if empty:
                cur[empty[0]] = c
            elif weak > 0:
                rng = _py_wang(rng)
                cur[strong + rng % weak] = c
    return g


def test_remote_global_k_closed_form(oracle):
    # (total - local) * 4, rounded up past the next multiple of 32, at least 64, at most 256 (cagra_opt.cu:808-810)
    assert [oracle.remote_global_k(t, l) for t, l in ((32, 28), (32, 16), (64, 48), (64, 32), (128, 0), (64, 63))] == \
        [64, 96, 96, 160, 256, 64]


@pytest.mark.parametrize("total,local,buckets", [(8, 5, 6), (12, 4, 11), (8, 8, 3), (6, 0, 4)])
def test_remote_edges_and_injection_match_independent_restatement(oracle, total, local, buckets):
    rng = np.random.default_rng(total * 100 + local)
    n, gk = 90, 24
    ts = np.sort(rng.integers(0, buckets, n)).astype(np.uint64)
    ts[0], ts[-1] = 0, buckets - 1
    graph = rng.integers(0, n, (n, total)).astype(np.uint32)
    cand = np.stack([rng.permutation(n)[:gk] for _ in range(n)]).astype(np.uint32)
    cand[rng.random((n, gk)) < 0.05] = 0xFFFFFFFF
    if total > local:
        got = oracle.remote_edges(cand, ts, graph, total, local)
        exp = _py_remote_edges(cand, ts, graph, total, local)
        assert np.array_equal(got, exp)
        assert np.array_equal(got[:, :local], graph[:, :local])               # local slots untouched
        rem = got[:, local:]
        changed = rem != graph[:, local:]
        assert (ts[rem[changed]] != np.repeat(ts[:, None], total - local, 1)[changed]).all()  # remote = other bucket
    else:
        got = graph
    inj = oracle.inject_reverse_remote(got, total, local)
    assert np.array_equal(inj, _py_inject(got, total, local))
    strong = (total - local) // 2
    assert np.array_equal(inj[:, :local + strong], got[:, :local + strong])   # only the weak half changes


def test_partitioned_build_local_slots_stay_inside_the_bucket(oracle):
    n, dim, total, local = 600, 32, 16, 12
    data = datasets.gaussian(n, dim, 9)
    sizes = [150, 90, 200, 160]
    ts = np.repeat(np.arange(4, dtype=np.uint64), sizes)
    g = oracle.build_time_partitioned(data, ts, sizes, total, local)
    starts = np.concatenate([[0], np.cumsum(sizes)])
    for b in range(4):
        rows = g[starts[b]:starts[b + 1]]
        loc = rows[:, :local]
        assert ((loc >= starts[b]) & (loc < starts[b + 1])).all()
        # the local part of a bucket is the bucket's own optimised graph (first `local` columns), shifted
        own = oracle.optimize(oracle.knn_graph(data[starts[b]:starts[b + 1]], 2 * total), total)
        assert np.array_equal(loc, own[:, :local] + starts[b])
    rem = g[:, local:]
    assert (ts[rem] != ts[:, None]).mean() > 0.95  # remote slots point into other buckets (leftovers of the local phase aside)
    assert not (g == np.arange(n, dtype=np.uint32)[:, None]).any()


# ---- insert into the time-partitioned graph ----
def _py_partitioned_update(graph, ts, li, gi, n_old, target_ts, local):
    """fill_new_nodes_kernel_opt / generate_update_requests_kernel_opt / apply_topology_updates_kernel_opt
    (src/index/insert.cu:444-727), written from their description.  New rows: local slots = the nearest
    bucket-list entries of the row's own timestamp; remote slots = the nearest global-list entries of another
    timestamp that are not local already, topped up with whatever else the global list holds.  Old rows: every
    new row that lists them asks for a slot; per old row the first local/2 local and (total-local)/2 remote
    requests are served in (new row, slot) order."""
    g = graph.copy()
    n_new, total = li.shape[0], g.shape[1]
    n_total = n_old + n_new
    remote = total - local
    for t in range(n_new):
        me = n_old + t
        ok = lambda c: 0 <= c < n_total and c != me
        loc = [int(c) for c in li[t] if ok(c) and ts[c] == ts[me]][:local]
        first = [(k, int(c)) for k, c in enumerate(gi[t]) if ok(c) and c not in loc and ts[c] != ts[me]][:remote]
        taken = {k for k, _ in first}
        rest = [(k, int(c)) for k, c in enumerate(gi[t]) if ok(c) and k not in taken][:remote - len(first)]
        g[me] = 0xFFFFFFFF
        g[me, :len(loc)] = loc
        rem = [c for _, c in first] + [c for _, c in rest]
        g[me, local:local + len(rem)] = rem
    boxes = {}
    for t in range(n_new):
        for slot in range(total):
            dest = int(g[n_old + t, slot])
            if dest >= n_old:
                continue
            kind = 0 if slot < local else 1
            if kind == 1 and ts[dest] == target_ts:
                continue
            boxes.setdefault(dest, ([], []))[kind].append(n_old + t)
    for dest, (lreq, rreq) in boxes.items():
        rng = _py_wang(dest)
        for c in lreq[:local // 2]:
            rng = _py_wang(rng)
            strong = rng % 100 < 10
            start, length = (0, local // 2) if strong else (local // 2, local - local // 2)
            if length:
                rng = _py_wang(rng)
                g[dest, start + rng % length] = c
        for c in rreq[:remote // 2]:
            near = abs(int(ts[c]) - int(ts[dest])) <= 20
            start, length = (local, remote // 3) if near else (local + remote // 3, remote - remote // 3)
            if length:
                rng = _py_wang(rng)
                g[dest, start + rng % length] = c
    return g


@pytest.mark.parametrize("total,local,buckets,spread", [(8, 5, 4, 1), (12, 8, 6, 30), (6, 1, 3, 1), (9, 8, 5, 50)])
def test_partitioned_insert_update_matches_independent_restatement(oracle, total, local, buckets, spread):
    rng = np.random.default_rng(total * 31 + local)
    n_old, n_new, sk = 120, 9, 16
    ts = (rng.integers(0, buckets, n_old + n_new) * spread).astype(np.uint64)
    target = int(ts[n_old])
    ts[n_old:] = target
    ts[n_old + 3] = (target + spread) % (buckets * spread)  # a row of another bucket inside the batch
    graph = rng.integers(0, n_old, (n_old + n_new, total)).astype(np.uint32)
    same = np.flatnonzero(ts == target)
    li = np.stack([rng.permutation(same)[:sk] if len(same) >= sk else rng.choice(same, sk) for _ in range(n_new)]).astype(np.int64)
    gi = np.stack([rng.permutation(n_old)[:sk] for _ in range(n_new)]).astype(np.int64)
    li[rng.random(li.shape) < 0.1] = -1
    gi[rng.random(gi.shape) < 0.1] = -1
    li[2, :4] = rng.integers(0, n_old, 4)  # entries of other buckets in a bucket list are passed over
    got = oracle.insert_partitioned_update(graph, ts, li, gi, n_old, n_new, target, local)
    exp = _py_partitioned_update(graph, ts, li, gi, n_old, target, local)
    assert np.array_equal(got, exp)
    new = got[n_old:]
    loc = new[:, :local]
    filled = loc != 0xFFFFFFFF
    assert (ts[loc[filled]] == np.repeat(ts[n_old:, None], local, 1)[filled]).all()   # local slots: same timestamp
    assert not (new == np.arange(n_old, n_old + n_new, dtype=np.uint32)[:, None]).any()  # no self loops
    changed = (got[:n_old] != graph[:n_old])
    assert (got[:n_old][changed] >= n_old).all()                 # old rows only ever gain new rows
    assert changed[:, :local].sum(1).max() <= local // 2          # at most one slot per served request
    assert changed[:, local:].sum(1).max() <= (total - local) // 2


def test_partitioned_insert_merges_batch_neighbours_by_distance_then_id(oracle):
    rng = np.random.default_rng(5)
    n_old, n_new, dim, sk = 50, 12, 16, 10
    old = datasets.gaussian(n_old, dim, 1)
    new = datasets.gaussian(n_new, dim, 2)
    new[7] = new[3]  # an exact duplicate inside the batch: ties order by id
    ids, dists = oracle.bruteforce_topk(old, new, sk)
    ids[:, -2:] = -1  # a short bucket list
    tmp = min(n_new, sk // 2)
    got = oracle.merge_batch_neighbours(new, n_old, sk, ids, dists)
    bi, bd = oracle.bruteforce_topk(new, new, tmp)
    for i in range(n_new):
        cand_id = np.concatenate([ids[i, :-2], bi[i] + n_old])
        cand_d = np.concatenate([dists[i, :-2], bd[i]])
        order = np.lexsort((cand_id, cand_d))[:sk]
        exp = np.full(sk, -1, np.int64)
        exp[:len(order)] = cand_id[order]
        assert np.array_equal(got[i], exp)
        assert got[i, 0] == n_old + (3 if i == 7 else i)  # the row itself (or its lower-numbered twin) comes first
    assert (got >= 0).sum(1).min() == sk  # 8 old + 5 batch candidates always fill the 10 places


def test_partitioned_insert_batch_invariants(oracle):
    n_old, n_new, dim, total, local = 600, 20, 32, 16, 12
    data = datasets.gaussian(n_old + n_new, dim, 9)
    sizes = [150, 90, 200, 160]
    ts = np.concatenate([np.repeat(np.arange(4, dtype=np.uint64), sizes), np.full(n_new, 2, np.uint64)])
    g0 = oracle.build_time_partitioned(data[:n_old], ts[:n_old], sizes, total, local)
    graph = np.concatenate([g0, np.zeros((n_new, total), np.uint32)])
    bucket = np.flatnonzero(ts[:n_old] == 2).astype(np.uint32)
    seeds = np.tile(bucket[:32], (n_new, 1))
    g, state = oracle.insert_partitioned_batch(data, ts, n_old, n_new, 2, graph, local, seeds, 64, 4, 100, 12, 77)
    assert state != 77
    new = g[n_old:]
    loc = new[:, :local]
    assert (loc != 0xFFFFFFFF).all() and (ts[loc] == 2).all()
    rem = new[:, local:]
    assert (rem != 0xFFFFFFFF).all() and (ts[rem] != 2).mean() > 0.9
    # the local slots are close to the exact nearest rows of the bucket (old rows and batch rows alike)
    pool = np.concatenate([bucket, np.arange(n_old, n_old + n_new, dtype=np.uint32)])
    exact, _ = oracle.bruteforce_topk(data[pool], data[n_old:], local + 1)
    hits = sum(len(set(pool[exact[i]].tolist()) & set(loc[i].tolist())) for i in range(n_new))
    assert hits / (n_new * local) > 0.8
    # old rows: only new ids arrive, local requests in local slots of the same bucket, remote ones elsewhere
    changed = g[:n_old] != g0
    assert (g[:n_old][changed] >= n_old).all()
    assert (ts[:n_old][changed[:, :local].any(1)] == 2).all()
    assert (ts[:n_old][changed[:, local:].any(1)] != 2).all()
