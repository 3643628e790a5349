"""Pins the oracle's beam search (and the search inside its insert) against literal Python models of the
reference's kernels (tests/ref_literal.py): flat queue, whole-queue sort, flag bit, table rebuilt before
the sort every 30 iterations.  Inputs are integer-valued, so every summation order gives the same float
and the model's float64 distances equal the oracle's canonical float32 ones bit for bit; queries are
chosen so that no two rows are equally far away (the reference's tie order depends on its sort routine).
No GPU."""
import numpy as np
import pytest

import ref_literal as lit

DEFAULT_FIXES = lit.FIX_SEEDS | lit.FIX_RESTORE_ORDER | lit.FIX_EMPTY_SLOTS


def _int_rows(n, dim, seed, hi=512):
    return np.random.default_rng(seed).integers(0, hi, (n, dim)).astype(np.float32)


def _distinct_queries(data, dim, seed, want):
    """Queries whose distances to all rows are pairwise different."""
    out = []
    pool = _int_rows(20 * want, dim, seed)
    for q in pool:
        d = ((data.astype(np.float64) - q.astype(np.float64)) ** 2).sum(axis=1)
        assert d.max() < 2 ** 24
        if np.unique(d).size == d.size:
            out.append(q)
            if len(out) == want:
                return np.stack(out)
    raise AssertionError("not enough tie-free queries")


@pytest.fixture(scope="module")
def world(oracle):
    n, dim, deg = 420, 16, 16
    data = _int_rows(n, dim, 101)
    graph = oracle.optimize(oracle.knn_graph(data, 32), deg)
    graph[::37, 11:] = 0xFFFFFFFF            # some rows with empty slots
    q = _distinct_queries(data, dim, 102, 6)
    ts = np.random.default_rng(103).permutation(n).astype(np.uint64)  # timestamps in no particular order
    return data, graph, q, ts


def _compare(oracle, world, variant, fixes, flags, itopk, sw, max_iter, bitlen, n_seeds, seeds, mask, k=10,
             active_degree=None, window=None, expect_full=False):
    data, graph, q, ts = world
    kind = oracle.FILTER_RANGE if variant == "range" else oracle.FILTER_NONE
    ids, dist, ctr = oracle.search(data, graph, q, k, itopk, sw, max_iter, bitlen, n_seeds, mask,
                                   active_degree=active_degree, seeds=seeds, filter_kind=kind,
                                   ts=ts if variant == "range" else None, win=window, flags=flags)
    total = dict(iterations=0, rescored=0, full=0)
    for i in range(q.shape[0]):
        scored = []

        def dist_fn(a, b, scored=scored):
            scored.append(b.tobytes())
            return lit.l2_exact(a, b)

        eids, edist, ectr = lit.search_one(data, graph, q[i], k, itopk, sw, max_iter, bitlen, n_seeds,
                                           None if seeds is None else seeds[i], mask, variant=variant,
                                           active_degree=active_degree, ts=ts, window=window, fixes=fixes, dist=dist_fn)
        assert ids[i].tolist() == eids, (variant, fixes, i)
        assert np.array_equal(dist[i].view(np.uint32), edist.view(np.uint32)), (variant, fixes, i)
        # counters: iterations, S, P, F (the library reads a timestamp only for first-visit neighbours), D, table full
        assert ctr[i].tolist() == [ectr["iterations"], ectr["S"], ectr["P"], ectr["F_fresh"], ectr["D"], ectr["full"]], \
            (variant, fixes, i, ctr[i].tolist(), ectr)
        total["iterations"] = max(total["iterations"], ectr["iterations"])
        total["rescored"] += len(scored) - len(set(scored))
        total["full"] += ectr["full"]
    assert (total["full"] > 0) == expect_full
    return total


def test_literal_unfiltered_two_resets(oracle, world):
    # width 1, list of 96: at least 96 iterations, so the table is rebuilt at 30, 60 and 90; the rebuild
    # forgets every row that has left the list, and such rows are scored again (duplicates in the queue)
    t = _compare(oracle, world, "plain", 0, oracle.FLAG_STRICT, 96, 1, 120, 12, 24, None, 0x9E3779B9)
    assert t["iterations"] >= 90 and t["rescored"] > 0
    # the iteration limit cuts the search between two rebuilds
    _compare(oracle, world, "plain", 0, oracle.FLAG_STRICT, 96, 1, 71, 12, 24, None, 0x9E3779B9)
    # wider: 3 parents, capacity 256
    t = _compare(oracle, world, "plain", 0, oracle.FLAG_STRICT, 128, 3, 80, 12, 32, None, 12345)
    assert t["iterations"] >= 31


def test_literal_provided_seeds_duplicates_and_out_of_range(oracle, world):
    data = world[0]
    n = data.shape[0]
    rng = np.random.default_rng(5)
    seeds = rng.integers(0, n, (6, 20)).astype(np.uint32)
    seeds[:, 3] = seeds[:, 2]                 # duplicate: queued twice by the reference
    seeds[:, 7] = 0xFFFFFFFF                  # out of range: replaced by the formula id
    seeds[:, 9] = n + 5
    # 28 seeds asked, 20 provided: slots 20..27 take formula ids
    t = _compare(oracle, world, "plain", 0, oracle.FLAG_STRICT, 64, 2, 75, 11, 28, seeds, 0xABCDEF01)
    assert t["iterations"] >= 31
    _compare(oracle, world, "plain", DEFAULT_FIXES, 0, 64, 2, 75, 11, 28, seeds, 0xABCDEF01)


def test_literal_range_filter(oracle, world):
    data, graph, q, ts = world
    n = data.shape[0]
    window = (100, 330)
    inside = np.nonzero((ts >= window[0]) & (ts < window[1]))[0]
    rng = np.random.default_rng(6)
    seeds = rng.choice(inside, (6, 16)).astype(np.uint32)
    seeds[:, 5] = np.nonzero(ts < 50)[0][:6]  # seeds outside the window pass in the reference
    for sw, itopk, iters in ((1, 128, 140), (2, 160, 100)):
        t = _compare(oracle, world, "range", 0, oracle.FLAG_STRICT, itopk, sw, iters, 12, 16, seeds, 77, window=window)
        assert t["iterations"] >= 61 and t["rescored"] > 0
        _compare(oracle, world, "range", DEFAULT_FIXES, 0, itopk, sw, iters, 12, 16, seeds, 77, window=window)
        _compare(oracle, world, "range", DEFAULT_FIXES | lit.FILTER_FIRST, oracle.FLAG_FILTER_FIRST, itopk, sw, iters, 12,
                 16, seeds, 77, window=window)
        _compare(oracle, world, "range", lit.FILTER_FIRST, oracle.FLAG_STRICT | oracle.FLAG_FILTER_FIRST, itopk, sw,
                 iters, 12, 16, seeds, 77, window=window)
    # no seeds given: formula ids, in or out of the window
    _compare(oracle, world, "range", 0, oracle.FLAG_STRICT, 64, 1, 80, 12, 16, None, 0x51ED270B, window=window)
    # a window nothing falls into: the default mode answers -1, the reference the (out-of-window) seeds
    _compare(oracle, world, "range", DEFAULT_FIXES, 0, 64, 1, 80, 12, 16, seeds, 77, window=(n + 10, n + 20))
    _compare(oracle, world, "range", 0, oracle.FLAG_STRICT, 64, 1, 80, 12, 16, seeds, 77, window=(n + 10, n + 20))


def test_literal_active_degree(oracle, world):
    data = world[0]
    seeds = np.random.default_rng(8).integers(0, data.shape[0], (6, 32)).astype(np.uint32)
    for active in (5, 11, 16):
        t = _compare(oracle, world, "strided", 0, oracle.FLAG_STRICT, 128, 1, 140, 12, 32, seeds, 3, active_degree=active)
        assert t["iterations"] >= 91
        _compare(oracle, world, "strided", DEFAULT_FIXES, 0, 128, 1, 140, 12, 32, seeds, 3, active_degree=active)


def test_literal_small_table_rebuild_matters(oracle, world):
    # 512 slots for 420 rows: never full, but every rebuild forgets the rows that have left the list, and the
    # walk scores them again.  Both sides must agree on every one of them.
    t = _compare(oracle, world, "plain", 0, oracle.FLAG_STRICT, 64, 2, 100, 9, 16, None, 0x1234567)
    assert t["iterations"] >= 31 and t["rescored"] > 20
    t2 = _compare(oracle, world, "plain", DEFAULT_FIXES, 0, 64, 2, 100, 9, 16, None, 0x1234567)
    assert t2["rescored"] > 0
    # 256 and 128 slots fill before the first rebuild: every insert fails ("full" reads as "seen",
    # hashmap.cuh:89-90), the walk starves, and the rebuild at iteration 30 is what lets it go on.  Inserts of
    # an iteration are played in slot order on both sides.
    for bitlen in (8, 7):
        t = _compare(oracle, world, "plain", 0, oracle.FLAG_STRICT, 64, 2, 100, bitlen, 16, None, 0x1234567, expect_full=True)
        assert t["iterations"] >= 31
        _compare(oracle, world, "plain", DEFAULT_FIXES, 0, 64, 2, 100, bitlen, 16, None, 0x1234567, expect_full=True)


def test_default_mode_is_the_reference_plus_three_fixes(oracle, world):
    """Each documented departure changes something on this input, and only all three together give the
    default mode."""
    data, graph, q, ts = world
    n = data.shape[0]
    window = (100, 330)
    inside = np.nonzero((ts >= window[0]) & (ts < window[1]))[0]
    seeds = np.random.default_rng(9).choice(inside, (6, 12)).astype(np.uint32)
    seeds[:, 1] = seeds[:, 0]
    seeds[:, 4] = np.nonzero(ts >= 400)[0][:6]
    ids, dist, ctr = oracle.search(data, graph, q, 10, 64, 1, 100, 12, 12, 0, seeds=seeds, filter_kind=oracle.FILTER_RANGE,
                                   ts=ts, win=window)
    differs = {f: False for f in (0, lit.FIX_SEEDS, lit.FIX_RESTORE_ORDER)}  # one of the two fixes missing
    for i in range(q.shape[0]):
        for f in differs:
            _, _, c = lit.search_one(data, graph, q[i], 10, 64, 1, 100, 12, 12, seeds[i], 0, variant="range", ts=ts,
                                     window=window, fixes=f | lit.FIX_EMPTY_SLOTS)
            if [c["iterations"], c["S"], c["P"], c["F_fresh"], c["D"]] != ctr[i].tolist()[:5]:
                differs[f] = True
        e, ed, c = lit.search_one(data, graph, q[i], 10, 64, 1, 100, 12, 12, seeds[i], 0, variant="range", ts=ts,
                                  window=window, fixes=DEFAULT_FIXES)
        assert ids[i].tolist() == e and np.array_equal(dist[i], ed)
        assert [c["iterations"], c["S"], c["P"], c["F_fresh"], c["D"]] == ctr[i].tolist()[:5]
    assert all(differs.values()), differs
    # the third: an unfilled slot
    one = np.array([[int(inside[0])]], np.uint32)
    sid = oracle.search(data, graph, q[:1], 4, 64, 1, 0, 12, 1, 0, seeds=one, flags=oracle.FLAG_STRICT)[0]
    did = oracle.search(data, graph, q[:1], 4, 64, 1, 0, 12, 1, 0, seeds=one)[0]
    assert sid[0].tolist() == lit.search_one(data, graph, q[0], 4, 64, 1, 0, 12, 1, one[0], 0)[0] == \
        [int(inside[0]), 0x7FFFFFFF, 0x7FFFFFFF, 0x7FFFFFFF]
    assert did[0].tolist() == lit.search_one(data, graph, q[0], 4, 64, 1, 0, 12, 1, one[0], 0, fixes=DEFAULT_FIXES)[0] == \
        [int(inside[0]), -1, -1, -1]


@pytest.mark.parametrize("strict", [True, False])
def test_insert_against_literal_model(oracle, strict):
    """orc_insert_batch, search included, against the literal model: same new rows, same overwritten slots."""
    n0, n_new, deg, dim = 260, 70, 8, 16       # 70 new rows: two search groups, two masks
    old = _int_rows(n0, dim, 201)
    data = np.concatenate([old, _distinct_queries(old, dim, 202, n_new)])  # no new row equally far from two old rows
    graph = np.full((n0 + n_new, deg), 0xFFFFFFFF, np.uint32)
    graph[:n0] = oracle.optimize(oracle.knn_graph(data[:n0], 16), deg)
    state = 4242
    m0, s1 = oracle.splitmix64(state)
    m1, _ = oracle.splitmix64(s1)
    masks = [m0 & 0xFFFFFFFF, m1 & 0xFFFFFFFF]
    for striped in (1, 0):
        after, _ = oracle.insert_batch(data, n0, n_new, graph, 64, 2, 70, 9, state, striped_sort=striped,
                                       flags=oracle.FLAG_STRICT if strict else 0)
        exp = lit.insert_batch(data, n0, n_new, graph, 64, 2, 70, 9, masks, striped=bool(striped),
                               fixes=0 if strict else DEFAULT_FIXES)
        assert np.array_equal(after, exp), (strict, striped, np.nonzero((after != exp).any(axis=1))[0][:10])
        assert (after[:n0] != graph[:n0]).any()
