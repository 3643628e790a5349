"""kNN-graph build (MFMA contraction + exact re-score) and graph optimisation on the GPU
against the CPU restatement: ids are compared bit for bit."""
import numpy as np
import pytest

import datasets

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,dim,k,kind", [(3000, 128, 64, "gauss"), (5000, 128, 128, "mix"), (700, 96, 32, "gauss"),
                                          (1500, 256, 48, "gauss"), (130, 128, 16, "gauss"), (2000, 768, 32, "unit")])
def test_knn_graph_matches_oracle(oracle, grab, n, dim, k, kind):
    data = {"gauss": lambda: datasets.gaussian(n, dim, 7), "mix": lambda: datasets.mixture(n, dim, 12, 10, 11),
            "unit": lambda: datasets.unit_rows(n, dim, 20)}[kind]()
    metric = 1 if kind == "unit" else 0
    exp = oracle.knn_graph(data, k, metric)
    got, _ = grab.generate_knn_graph(grab.DeviceArray.from_numpy(data), n, dim, k, metric)
    got = got.numpy()
    bad = np.nonzero((exp != got).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} rows differ, first {bad[0]}: {exp[bad[0]][:8]} vs {got[bad[0]][:8]}"
    assert not (got == np.arange(n, dtype=np.uint32)[:, None]).any()  # no self loops


def test_knn_graph_points_on_a_line(grab):
    # recipe of the reference's tests/test_knn_build.cu:32-38,58-117 (N=10000, dim 1024, K=10):
    # vector i has every component equal to i*0.001, so the ideal neighbours are the nearest indices
    n, dim, k = 10000, 1024, 10
    data = np.repeat((np.arange(n, dtype=np.float32) * np.float32(0.001))[:, None], dim, axis=1)
    got = grab.generate_knn_graph(grab.DeviceArray.from_numpy(data), n, dim, k)[0].numpy()
    assert not (got == np.arange(n, dtype=np.uint32)[:, None]).any()
    hit = 0
    for i in range(0, n, 7):
        ideal = sorted(range(max(0, i - k), min(n, i + k + 1)), key=lambda j: (abs(j - i), j))[1:k + 1]
        hit += len(set(ideal) & set(got[i].tolist())) / k
    assert hit / len(range(0, n, 7)) > 0.99


def test_knn_graph_small_n_pads_with_invalid(oracle, grab):
    data = datasets.gaussian(20, 128, 3)
    got = grab.generate_knn_graph(grab.DeviceArray.from_numpy(data), 20, 128, 32)[0].numpy()
    assert np.array_equal(got, oracle.knn_graph(data, 32))
    assert (got[:, 19:] == 0xFFFFFFFF).all()


def test_bruteforce_topk_matches_oracle(oracle, grab):
    data = datasets.mixture(20000, 128, 20, 10, 11)
    q = datasets.mixture(300, 128, 20, 10, 12)
    ts = np.arange(20000, dtype=np.uint64)
    ws, we = datasets.windows(20000, 300, 0.1, 13)
    d_data, d_q = grab.DeviceArray.from_numpy(data), grab.DeviceArray.from_numpy(q)
    ids, dist, _ = grab.bruteforce_topk(d_data, 20000, 128, d_q, 300, 10)
    eids, edist = oracle.bruteforce_topk(data, q, 10)
    assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    ids, dist, _ = grab.bruteforce_topk(d_data, 20000, 128, d_q, 300, 10, filter_kind=1, d_ts=grab.DeviceArray.from_numpy(ts),
                                        d_win_start=grab.DeviceArray.from_numpy(ws), d_win_end=grab.DeviceArray.from_numpy(we))
    eids, edist = oracle.bruteforce_topk(data, q, 10, filter_kind=1, ts=ts, win_start=ws, win_end=we)
    assert np.array_equal(ids, eids) and np.array_equal(dist.view(np.uint32), edist.view(np.uint32))
    # a window smaller than k leaves -1 in the tail
    ids, dist, _ = grab.bruteforce_topk(d_data, 20000, 128, d_q, 300, 10, filter_kind=1, d_ts=grab.DeviceArray.from_numpy(ts), win=(5, 9))
    eids, edist = oracle.bruteforce_topk(data, q, 10, filter_kind=1, ts=ts, win=(5, 9))
    assert np.array_equal(ids, eids) and (ids[:, 4:] == -1).all()


def test_bruteforce_topk_mask_ip(oracle, grab):
    data = datasets.unit_rows(6000, 768, 20)
    labels = datasets.zipf_labels(6000, 64, 1.1, 21)
    q = datasets.unit_rows(64, 768, 22)
    masks = datasets.label_masks(64, 64, 23)
    ids, dist, _ = grab.bruteforce_topk(grab.DeviceArray.from_numpy(data), 6000, 768, grab.DeviceArray.from_numpy(q), 64, 10,
                                        metric=1, filter_kind=2, d_labels=grab.DeviceArray.from_numpy(labels),
                                        d_masks=grab.DeviceArray.from_numpy(masks))
    eids, edist = oracle.bruteforce_topk(data, q, 10, metric=1, filter_kind=2, labels=labels, masks=masks)
    assert np.array_equal(ids, eids)
    assert np.array_equal(dist.view(np.uint32), edist.view(np.uint32))


@pytest.mark.parametrize("n,kin,kout", [(3000, 64, 32), (2000, 128, 64), (300, 32, 32), (40, 64, 16)])
def test_optimize_steps_match_oracle(oracle, grab, n, kin, kout):
    data = datasets.gaussian(n, 64, n)
    knn = oracle.knn_graph(data, kin)  # n=40,kin=64 exercises 0xFFFFFFFF padding
    d_knn = grab.DeviceArray.from_numpy(knn)
    assert np.array_equal(grab.detour_counts(d_knn, n, kin).numpy(), oracle.detour_counts(knn))
    pruned = grab.optimize_prune(d_knn, n, kin, kout)
    epruned = oracle.prune(knn, kout)
    assert np.array_equal(pruned.numpy(), epruned)
    rev, cnt = grab.optimize_create_reverse_graph(pruned, n, kout)
    erev, ecnt = oracle.reverse_graph(epruned)
    assert np.array_equal(cnt.numpy(), ecnt)
    assert np.array_equal(rev.numpy(), erev)
    grab.optimize_merge_graphs(pruned, rev, cnt, n, kout)
    assert np.array_equal(pruned.numpy(), oracle.merge_graphs(epruned, erev, ecnt))
    full = grab.build_graph(None, n, d_knn, kin, kout).numpy()
    assert np.array_equal(full, oracle.optimize(knn, kout))


def test_prune_duplicate_ids_and_hubs(oracle, grab):
    # rows with repeated ids and one hub that everybody points to (long reverse segment)
    rng = np.random.default_rng(5)
    n, deg = 600, 32
    g = rng.integers(0, n, (n, deg)).astype(np.uint32)
    g[:, 0] = 7
    g[::3, 5] = g[::3, 4]
    d_g = grab.DeviceArray.from_numpy(g)
    assert np.array_equal(grab.detour_counts(d_g, n, deg).numpy(), oracle.detour_counts(g))
    rev, cnt = grab.optimize_create_reverse_graph(d_g, n, deg)
    erev, ecnt = oracle.reverse_graph(g)
    assert np.array_equal(cnt.numpy(), ecnt) and np.array_equal(rev.numpy(), erev)
    grab.optimize_merge_graphs(d_g, rev, cnt, n, deg)
    assert np.array_equal(d_g.numpy(), oracle.merge_graphs(g, erev, ecnt))


def test_prune_rejects_large_degree(grab):
    d = grab.DeviceArray((4, 600), np.uint32)
    with pytest.raises(grab.GrabError):  # the reference throws above 512 (src/index/cagra.cu:295-297)
        grab.optimize_prune(d, 4, 600, 64)


@pytest.mark.parametrize("n,dim,k,kind", [(20000, 64, 32, "gauss"), (17000, 128, 128, "mix"), (30000, 32, 64, "unit"),
                                          (16384, 96, 16, "dup"), (25001, 128, 100, "gauss"), (22000, 100, 24, "shifted"),
                                          (20000, 64, 32, "wide"), (6000, 128, 32, "gauss"), (4097, 40, 64, "mix"),
                                          (6000, 64, 16, "unit"), (17000, 256, 32, "gauss"), (16384, 768, 16, "unit"),
                                          (16500, 160, 24, "shifted"), (16400, 192, 16, "wide"), (16400, 384, 40, "unit"),
                                          (16400, 132, 16, "gauss"), (16390, 256, 20, "dup")])
def test_knn_graph_symmetric_pass_matches_oracle(oracle, grab, n, dim, k, kind):
    # from 16384 rows on - from 4096 where the pass can run on bf16 instructions: squared L2, up to 128 dimensions -
    # only the tiles on and above the diagonal are computed; a tile also serves the rows behind its columns.  Ties ("mix": integer data, "dup": every row twice), the inner product and a ragged last tile.
    # "shifted": rows far from the origin - the bounds of the pass are estimated from bf16 copies, which are centred
    # first so that eight bits of mantissa go to what differs between rows; uncentred, every estimate would be noise,
    # the bounds useless and every row redone.  "wide": coordinates whose scales span six decades - with squared L2 and
    # up to 128 dimensions the pass itself forms its products from two bf16 halves per value (16 of the 24 bits), which
    # the exact re-scoring and the check after it must make good.  The inner product and longer rows (whole chunks of
    # 32 dimensions) take the general kernel on rows split the same way, centred too where the metric is squared L2;
    # 132 dimensions is the case left to fp32 instructions.
    if kind == "gauss":
        data = datasets.gaussian(n, dim, 7)
    elif kind == "shifted":
        data = (datasets.gaussian(n, dim, 7) + np.float32(300.0)).astype(np.float32)
    elif kind == "wide":
        data = (datasets.gaussian(n, dim, 9) * np.logspace(-3.0, 3.0, dim, dtype=np.float32)).astype(np.float32)
    elif kind == "mix":
        data = datasets.mixture(n, dim, 12, 10, 11)
    elif kind == "unit":
        data = datasets.unit_rows(n, dim, 20)
    else:
        data = datasets.mixture(n, dim, 5, 10, 3)
        data[n // 2:] = data[:n - n // 2]
    metric = 1 if kind == "unit" else 0
    exp = oracle.knn_graph(data, k, metric)
    got, _ = grab.generate_knn_graph(grab.DeviceArray.from_numpy(data), n, dim, k, metric)
    flop, redone = grab.last_knn_stats()
    flop_bf16 = grab.last_knn_bf16_flop()
    got = got.numpy()
    bad = np.nonzero((exp != got).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} rows differ, first {bad[0]}: {exp[bad[0]][:8]} vs {got[bad[0]][:8]}"
    tiles = (n + 127) // 128
    # squared L2 up to 128 dimensions: the pass and its bounds run on bf16 instructions (three a product, rows padded to
    # 128 dimensions), the fp32 ones are left with the redone rows; otherwise the general kernel on split rows where
    # the rows are whole chunks of 32 dimensions - also below 16384 rows, where it computes all tiles (from 4096 rows)
    symmetric = n >= (4096 if metric == 0 and dim <= 128 else 16384)
    on_bf16 = (symmetric and metric == 0 and dim <= 128) or (dim % 32 == 0 and n >= 4096)
    assert (flop_bf16 > 0) == on_bf16
    if on_bf16:
        assert flop_bf16 >= 3.0 * 2.0 * 128 * 128 * (128 if metric == 0 and dim <= 128 else dim) * tiles * (tiles + 1) / 2
        if not (metric == 0 and dim <= 128):
            assert flop == 0       # bounding pass, symmetric pass and redone rows all ran on the split rows
    if kind in ("gauss", "unit", "shifted", "wide"):
        assert redone < 0.1 * n                                # the sample bounds nearly every row well
    if kind == "unit" and n >= 16384:
        # under the all-pairs count even here, where the bounding sample is a sixteenth of the rows (1/20 at a million)
        assert flop_bf16 / 3.0 < 0.9 * 2.0 * (tiles * 128) ** 2 * dim


def test_knn_graph_is_the_same_on_fp32_and_on_bf16_instructions(grab):
    # the process-wide switch: candidates from fp32 matrix instructions only; the graph does not notice
    n, dim, k = 40000, 128, 64
    data = datasets.mixture(n, dim, 40, 10, 5)
    d = grab.DeviceArray.from_numpy(data)
    a, _ = grab.generate_knn_graph(d, n, dim, k)
    assert grab.last_knn_bf16_flop() > 0
    assert grab.knn_allow_bf16(False) is True
    try:
        b, _ = grab.generate_knn_graph(d, n, dim, k)
        flop, _ = grab.last_knn_stats()
        assert grab.last_knn_bf16_flop() == 0 and flop > 2.0 * 128 * 128 * dim * (n // 128) ** 2 / 2
    finally:
        assert grab.knn_allow_bf16(True) is False
    assert np.array_equal(a.numpy(), b.numpy())


def test_knn_graph_symmetric_pass_redoes_rows_with_useless_bounds(oracle, grab):
    # The bounding sample is every (n / sample)-th row.  Here exactly those rows are far outliers, so a row's bound
    # (its distance to the 28th nearest sample row) admits every column: the lists overflow and every row must come
    # out of the plain pass - with the same neighbours.  A second set has a sample that looks nearer than the rest
    # is: the bounds admit too few keys.
    n, dim, k = 16384, 32, 16
    sample = n // 16
    spaced = (np.arange(sample, dtype=np.int64) * n // sample)
    for kind in ("far", "near"):
        data = datasets.gaussian(n, dim, 9)
        if kind == "far":
            data[spaced] *= 30.0          # scaled, not shifted: the distances among them stay well conditioned
        else:
            data[spaced] *= 0.05          # a tight ball at the origin: close to every row
            mask = np.ones(n, bool)
            mask[spaced] = False
            data[mask] += np.sign(data[mask]) * 3.0   # the other rows far from one another
        exp = oracle.knn_graph(data, k)
        got, _ = grab.generate_knn_graph(grab.DeviceArray.from_numpy(data), n, dim, k)
        _, redone = grab.last_knn_stats()
        assert np.array_equal(got.numpy(), exp), kind
        print(kind, "rows redone:", redone)
        assert redone > n // 4
        assert grab.last_knn_bf16_flop() > 0  # the pass whose bounds were useless ran on the bf16 instructions


@pytest.mark.parametrize("kind", ["offset", "near_duplicates", "offset_ip", "filtered_topk", "symmetric"])
def test_rows_the_candidates_cannot_prove_take_the_exact_pass(oracle, grab, kind):
    # Distances far below the rounding error of |a|^2+|b|^2-2ab: a large common offset with a tiny spread, or a swarm
    # of near-duplicates.  The candidate lists then hold arbitrary columns; the check after the exact scoring must
    # notice and the exact pass must give the oracle's graph bit for bit.  On well-conditioned data no row takes it.
    rng = np.random.default_rng(11)
    n, dim, k = 3000, 64, 48
    if kind == "symmetric":
        n = 17000  # from 16384 rows on only the tiles on and above the diagonal are computed
        k = 32
    if kind == "near_duplicates":
        # 2 swarms of rows that differ in the last bits: any slice of the columns holds more rows of a swarm (about 375)
        # than candidates are kept per slice (256)
        centers = rng.uniform(50.0, 60.0, (2, dim)).astype(np.float32)
        data = centers[rng.integers(0, 2, n)] + (rng.standard_normal((n, dim)) * 2e-5).astype(np.float32)
    else:
        data = (1000.0 + 0.01 * rng.standard_normal((n, dim))).astype(np.float32)
    d_data = grab.DeviceArray.from_numpy(data)
    if kind == "filtered_topk":
        nq = 200
        q = (1000.0 + 0.01 * rng.standard_normal((nq, dim))).astype(np.float32)
        ts = np.arange(n, dtype=np.uint64)
        ws, we = datasets.windows(n, nq, 0.3, 5)
        got, gd, _ = grab.bruteforce_topk(d_data, n, dim, grab.DeviceArray.from_numpy(q), nq, 10, filter_kind=grab.FILTER_RANGE,
                                          d_ts=grab.DeviceArray.from_numpy(ts), d_win_start=grab.DeviceArray.from_numpy(ws),
                                          d_win_end=grab.DeviceArray.from_numpy(we))
        exp, ed = oracle.bruteforce_topk(data, q, 10, filter_kind=oracle.FILTER_RANGE, ts=ts, win_start=ws, win_end=we)
        assert np.array_equal(got, exp) and np.array_equal(gd.view(np.uint32), ed.view(np.uint32))
        assert grab.last_knn_exact_rows() > 0
        return
    metric = 1 if kind == "offset_ip" else 0
    got = grab.generate_knn_graph(d_data, n, dim, k, metric)[0].numpy()
    redone = grab.last_knn_exact_rows()
    exp = oracle.knn_graph(data, k, metric)
    bad = np.nonzero((exp != got).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} rows differ, first {bad[0]}: {exp[bad[0]][:8]} vs {got[bad[0]][:8]}"
    assert redone > 0
    # the benchmark's kind of data: every row is proven by its candidates
    easy = datasets.mixture(4000, 128, 12, 10, 11)
    grab.generate_knn_graph(grab.DeviceArray.from_numpy(easy), 4000, 128, 64)
    assert grab.last_knn_exact_rows() == 0
