"""Device building blocks against their CPU models (wave sort, visited set, distance).

Mirrors the reference's own unit tests: tests/test_bitonic.cu, tests/test_sort_impl.cu,
tests/test_hashmap.cu.  Every call goes through the C ABI.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _fixtures():
    with open(os.path.join(HERE, "golden", "sort_fixtures.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("idx", range(7))
def test_sort_fixture(grab, idx):
    fx = _fixtures()[idx]
    keys = np.array(fx["key_bits"], np.uint32).view(np.float32)
    vals = np.arange(fx["n"], dtype=np.uint32)
    k, v = grab.sort_pairs(keys, vals)
    assert np.array_equal(k.view(np.uint32), np.array(fx["sorted_key_bits"], np.uint32))
    assert np.array_equal(v, np.array(fx["sorted_vals"], np.uint32))


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 100, 300, 777, 1024])
def test_sort_ragged_and_ties(grab, oracle, n):
    rng = np.random.default_rng(n)
    keys = rng.integers(0, 8, n).astype(np.float32)  # many equal keys: ties go to the lower value
    vals = rng.permutation(n).astype(np.uint32)
    k, v = grab.sort_pairs(keys, vals)
    ek, ev = oracle.sort_pairs(keys, vals)
    assert np.array_equal(k, ek) and np.array_equal(v, ev)


def test_sort_special_inputs(grab, oracle):
    for keys in (np.full(256, 5.0, np.float32), np.arange(256, 0, -1, dtype=np.float32),
                 np.arange(256, dtype=np.float32), np.r_[np.arange(100, dtype=np.float32), np.full(156, 3.40282e38, np.float32)],
                 -np.arange(256, dtype=np.float32)):
        vals = np.arange(keys.size, dtype=np.uint32)[::-1].copy()
        k, v = grab.sort_pairs(keys, vals)
        ek, ev = oracle.sort_pairs(keys, vals)
        assert np.array_equal(k, ek) and np.array_equal(v, ev)


@pytest.mark.parametrize("bitlen,n_unique,dup", [(10, 500, 0.4), (8, 200, 0.0), (8, 256, 0.0), (13, 6000, 0.5), (15, 20000, 0.1)])
def test_hash_reference_cases(grab, bitlen, n_unique, dup):
    # tests/test_hashmap.cu:171-187 plus two larger tables
    keys = np.r_[np.arange(1, n_unique + 1), np.arange(1, int(n_unique * dup) + 1)].astype(np.uint32)
    res, table = grab.hash_insert_many(bitlen, keys)
    assert int(res.sum()) == n_unique
    occupied = table[table != 0xFFFFFFFF]
    assert occupied.size == n_unique
    assert set(occupied.tolist()) == set(range(1, n_unique + 1))
    # every key sits on its probe path: between its home slot and its position there is no hole
    mask = (1 << bitlen) - 1
    pos = {int(k): i for i, k in enumerate(table) if k != 0xFFFFFFFF}
    for k, p in pos.items():
        h = (k ^ (k >> bitlen)) & mask
        j = h
        while j != p:
            assert table[j] != 0xFFFFFFFF
            j = (j + 1) & mask


def test_hash_full_table_rejects(grab):
    keys = np.arange(1, 300, dtype=np.uint32)  # 299 unique keys into 256 slots
    res, table = grab.hash_insert_many(8, keys)
    assert int(res.sum()) == 256
    assert (table != 0xFFFFFFFF).all()


@pytest.mark.parametrize("dim", [4, 32, 96, 128, 132, 256, 768, 960, 1024, 2048])
@pytest.mark.parametrize("metric", [0, 1])
def test_distance_bit_exact_vs_oracle(grab, oracle, dim, metric):
    rng = np.random.default_rng(dim + metric)
    data = rng.standard_normal((64, dim)).astype(np.float32)
    q = rng.standard_normal(dim).astype(np.float32)
    ids = rng.permutation(64).astype(np.uint32)
    got = grab.distance_many(q, data, ids, metric)
    exp = oracle.distance_many(q, data, ids, metric)
    assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))
    q64, d64 = q[None, :].astype(np.float64), data[ids].astype(np.float64)
    ref = ((q64 - d64) ** 2).sum(1) if metric == 0 else -(q64 * d64).sum(1)
    # 1e-5 relative to the magnitude of the summed terms (a dot product can cancel to ~0)
    scale = ((q64 - d64) ** 2).sum(1) if metric == 0 else np.abs(q64 * d64).sum(1)
    assert (np.abs(got - ref) <= 1e-5 * scale + 1e-12).all()


def test_distance_rejects_bad_dim(grab):
    with pytest.raises(grab.GrabError):
        grab.distance_many(np.zeros(6, np.float32), np.zeros((2, 6), np.float32), np.array([0], np.uint32))
