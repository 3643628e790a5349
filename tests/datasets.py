"""Seeded synthetic inputs shared by the tests and the benchmark.

Generators use numpy's PCG64 so that the same seed gives the same bytes everywhere.
"""
import numpy as np


def gaussian(n, dim, seed):
    """i.i.d. N(0,1) fp32 rows (the CPU-plumbing configuration)."""
    return np.random.default_rng(seed).standard_normal((n, dim), dtype=np.float32)


def mixture(n, dim, n_centroids, seed_centroids, seed_points, sigma=16.0):
    """Gaussian mixture: centroids U[0,128]^dim, point = round(clip(c + sigma*N(0,1), 0, 255)).

    Every value is an integer in [0,255], so squared L2 distances are exact in fp32
    whatever the summation order (dim*255^2 < 2^24 for dim <= 256)."""
    cent = np.random.default_rng(seed_centroids).uniform(0.0, 128.0, (n_centroids, dim)).astype(np.float32)
    rng = np.random.default_rng(seed_points)
    out = np.empty((n, dim), np.float32)
    step = 1 << 16
    for s in range(0, n, step):
        e = min(n, s + step)
        which = rng.integers(0, n_centroids, e - s)
        x = cent[which] + sigma * rng.standard_normal((e - s, dim), dtype=np.float32)
        out[s:e] = np.rint(np.clip(x, 0.0, 255.0))
    return out


def windows(n, nq, fraction, seed):
    """One contiguous timestamp window per query covering `fraction` of [0,n)."""
    w = max(1, int(round(n * fraction)))
    start = np.random.default_rng(seed).integers(0, n - w + 1, nq).astype(np.uint64)
    return start, start + np.uint64(w)


def unit_rows(n, dim, seed):
    x = gaussian(n, dim, seed)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    return x.astype(np.float32)


def zipf_labels(n, n_labels, s, seed):
    p = 1.0 / np.arange(1, n_labels + 1) ** s
    p /= p.sum()
    return np.random.default_rng(seed).choice(n_labels, size=n, p=p).astype(np.uint8)


def label_masks(nq, n_labels, seed):
    rng = np.random.default_rng(seed)
    masks = np.zeros(nq, np.uint64)
    for i in range(nq):
        cnt = rng.integers(1, 5)
        for b in rng.choice(n_labels, size=cnt, replace=False):
            masks[i] |= np.uint64(1) << np.uint64(b)
    return masks


def recall(ids, gt):
    """|result ∩ gt| / |gt valid| per the reference's drivers (tests/test_cagra_auto.cu:185-199)."""
    hit = tot = 0
    for r, g in zip(ids, gt):
        gs = set(int(x) for x in g if x >= 0)
        if not gs:
            continue
        hit += len(gs.intersection(int(x) for x in r if x >= 0))
        tot += len(gs)
    return hit / max(tot, 1)
