"""The error bounds that the library's checks rest on where inner products are formed from bf16 halves
(grab-anns_amd/csrc/topk_gemm.hip: sym_split_kernel and refine_kernel's check; csrc/entry_probe.hip: centroid ranking).

A value x is stored as hi = bf16(x) and lo = bf16(x - hi), round to nearest even; a product q.c is taken as
q_lo.c_hi + q_hi.c_lo + q_hi.c_hi.  bf16 keeps 8 significant bits, so |x - hi| <= 2^-8 |x| and what the two halves
leave is at most 2^-16 |x|; the three things a product then lacks (q_lo.c_lo and the two remainders against the other
vector) are at most 2^-16 |q||c| each.  The check after the exact re-scoring allows 3 * 2^-16 |q||c|; the norms ride
along as three bf16 pieces of -|x|^2/2, which must give the fp32 value back.  The arithmetic is restated here in numpy
(integer bit operations, float64 sums) and the bounds are tested on random and on unfriendly vectors."""
import numpy as np
import pytest


def bf16_rne(x):
    """float32 -> float32 holding the nearest bf16 (ties to even), by the bit rule of the kernels"""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


def split(x):
    hi = bf16_rne(x)
    lo = bf16_rne((np.asarray(x, np.float32) - hi).astype(np.float32))
    return hi, lo


def vectors(kind, n, dim, rng):
    if kind == "gauss":
        return rng.standard_normal((n, dim)).astype(np.float32)
    if kind == "decades":
        return (rng.standard_normal((n, dim)) * np.logspace(-3, 3, dim)).astype(np.float32)
    if kind == "same_sign":  # no cancellation to hide behind: every product positive
        return np.abs(rng.standard_normal((n, dim))).astype(np.float32) + np.float32(1.0)
    if kind == "just_above_a_tie":  # mantissas that sit next to a rounding boundary of bf16
        base = np.float32(1.0) + np.float32(2.0 ** -8) + np.float32(2.0 ** -23)
        return (base * (2.0 ** rng.integers(-4, 5, (n, dim)))).astype(np.float32) * rng.choice(np.float32([-1, 1]), (n, dim))
    raise ValueError(kind)


@pytest.mark.parametrize("kind", ["gauss", "decades", "same_sign", "just_above_a_tie"])
def test_a_value_is_its_two_halves_to_2_to_the_minus_16(kind):
    x = vectors(kind, 64, 128, np.random.default_rng(1)).ravel()
    hi, lo = split(x)
    # x - hi is exact in fp32 (hi is x's leading bits), so lo is the rounding of the true remainder
    assert np.array_equal((x.astype(np.float64) - hi.astype(np.float64)).astype(np.float32).astype(np.float64),
                          x.astype(np.float64) - hi.astype(np.float64))
    left = np.abs(x.astype(np.float64) - hi.astype(np.float64) - lo.astype(np.float64))
    assert np.all(left <= 2.0 ** -16 * np.abs(x.astype(np.float64)))
    assert np.all(np.abs(lo.astype(np.float64)) <= 2.0 ** -8 * (1 + 2.0 ** -8) * np.abs(x.astype(np.float64)))
    if kind == "just_above_a_tie":  # the bound on the first half is reached to within a factor of two there
        assert np.max(np.abs(x.astype(np.float64) - hi.astype(np.float64)) / np.abs(x.astype(np.float64))) > 2.0 ** -9


@pytest.mark.parametrize("kind", ["gauss", "decades", "same_sign", "just_above_a_tie"])
def test_three_products_are_within_3_times_2_to_the_minus_16_of_the_inner_product(kind):
    rng = np.random.default_rng(2)
    q, c = vectors(kind, 200, 128, rng), vectors(kind, 200, 128, rng)
    qh, ql = (a.astype(np.float64) for a in split(q))
    ch, cl = (a.astype(np.float64) for a in split(c))
    approx = (ql * ch).sum(1) + (qh * cl).sum(1) + (qh * ch).sum(1)
    exact = (q.astype(np.float64) * c.astype(np.float64)).sum(1)
    nq, nc = np.sqrt((q.astype(np.float64) ** 2).sum(1)), np.sqrt((c.astype(np.float64) ** 2).sum(1))
    err = np.abs(approx - exact)
    assert np.all(err <= 3.0 * 2.0 ** -16 * nq * nc)
    # dropping a cross term would not pass: the test can tell the formula from a wrong one
    wrong = (qh * cl).sum(1) + (qh * ch).sum(1)
    if kind in ("same_sign", "just_above_a_tie"):
        assert np.any(np.abs(wrong - exact) > 3.0 * 2.0 ** -16 * nq * nc)


def test_three_pieces_give_the_norm_term_back():
    # h = -|x|^2 / 2 as h0 + h1 + h2, each a bf16 of what the ones before left: all 24 bits of the fp32 value
    rng = np.random.default_rng(3)
    h = (-0.5 * (rng.standard_normal(100000) * np.logspace(-6, 6, 100000)) ** 2).astype(np.float32)
    h0 = bf16_rne(h)
    r1 = (h - h0).astype(np.float32)
    h1 = bf16_rne(r1)
    h2 = bf16_rne((r1 - h1).astype(np.float32))
    back = h0.astype(np.float64) + h1.astype(np.float64) + h2.astype(np.float64)
    assert np.all(np.abs(back - h.astype(np.float64)) <= 2.0 ** -25 * np.abs(h.astype(np.float64)))
    assert np.mean(back == h.astype(np.float64)) > 0.9


def test_distance_from_the_extended_vectors():
    # row . column of the extended vectors = q.c - |q|^2/2 - |c|^2/2 = -d/2: the layout of the 16 extra values
    rng = np.random.default_rng(4)
    q, c = rng.standard_normal(128).astype(np.float32), rng.standard_normal(128).astype(np.float32)

    def pieces(x):
        h = np.float32(-0.5) * np.float32((x.astype(np.float64) ** 2).sum())
        h0 = bf16_rne(h)
        r1 = np.float32(h - h0)
        h1 = bf16_rne(r1)
        return [float(h0), float(h1), float(bf16_rne(np.float32(r1 - h1)))]

    as_row = pieces(q) + [1.0, 1.0, 1.0, 0.0, 0.0]
    as_col = [1.0, 1.0, 1.0] + pieces(c) + [0.0, 0.0]
    g = float(q.astype(np.float64) @ c.astype(np.float64)) + float(np.dot(as_row, as_col))
    d = float(((q.astype(np.float64) - c.astype(np.float64)) ** 2).sum())
    assert abs(-2.0 * g - d) <= 2.0 ** -22 * d
