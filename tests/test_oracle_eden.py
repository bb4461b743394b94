"""The EDEN / THC restatements of the oracle against the reference's own outputs
(tests/golden/eden_golden.npz, written by the reference's CPU code) and against what the
mathematics fixes.  Tolerances: the reference reduces and transforms with torch's CPU kernels
(unspecified summation order, butterfly written as (a+b)-2b), so bins may differ where a
rotated coordinate lies within rounding error of a boundary (<= 0.2 % of the coordinates
here; each such flip also moves `scale` a little) and `scale` agrees to 1e-4 relative."""
import math
import os

import numpy as np
import pytest

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "eden_golden.npz"))


def _oracle_slice(oracle, x, nbits, seed, num_hadamard):
    """srrcomp.py:293-326 with oracle calls; returns bins, scale"""
    n = x.size
    if n & (n - 1) or n < 32:
        p = max(1 << int(math.ceil(math.log2(n))), 32)
        x = np.concatenate([x, np.zeros(p - n, np.float32)])
        n = p
    inv = np.float32(1.0) / np.float32(math.sqrt(n))
    v = x.astype(np.float32).copy()
    for i in range(num_hadamard):
        v = oracle.rht_blocked(v, oracle.rand_diag(n, seed + i), n, inv)
    bins, result = oracle.eden_quantize(v, GOLD["boundaries_%d" % nbits], GOLD["centroids_%d" % nbits], nbits)
    return bins, result, v


def _slices(dim):
    """the reference's slicing rule (srrcomp.py:262-291) for max_padding_overhead = 0.1"""
    out, remaining, cur = [], dim, 0
    hi = lambda n: 2 ** int(np.ceil(np.log2(n)))
    lo = lambda n: 2 ** int(np.log2(n))
    while (hi(remaining) - remaining) / dim > 0.1:
        low = lo(remaining)
        out.append((cur, low, 1 + (low < 1024)))
        cur += low
        remaining -= low
    out.append((cur, dim - cur, 1 + (dim - cur < 1024)))
    return out


@pytest.mark.parametrize("case", [tuple(c) for c in GOLD["cases"]])
def test_oracle_eden_chain_against_reference_outputs(oracle, case):
    dim, nbits, seed, nslices = (int(v) for v in case)
    x = GOLD["x_%d" % dim]
    sl = _slices(dim)
    assert len(sl) == nslices
    key = "%d_%d_%d" % (dim, nbits, seed)
    for k, (start, length, nh) in enumerate(sl):
        scale_g, orig_g, nh_g = GOLD["meta_%s_%d" % (key, k)]
        assert (int(orig_g), int(nh_g)) == (length, nh)
        bins, result, _ = _oracle_slice(oracle, x[start:start + length], nbits, seed, nh)
        bins_g = oracle.bits_to_bins(GOLD["packed_%s_%d" % (key, k)].view(np.uint32), nbits)
        assert bins.size == bins_g.size
        diff = bins != bins_g
        assert diff.mean() <= 2e-3 and (np.abs(bins - bins_g) <= 1).all()
        assert abs(result[2] - scale_g) <= 1e-4 * abs(scale_g)


def test_eden_quantize_closed_forms(oracle):
    b1, c1 = GOLD["boundaries_1"], GOLD["centroids_1"]
    # one bit: bin = (x > 0); scale = ||x||^2 / (c * sum |x|); for x = +-a: scale = a / c
    x = np.array([0.5, -0.5] * 32, np.float32)
    bins, res = oracle.eden_quantize(x, b1, c1, 1)
    assert (bins == np.array([1, 0] * 32)).all()
    assert res[0] == 16.0 and res[3] == 4.0 and abs(res[2] - 0.5 / c1[1]) < 1e-6
    # right=False: a value exactly on a boundary belongs to the lower bin
    b2, c2 = GOLD["boundaries_2"], GOLD["centroids_2"]
    n = 64
    x = np.full(n, 1.0, np.float32)          # normalised coordinates are all exactly 1
    bnd = np.array([-1.0, 1.0, 2.0], np.float32)
    bins, _ = oracle.eden_quantize(x, bnd, c2, 2)
    assert (bins == 1).all()
    bins, _ = oracle.eden_quantize(x, np.array([-1.0, np.nextafter(np.float32(1), np.float32(0)), 2.0], np.float32), c2, 2)
    assert (bins == 2).all()
    # the documented summation order equals an exact (math.fsum) sum to double rounding
    g = np.random.default_rng(3)
    v = (g.standard_normal(10000 // 32 * 32) * 1e-3).astype(np.float32)
    _, res = oracle.eden_quantize(v, GOLD["boundaries_4"], GOLD["centroids_4"], 4)
    assert res[0] == np.float32(math.fsum(float(t) ** 2 for t in v))
    assert (oracle.eden_dequantize(np.arange(16, dtype=np.int32), GOLD["centroids_4"]) == GOLD["centroids_4"]).all()


def test_lloyd_max_tables_against_reference_literals():
    """own tables: stationary to 1e-12, optimal (never worse distortion than the reference's literals), and within the
    literals' own inaccuracy of them"""
    from scipy.stats import norm
    from scipy import integrate
    from dynamiq_sigcomm_artifact_amd import eden

    def distortion(c):
        b = np.concatenate(([-np.inf], (c[:-1] + c[1:]) / 2, [np.inf]))
        # E[(X - c_i)^2; b_i < X < b_i+1] in closed form
        pdf, cdf = norm.pdf, norm.cdf
        lo, hi = b[:-1], b[1:]
        m0 = cdf(hi) - cdf(lo)
        m1 = pdf(lo) - pdf(hi)
        lo_t = np.where(np.isinf(lo), 0.0, lo) * pdf(lo)
        hi_t = np.where(np.isinf(hi), 0.0, hi) * pdf(hi)
        m2 = m0 + lo_t - hi_t
        return float(np.sum(m2 - 2 * c * m1 + c * c * m0))

    tol = {1: 1e-7, 2: 1e-7, 3: 2e-7, 4: 1e-6, 5: 1e-5, 6: 5e-5, 7: 2e-4, 8: 2e-3}
    for nbits in range(1, 9):
        c = eden.lloyd_max_normal(nbits)
        assert np.max(np.abs(c - eden._conditional_means(c))) < 1e-12
        assert np.allclose(c, -c[::-1])
        ref = GOLD["centroids_%d" % nbits].astype(np.float64)
        assert np.max(np.abs(c - ref)) < tol[nbits]
        assert distortion(c) <= distortion(ref) + 1e-15
    assert abs(eden.lloyd_max_normal(1)[1] - math.sqrt(2 / math.pi)) < 1e-15


def test_thc_oracle_closed_forms(oracle):
    lo, delta, levels = -1.0, 2.0 / 63, 64
    v = np.array([-2.0, -1.0, 1.0, 5.0, -1.0 + 10.25 * delta, np.nan], np.float32)
    u0 = np.zeros(6, np.float32)
    u1 = np.full(6, 0.999, np.float32)
    from helpers import bits_to_f32, BF16
    got0 = bits_to_f32(oracle.thc_quantize(v, u0, lo, delta, levels), BF16)
    got1 = bits_to_f32(oracle.thc_quantize(v, u1, lo, delta, levels), BF16)
    assert got0[:4].tolist() == [0.0, 0.0, 63.0, 63.0] and got1[:4].tolist() == [0.0, 0.0, 63.0, 63.0]
    assert got0[4] == 11.0 and got1[4] == 10.0 and np.isnan(got0[5])
    # unbiased: E[level] = x
    g = np.random.default_rng(1)
    x = np.full(200000, -1.0 + 17.3 * delta, np.float32)
    lev = bits_to_f32(oracle.thc_quantize(x, g.random(x.size, dtype=np.float32), lo, delta, levels), BF16)
    assert abs(lev.mean() - 17.3) < 0.01
    back = oracle.thc_dequantize(oracle.thc_quantize(v[:4], u0[:4], lo, delta, levels), np.float32(delta), np.float32(lo))
    assert np.allclose(back, [-1, -1, 1, 1], atol=1e-6)


def test_nan_goes_to_the_last_bin_like_torch_bucketize(oracle):
    """an all-zero slice: 0/0 = NaN for every element; torch.bucketize(right=False) is a lower-bound search whose
    comparison `!(boundary >= x)` holds for NaN at every step, so every bin is the last one"""
    import torch
    bnd = np.array([-1.0, 0.0, 1.0], np.float32)
    cen = np.array([-1.5, -0.5, 0.5, 1.5], np.float32)
    bins, res = oracle.eden_quantize(np.zeros(64, np.float32), bnd, cen, 2)
    want = torch.bucketize(torch.full((64,), float("nan")), torch.from_numpy(bnd)).numpy()
    assert (bins == want).all() and (bins == 3).all()
    x = np.array([-2.0, -1.0, -0.5, 0.0, 0.5, 1.0, 2.0, np.nan] * 4, np.float32)
    got = np.array([sum(1 for b in bnd if not (b >= v)) for v in x])
    assert (got == torch.bucketize(torch.from_numpy(x), torch.from_numpy(bnd)).numpy()).all()
