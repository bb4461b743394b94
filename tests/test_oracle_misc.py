"""Pins of the remaining oracle functions (no GPU): number formats, log2, the
superchunk statistics, Walsh-Hadamard, randDiag / bit-plane packing golden
vectors written from the reference's own torch code, the bit-width rule."""
import math
import os

import numpy as np
import pytest
import torch

from helpers import BF16, F16, F32, TORCH_DT, bits_to_f32, to_bits

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "srrcomp_golden.npz")


# ---- number formats ------------------------------------------------------------------------

def test_conversions_match_numpy_and_torch(oracle):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(50000) * np.exp(rng.uniform(-45, 45, 50000))).astype(np.float32)
    x[:8] = [0.0, -0.0, np.inf, -np.inf, 65519.99, 65520.0, 5.96e-8, 2.98e-8]
    with np.errstate(over="ignore"):
        assert (oracle.f32_to_f16(x) == x.astype(np.float16).view(np.uint16)).all()
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (oracle.f32_to_bf16(x) == want).all()
    xs = rng.uniform(-7e-5, 7e-5, 50000).astype(np.float32)          # half subnormals
    assert (oracle.f32_to_f16(xs) == xs.astype(np.float16).view(np.uint16)).all()
    allh = np.arange(65536, dtype=np.uint16)
    L = oracle.lib()
    got = np.array([L.dqo_f16_to_f32(int(h)) for h in allh[::7]], np.float32)
    want = allh[::7].view(np.float16).astype(np.float32)
    assert ((got == want) | (np.isnan(got) & np.isnan(want))).all()
    # ties to even
    assert oracle.f32_to_bf16(np.array([1.00390625, 1.01171875], np.float32)).tolist() == [0x3F80, 0x3F82]


def test_log2_accuracy_and_special_values(oracle):
    rng = np.random.default_rng(1)
    a = np.concatenate([np.exp(rng.uniform(-87, 88, 40000)), 1 + rng.uniform(0, 1e-3, 5000),
                        rng.uniform(0.5, 2.0, 20000), 2.0 ** np.arange(-126, 127)]).astype(np.float32)
    got = oracle.log2f(a).astype(np.float64)
    ref = np.log2(a.astype(np.float64))
    ulp = np.spacing(np.abs(ref).astype(np.float32)).astype(np.float64)
    assert (np.abs(got - ref) <= 1.75 * ulp).all()
    exact = oracle.log2f(np.array([1.0, 2.0, 0.5, 1024.0, 2.0 ** -130], np.float32))
    assert exact.tolist() == [0.0, 1.0, -1.0, 10.0, -130.0]
    sp = oracle.log2f(np.array([0.0, np.inf, -1.0, np.nan], np.float32))
    assert sp[0] == -np.inf and sp[1] == np.inf and np.isnan(sp[2]) and np.isnan(sp[3])


# ---- superchunk statistics -------------------------------------------------------------------

@pytest.mark.parametrize("dt", [F16, BF16, F32])
def test_mean_center_closed_forms(oracle, dt):
    tdt = TORCH_DT[dt]
    # constant block: residual 0, stats (c/W, 256 (c/W)^2)
    src = to_bits(torch.full((512,), 0.5).to(tdt))
    res, stats = oracle.superchunk_mean_center(src, 512, 4, dt)
    assert (bits_to_f32(res, dt) == 0).all()
    assert bits_to_f32(stats, BF16).tolist() == [0.125, 4.0, 0.125, 4.0]
    # ragged tail: mean over the valid elements only, padded residual is zero
    n = 256 + 10
    x = torch.arange(n, dtype=torch.float32).remainder(5).to(tdt)
    res, stats = oracle.superchunk_mean_center(to_bits(x), n, 1, dt)
    st = bits_to_f32(stats, BF16)
    tail = x[256:].float().numpy()
    assert st[2] == bits_to_f32(to_bits(torch.tensor([tail.mean()]).to(torch.bfloat16)), BF16)[0]
    assert st[3] == float((tail ** 2).sum())             # un-centred sum of squares
    assert (bits_to_f32(res, dt)[n:] == 0).all() and res.size == 512
    # tree order (stride 128 -> 1) == numpy pairwise halving in float32
    g = torch.Generator().manual_seed(2)
    y = (torch.randn(256, generator=g) * 3).to(tdt)
    v = (bits_to_f32(to_bits(y), dt) / np.float32(3.0)).astype(np.float32)
    s, q = v.copy(), (v * v).astype(np.float32)
    while s.size > 1:
        h = s.size // 2
        s = (s[:h] + s[h:]).astype(np.float32)
        q = (q[:h] + q[h:]).astype(np.float32)
    res, stats = oracle.superchunk_mean_center(to_bits(y), 256, 3, dt)
    mean = np.float32(s[0] / np.float32(256))
    assert stats[0] == to_bits(torch.tensor([mean]).to(torch.bfloat16))[0]
    assert stats[1] == to_bits(torch.tensor([q[0]]).to(torch.bfloat16))[0]
    want_res = to_bits(torch.from_numpy((v - mean).astype(np.float32)).to(tdt))
    assert (res == want_res).all()


def test_superchunk_stats_means(oracle):
    """the statistics-only variant: same stats as mean_center, and the unrounded binary32 means it reports are the ones
    the residual is formed with (numpy pairwise halving in float32; the ragged last superchunk divides by its length)"""
    g = torch.Generator().manual_seed(9)
    n, W = 256 * 3 + 50, 3
    x = (torch.randn(n, generator=g) * 1e-2 + 0.03).to(torch.bfloat16)
    res, stats = oracle.superchunk_mean_center(to_bits(x), n, W, BF16)
    stats2, means = oracle.superchunk_stats(to_bits(x), n, W, BF16)
    assert (stats == stats2).all() and means.dtype == np.float32 and means.size == 4
    v = (bits_to_f32(to_bits(x), BF16) / np.float32(W)).astype(np.float32)
    for b in range(4):
        blk = np.zeros(256, np.float32)
        valid = min(256, n - 256 * b)
        blk[:valid] = v[256 * b:256 * b + valid]
        s = blk.copy()
        while s.size > 1:
            h = s.size // 2
            s = (s[:h] + s[h:]).astype(np.float32)
        mean = np.float32(s[0] / np.float32(valid))
        assert means[b] == mean
        want = to_bits(torch.from_numpy((blk[:valid] - mean).astype(np.float32)).to(torch.bfloat16))
        assert (res[256 * b:256 * b + valid] == want).all()


def test_add_mean_restores_input(oracle):
    g = torch.Generator().manual_seed(4)
    n, W = 256 * 5 + 77, 8
    x = (torch.randn(n, generator=g) * 1e-2 + 0.02).to(torch.bfloat16)
    res, stats = oracle.superchunk_mean_center(to_bits(x), n, W, BF16)
    back = bits_to_f32(oracle.superchunk_add_mean_copy(res, stats, n, BF16), BF16)
    want = x.float().numpy() / W
    assert np.abs(back - want).max() <= 2 ** -7 * np.abs(want).max()


# ---- Walsh-Hadamard -------------------------------------------------------------------------------

def _sylvester(n):
    h = np.array([[1.0]])
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h


@pytest.mark.parametrize("n", [1, 2, 4, 16, 64, 256])
def test_fwht_equals_sylvester_matrix(oracle, n):
    rng = np.random.default_rng(n)
    x = rng.integers(-50, 50, n).astype(np.float32)          # integers: every sum is exact
    assert (oracle.fwht(x) == (_sylvester(n) @ x.astype(np.float64)).astype(np.float32)).all()


def test_fwht_identities(oracle):
    n = 1 << 12
    rng = np.random.default_rng(0)
    x = rng.integers(-8, 9, n).astype(np.float32)
    assert (oracle.fwht(oracle.fwht(x)) == n * x).all()
    ones = oracle.fwht(np.ones(n, np.float32))
    assert ones[0] == n and (ones[1:] == 0).all()
    e = np.zeros(n, np.float32)
    e[1234] = 1
    row = oracle.fwht(e)
    par = np.array([bin(i & 1234).count("1") & 1 for i in range(n)])
    assert (row == 1 - 2 * par).all()
    y = rng.standard_normal(n).astype(np.float32)
    ref = _sylvester(256) @ y[:256].astype(np.float64)
    assert np.abs(oracle.fwht(y[:256]) - ref).max() <= 1e-5 * np.abs(ref).max()


def test_fwht_against_reference_torch_butterfly():
    import oracle as O
    gold = np.load(GOLDEN)
    for k in (3, 6, 10):
        got = O.fwht(gold["had_in_%d" % k])
        ref = gold["had_out_%d" % k]
        assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()


def test_rht_blocked_is_diag_fwht_scale(oracle):
    rng = np.random.default_rng(5)
    n, B = 4096, 1024
    x = rng.standard_normal(n).astype(np.float32)
    s = rng.choice([-1.0, 1.0], n).astype(np.float32)
    sc = np.float32(1 / math.sqrt(B))
    fwd = oracle.rht_blocked(x, s, B, sc)
    for b in range(n // B):
        blk = slice(b * B, (b + 1) * B)
        assert (fwd[blk] == (oracle.fwht(x[blk] * s[blk]) * sc).astype(np.float32)).all()
    back = oracle.rht_blocked(fwd, s, B, sc, inverse=True)
    assert np.abs(back - x).max() <= 1e-5 * np.abs(x).max()


# ---- golden vectors from the reference's torch code -----------------------------------------------------

def test_rand_diag_golden(oracle):
    gold = np.load(GOLDEN)
    for size, seed in gold["randdiag_cases"]:
        size, seed = int(size), int(seed)
        want = np.unpackbits(gold["randdiag_%d_%d" % (size, seed)])[:size]
        got = (oracle.rand_diag(size, seed) > 0).astype(np.uint8)
        assert (got == want).all(), (size, seed)
    # roughly balanced signs
    s = oracle.rand_diag(1 << 16, 7)
    assert set(np.unique(s)) == {-1.0, 1.0} and abs(s.mean()) < 0.02


def test_bit_plane_packing_golden_and_roundtrip(oracle):
    gold = np.load(GOLDEN)
    for nbits in range(1, 9):
        for nbins in (64, 256):
            bins = gold["pack_bins_%d_%d" % (nbits, nbins)]
            bits = gold["pack_bits_%d_%d" % (nbits, nbins)]
            assert (oracle.bins_to_bits(bins, nbits).view(np.int32) == bits).all()
            assert (oracle.bits_to_bins(bits.view(np.uint32).copy(), nbits) == bins).all()
    rng = np.random.default_rng(3)
    for nbits in range(1, 9):
        bins = rng.integers(0, 1 << nbits, 32 * 37).astype(np.int32)
        arr = oracle.bins_to_bits(bins, nbits)
        # closed form: word w of plane p, bit t = bit p of bins[32 w + t]
        w, t, p = 11, 5, nbits - 1
        assert (arr[p * 37 + w] >> t) & 1 == (bins[32 * w + t] >> p) & 1
        assert (oracle.bits_to_bins(arr, nbits) == bins).all()


# ---- dynamic bit-width rule ------------------------------------------------------------------------------

def _torch_qbits(norms, u):
    """testbed_evaluation/new_comm_hooks/comm_hooks.py:64-70, torch ops on the tensor as given"""
    eps = 1e-20
    log_norms = torch.log2(torch.clamp(norms, min=eps))
    score = log_norms.mul(4.0 / (512.0 / 17.0)).add(float(u))
    z = torch.floor(torch.log2(torch.clamp(score, min=eps))).to(torch.int64)
    z.clamp_(1, 3)
    return torch.bitwise_left_shift(torch.ones_like(z), z)


def _torch_qbits_binary32_scalar(norms, u):
    """the same sequence with the scalar add done the way torch's device kernel does it: in binary32, rounded to the
    tensor's dtype afterwards"""
    eps = 1e-20
    ln = torch.log2(torch.clamp(norms, min=eps)).mul(4.0 / (512.0 / 17.0))
    score = (ln.float() + torch.tensor(float(u), dtype=torch.float32)).to(norms.dtype)
    z = torch.floor(torch.log2(torch.clamp(score, min=eps))).to(torch.int64)
    z.clamp_(1, 3)
    return torch.bitwise_left_shift(torch.ones_like(z), z)


def test_dynamic_bitrate_rule(oracle):
    g = torch.Generator().manual_seed(6)
    norms = torch.exp(torch.randn(20000, generator=g) * 6 - 8).to(torch.bfloat16)
    nb = to_bits(norms)
    assert (oracle.dynamic_bitrate_qbits(nb, 60.0) == 8).all()          # score >= 51 -> z clamps to 3
    assert (oracle.dynamic_bitrate_qbits(nb, -10.0) == 2).all()         # score < 0 -> eps -> z = 1
    prev = None
    for u in np.linspace(-10, 60, 71):
        q = oracle.dynamic_bitrate_qbits(nb, float(u))
        assert set(np.unique(q)) <= {2, 4, 8}
        if prev is not None:
            assert (q >= prev).all()                                   # monotone in u
        prev = q
        # torch's CPU kernel rounds the scalar u to bf16 before the add, its device kernel (what the reference runs, and
        # what the rule restates) adds it in binary32: the plain CPU sequence differs on a few norms per offset ...
        assert (q != _torch_qbits(norms, float(u)).numpy()).mean() < 1e-3
        # ... and with the add done in binary32 it agrees on every one
        assert (q == _torch_qbits_binary32_scalar(norms, float(u)).numpy()).all()
    # every finite non-negative bf16 norm, offsets off the bf16 grid
    pat = np.arange(0, 0x7f80, dtype=np.uint16)
    every = torch.from_numpy(pat.view(np.int16)).view(torch.bfloat16)
    for u in np.random.default_rng(0).uniform(-10, 60, 60):
        assert (oracle.dynamic_bitrate_qbits(pat, float(u)) == _torch_qbits_binary32_scalar(every, float(u)).numpy()).all()
    # norm 1 -> log2 = 0 -> score = bf16(u): 2 bits below 4, 4 bits in [4, 8), 8 bits from 8 on;
    # bf16(7.97) = 7.96875 has log2 = 2.9943, which ROUNDS to 3.0 in bf16 and therefore already gets 8 bits
    one = to_bits(torch.tensor([1.0]).to(torch.bfloat16))
    us = (3.98, 4.0, 7.9, 7.97, 8.0)
    assert [int(oracle.dynamic_bitrate_qbits(one, u)[0]) for u in us] == [2, 4, 4, 8, 8]
    assert [int(_torch_qbits(torch.tensor([1.0]).to(torch.bfloat16), u)[0]) for u in us] == [2, 4, 4, 8, 8]


def test_offset_search_closed_forms_and_torch_sequence(oracle, monkeypatch):
    """the oracle's two searches for u: cases that can be followed by hand, and the package's torch restatement of
    comm_hooks.py:94-139 run on the CPU with the scalar add done in binary32 (what the device kernel of torch does;
    torch's CPU kernel rounds the scalar u to bf16 first, which is not what the reference's GPU run computes)"""
    ones = [to_bits(torch.ones(1000).to(torch.bfloat16))]
    # all norms 1.0: width 2 below u = 4, 4 up to bf16(u) = 7.9375, 8 from 7.96875 on.  Probes 60, 25, 7.5:
    assert oracle.dynamic_bitrate_binary_search_u(ones, 4.0) == (7.5, 4.0, 0.0)
    # 3 bits cannot be met: the first probe at distance 1 (u = 7.5) stays the best of 33
    assert oracle.dynamic_bitrate_binary_search_u(ones, 3.0) == (7.5, 4.0, -1.0)
    assert oracle.dynamic_bitrate_adjust_u(ones, 60.0, 4.0) == (56.0, 8.0, -4.0)     # deficit keeps its sign: returned
    assert oracle.dynamic_bitrate_adjust_u(ones, 7.0, 4.0) == (7.0, 4.0, 0.0)
    assert oracle.dynamic_bitrate_adjust_u(ones, 100.0, 8.0) == (60.0, 8.0, 0.0)     # prev_u is clipped to [-10, 60]
    assert oracle.dynamic_bitrate_binary_search_u([], 4.375) == (60.0, 0.0, 4.375)

    from dynamiq_sigcomm_artifact_amd import bitrate as B

    monkeypatch.setattr(B, "dynamic_bitrate_qbits", _torch_qbits_binary32_scalar)
    g = torch.Generator().manual_seed(0)
    for trial in range(4):
        norms = [torch.exp(torch.randn(5000 + 17 * trial, generator=g) * (1 + trial) - 6 - trial).to(torch.bfloat16)
                 for _ in range(3)]
        nb = [to_bits(t) for t in norms]
        for target in (1.375, 3.375, 4.375, 7.375):
            a = B.dynamic_bitrate_binary_search_u(norms, target)
            assert a == tuple(oracle.dynamic_bitrate_binary_search_u(nb, target))
            for prev in (a[0], a[0] + 6, a[0] - 3, 60.0, -10.0):
                assert B.dynamic_bitrate_adjust_u(norms, prev, target) == tuple(oracle.dynamic_bitrate_adjust_u(nb, prev, target))


def test_bit_width_rule_non_finite_norms(oracle):
    """the device conversion to int64 saturates: +inf norms land in the 8-bit group, NaN norms in the 2-bit group"""
    import numpy as np
    from helpers import to_bits
    import torch
    norms = torch.tensor([float("inf"), float("nan"), 0.0, -1.0, 1e-30], dtype=torch.bfloat16)
    assert oracle.dynamic_bitrate_qbits(to_bits(norms), 60.0).tolist() == [8, 2, 8, 8, 8]
    assert oracle.dynamic_bitrate_qbits(to_bits(norms), -10.0).tolist() == [8, 2, 2, 2, 2]


def test_philox_known_answers(oracle):
    """Philox4x32-10 known-answer vectors published with Random123 (kat_vectors: zeros, all ones, digits of pi)"""
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
        ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
        ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
         [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    ]
    for ctr, key, want in kat:
        assert oracle.philox4x32_10(ctr, key).tolist() == want
    # the stream of the rounding mode: element e = byte e % 16 of block (chunk e / 16, step), key = seed
    import numpy as np
    seed, step = 0x299f31d0a4093822, 0x0370734413198a2e
    u = oracle.philox_uniform(40, seed, step)
    for chunk in (0, 1, 2):
        w = oracle.philox4x32_10([chunk, 0, step & 0xffffffff, step >> 32], [seed & 0xffffffff, seed >> 32])
        want = (np.frombuffer(w.astype("<u4").tobytes(), np.uint8) | 1).astype(np.float32) / 256
        got = u[16 * chunk: 16 * chunk + 16]
        assert (got == want[:got.size]).all()


# ---- quantization_compression (cuda_hadamard.cu:607-627) ------------------------------------------------

def test_quantization_oracle_closed_forms(oracle):
    """integers stay, values land on floor or floor + 1 of the clamped quotient, the direction is decided by the
    Philox word the documentation names (re-derived here from the known-answer-pinned block function)"""
    n, seed = 1003, 0x1234567890ABCDEF
    rng = np.random.default_rng(5)
    v = (rng.random(n, dtype=np.float32) * 30.0 - 15.0).astype(np.float32)
    v[:8] = [0.0, 1.0, -1.0, 2.5, -2.5, 1e9, -1e9, 0.5]
    div, tmax = np.float32(0.5), np.float32(10.0)
    got = oracle.quantization(v, div, tmax, seed)
    t = np.clip((v / div).astype(np.float32), -tmax, tmax)
    fl = np.floor(t)
    u = np.zeros(n, np.float32)
    for g in range((n + 3) // 4):
        w = oracle.philox4x32_10([g & 0xffffffff, g >> 32, 0, 0], [seed & 0xffffffff, seed >> 32])
        for k in range(min(4, n - 4 * g)):
            u[4 * g + k] = np.float32(int(w[k]) >> 8) * np.float32(2.0 ** -24)
    want = fl + (u < (t - fl)).astype(np.float32)
    assert (got == want).all()
    assert got[0] == 0.0 and got[1] == 2.0 and got[2] == -2.0 and got[3] == 5.0 and got[4] == -5.0
    assert got[5] == 10.0 and got[6] == -10.0 and got[7] == 1.0            # clamped, and exact quotients never move
    # unbiased: the mean rounding error vanishes
    big = (rng.random(1 << 18, dtype=np.float32) * 8.0 - 4.0).astype(np.float32)
    q = oracle.quantization(big, np.float32(0.37), np.float32(100.0), 7)
    assert abs(float((q - big / np.float32(0.37)).mean())) < 5e-3
    assert not (oracle.quantization(big, 0.37, 100.0, 8) == q).all()
