"""The torch-CPU restatements that bench.py times as the CPU baseline compute what they claim: the diagonal and the
bit planes equal the reference's own outputs (tests/golden/srrcomp_golden.npz), the butterfly is the Hadamard
transform, and the hierarchical quantiser's round trip equals the oracle's decompress(compress(x))."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
import cpu_baselines as B          # noqa: E402

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "srrcomp_golden.npz"))
EDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "eden_golden.npz"))


def test_rand_diag_matches_reference_outputs():
    for size, seed in GOLD["randdiag_cases"]:
        want = np.unpackbits(GOLD["randdiag_%d_%d" % (size, seed)])[:size]
        got = (B.rand_diag(int(size), int(seed)).numpy() > 0).astype(np.uint8)
        assert (got == want).all(), (size, seed)


def test_bit_planes_match_reference_outputs():
    for nbits in range(1, 9):
        for nbins in (64, 256):
            bins = torch.from_numpy(GOLD["pack_bins_%d_%d" % (nbits, nbins)])
            bits = B.bins_to_bits(bins.clone(), nbits)
            assert (bits.numpy() == GOLD["pack_bits_%d_%d" % (nbits, nbins)]).all()
            assert torch.equal(B.bits_to_bins(bits, nbits).to(torch.int32), bins)


def test_hadamard_is_the_sylvester_transform():
    x = torch.arange(64, dtype=torch.float32) - 20.0
    H = torch.tensor([[1.0]])
    while H.shape[0] < 64:
        H = torch.cat((torch.cat((H, H), 1), torch.cat((H, -H), 1)), 0)
    assert torch.equal(B.hadamard(x.clone()), H @ x)


@pytest.mark.parametrize("nbits", [4, 8])
def test_hier_roundtrip_equals_oracle(oracle, nbits):
    g = torch.Generator().manual_seed(nbits)
    n = 256 * 50
    x = torch.randn(n, generator=g) * torch.exp(torch.randn(n // 256, 1, generator=g) * 2 - 6).repeat_interleave(256, 0).reshape(-1)
    r = torch.rand(n, generator=g)
    got = B.hier_roundtrip(x, r, nbits).numpy()
    enc = oracle.scaling_compress(x.numpy(), r.numpy(), n, nbits, 16, 2, oracle.F32)
    dec = np.zeros(n, np.float32)
    oracle.scaling_decompress(enc, dec, n, nbits, 16, 2, oracle.F32)
    assert (got == dec).all()


def test_rht_roundtrip_reconstructs():
    nbits = 4
    cen, bnd = torch.from_numpy(EDEN["centroids_4"]), torch.from_numpy(EDEN["boundaries_4"])
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4096, generator=g) * 1e-3
    rec = B.rht_roundtrip(x.clone(), nbits, 17, cen, bnd)
    nmse = float(((rec - x) ** 2).sum() / (x ** 2).sum())
    assert 0.005 < nmse < 0.015          # 4-bit Lloyd-Max on a Gaussian: 0.0095
