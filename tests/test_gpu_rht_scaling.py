"""The transform fused with the quantiser (dq_rht_scaling_compress, dq_scaling_decompress_irht) against the two-call
sequences it replaces -- rht_blocked + scaling_compress, scaling_decompress + inverse rht_blocked -- byte for byte /
bit for bit, and one case straight against the oracle."""
import math

import numpy as np
import pytest
import torch

from helpers import F32, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(n, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(n, generator=g) * 1e-3).to(DEV)
    sign = (torch.randint(0, 2, (n,), generator=g).float() * 2 - 1).to(DEV)
    return g, x, sign


@pytest.mark.parametrize("block", [2, 64, 256, 1024, 4096, 8192, 16384, 32768])
@pytest.mark.parametrize("nbits,strategy", [(2, 2), (4, 2), (5, 3), (8, 3), (8, 2)])
def test_fused_equals_two_calls(capi, block, nbits, strategy):
    # a vector that is not a whole number of 8192-element tiles, and at least two transform blocks
    n = max(3 * 8192 + 2048 + 256, 2 * block)
    n = (n + block - 1) // block * block
    n = (n + 255) // 256 * 256
    assert n % block == 0
    g, x, sign = _case(n, block + nbits)
    scale = 1.0 / np.sqrt(block)
    nb = capi.required_bytes(n, nbits, 16, strategy)
    for pool_dt in (torch.float32, torch.bfloat16, None):
        rot = x.clone()
        capi.rht_blocked(rot, sign, block, scale, False)
        want = torch.zeros(nb, dtype=torch.uint8, device=DEV)
        if pool_dt is None:
            capi.scaling_compress_philox(rot, want, n, nbits, 16, strategy, 11, 3)
            pool = None
        else:
            pool = torch.rand(n, generator=g).to(pool_dt).to(DEV)
            capi.scaling_compress(rot, want, pool, n, nbits, 16, strategy)
        x_before = x.clone()
        got = torch.full((nb + 32,), 0x5A, dtype=torch.uint8, device=DEV)
        capi.rht_scaling_compress(x, sign, got, block, scale, nbits, strategy, rand_pool=pool, seed=11, step=3)
        assert torch.equal(x, x_before)
        assert torch.equal(got[:nb], want), (block, nbits, strategy, pool_dt)
        assert bool((got[nb:] == 0x5A).all())
    # the signs as one bit per element: same bytes (the last `want` is the in-kernel random stream's)
    bits = capi.pack_signs(sign)
    got = torch.zeros(nb, dtype=torch.uint8, device=DEV)
    capi.rht_scaling_compress(x, bits, got, block, scale, nbits, strategy, seed=11, step=3)
    assert torch.equal(got, want)
    # the way back
    dec = torch.empty(n, dtype=torch.float32, device=DEV)
    capi.scaling_decompress(want, dec, n, nbits, 16, strategy)
    capi.rht_blocked(dec, sign, block, scale, True)
    back = torch.full((n + 8,), 7.0, dtype=torch.float32, device=DEV)
    capi.scaling_decompress_irht(want, sign, back[:n], block, scale, nbits, strategy)
    assert torch.equal(back[:n].view(torch.int32), dec.view(torch.int32))
    assert bool((back[n:] == 7.0).all())
    back2 = torch.empty(n, dtype=torch.float32, device=DEV)
    capi.scaling_decompress_irht(want, bits, back2, block, scale, nbits, strategy)
    assert torch.equal(back2.view(torch.int32), dec.view(torch.int32))
    err = float((back[:n] - x).pow(2).sum() / x.pow(2).sum())
    assert err < {2: 1.0, 4: 0.05, 5: 0.02, 8: 2e-3}[nbits]


@pytest.mark.parametrize("nbits", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("strategy", [2, 3])
@pytest.mark.parametrize("block", [16384, 32768])
def test_blocks_taken_in_two_halves_every_width(capi, nbits, strategy, block):
    """the forward kernel for blocks of 2^14 and 2^15 takes a block in two halves and keeps the second one in the LDS
    through the quantiser of the first (blocks of 2^15: up to 6-bit codes, its record windows then lie behind the tile;
    one workgroup per CU above): every width, every rounding source, against the two calls"""
    n = 3 * block
    g, x, sign = _case(n, 77 + nbits)
    bits = capi.pack_signs(sign)
    scale = 1.0 / np.sqrt(block)
    nb = capi.required_bytes(n, nbits, 16, strategy)
    rot = x.clone()
    capi.rht_blocked(rot, sign, block, scale, False)
    for pool_dt in (None, torch.bfloat16, torch.float32):
        want = torch.zeros(nb, dtype=torch.uint8, device=DEV)
        if pool_dt is None:
            pool = None
            capi.scaling_compress_philox(rot, want, n, nbits, 16, strategy, 5, 9)
        else:
            pool = torch.rand(n, generator=g).to(pool_dt).to(DEV)
            capi.scaling_compress(rot, want, pool, n, nbits, 16, strategy)
        got = torch.full((nb + 32,), 0x5A, dtype=torch.uint8, device=DEV)
        capi.rht_scaling_compress(x, bits, got, block, scale, nbits, strategy, rand_pool=pool, seed=5, step=9)
        assert torch.equal(got[:nb], want), (nbits, strategy, pool_dt)
        assert bool((got[nb:] == 0x5A).all())
    dec = torch.empty(n, dtype=torch.float32, device=DEV)
    capi.scaling_decompress(want, dec, n, nbits, 16, strategy)
    capi.rht_blocked(dec, sign, block, scale, True)
    back = torch.empty(n, dtype=torch.float32, device=DEV)
    capi.scaling_decompress_irht(want, bits, back, block, scale, nbits, strategy)
    assert torch.equal(back.view(torch.int32), dec.view(torch.int32))


@pytest.mark.parametrize("n,block", [(256, 256), (256, 16), (512, 512), (768, 256), (1280, 256), (2048, 1024)])
def test_small_vectors_no_sign_unaligned(capi, n, block):
    g, x, _ = _case(n, n + block)
    pool = torch.rand(n, generator=g).to(DEV)
    nb = capi.required_bytes(n, 4, 16, 2)
    rot = x.clone()
    capi.rht_blocked(rot, None, block, 0.5, False)
    want = torch.zeros(nb, dtype=torch.uint8, device=DEV)
    capi.scaling_compress(rot, want, pool, n, 4, 16, 2)
    # source, pool and stream at addresses that are only element / byte aligned
    xs = torch.zeros(n + 8, device=DEV)[1:1 + n].copy_(x)
    ps = torch.zeros(n + 8, device=DEV)[3:3 + n].copy_(pool)
    got = torch.zeros(nb + 16, dtype=torch.uint8, device=DEV)[7:7 + nb]
    capi.rht_scaling_compress(xs, None, got, block, 0.5, 4, 2, rand_pool=ps)
    assert torch.equal(got, want)
    dec = torch.empty(n, device=DEV)
    capi.scaling_decompress(want, dec, n, 4, 16, 2)
    capi.rht_blocked(dec, None, block, 0.5, True)
    back = torch.zeros(n + 8, device=DEV)[1:1 + n]
    capi.scaling_decompress_irht(got, None, back, block, 0.5, 4, 2)
    assert torch.equal(back.view(torch.int32), dec.view(torch.int32))


@pytest.mark.parametrize("n", [1, 31, 32, 33, 64, 255, 1000, 100003])
def test_pack_signs(capi, n):
    g = torch.Generator().manual_seed(n)
    sign = (torch.randint(0, 2, (n,), generator=g).float() * 2 - 1)
    bits = capi.pack_signs(sign.to(DEV)).cpu().numpy().view(np.uint32)
    want = np.packbits((sign.numpy() < 0).astype(np.uint8), bitorder="little")
    want = np.concatenate([want, np.zeros(-want.size % 4, np.uint8)]).view(np.uint32)
    mask = np.full(want.size, 0xFFFFFFFF, np.uint32)
    if n % 32:
        mask[-1] = (1 << (n % 32)) - 1
    assert ((bits & mask) == want).all()


def test_fused_against_oracle(capi, oracle):
    n, block, nbits, strategy = 8192 + 4096, 4096, 5, 3
    g, x, sign = _case(n, 99)
    pool = torch.rand(n, generator=g)
    scale = np.float32(1.0 / np.sqrt(block))
    got = torch.zeros(capi.required_bytes(n, nbits, 16, strategy), dtype=torch.uint8, device=DEV)
    capi.rht_scaling_compress(x, sign, got, block, float(scale), nbits, strategy, rand_pool=pool.to(DEV))
    rot = oracle.rht_blocked(x.cpu().numpy(), sign.cpu().numpy(), block, scale)
    want = oracle.scaling_compress(rot, pool.numpy(), n, nbits, 16, strategy, F32)
    assert (got.cpu().numpy() == want).all()
    dec = np.zeros(n, np.float32)
    oracle.scaling_decompress(want, dec, n, nbits, 16, strategy, F32)
    back_o = oracle.rht_blocked(dec, sign.cpu().numpy(), block, scale, inverse=True)
    back = torch.empty(n, device=DEV)
    capi.scaling_decompress_irht(got, sign, back, block, float(scale), nbits, strategy)
    assert (back.cpu().numpy().view(np.uint32) == back_o.view(np.uint32)).all()


def test_fused_full_size_properties(capi):
    """2^26 elements, block 2^15 (the largest tile): round trip error and the same bytes as the two calls on a slice"""
    n, block, nbits = 1 << 26, 1 << 15, 4
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(n, generator=g, device=DEV) * 1e-3
    sign = torch.empty(n, device=DEV)
    capi.rand_diag(sign, 5)
    scale = 1.0 / np.sqrt(block)
    enc = torch.zeros(capi.required_bytes(n, nbits, 16, 2), dtype=torch.uint8, device=DEV)
    capi.rht_scaling_compress(x, sign, enc, block, scale, nbits, 2, seed=1, step=2)
    back = torch.empty_like(x)
    capi.scaling_decompress_irht(enc, sign, back, block, scale, nbits, 2)
    err = float((back - x).pow(2).sum() / x.pow(2).sum())
    assert 0.005 < err < 0.03, err
    rot = x.clone()
    capi.rht_blocked(rot, sign, block, scale, False)
    want = torch.zeros_like(enc)
    capi.scaling_compress_philox(rot, want, n, nbits, 16, 2, 1, 2)
    assert torch.equal(enc, want)


@pytest.mark.parametrize("strategy", [2, 3])
def test_fused_special_values(capi, strategy):
    """non-finite and extreme inputs spread over whole transform blocks by the butterflies: still the two-call bytes"""
    n, block, nbits = 8192 * 3, 1024, 4
    g, x, sign = _case(n, 5)
    x[3] = float("inf"); x[1024 + 7] = float("nan"); x[2048:3072] = 0.0; x[4096] = 3e38; x[4097] = 3e38
    x[5120:6144] = 1e-40
    pool = torch.rand(n, generator=g).to(DEV)
    pool[9000] = 2.0
    scale = 1.0 / 32
    rot = x.clone()
    capi.rht_blocked(rot, sign, block, scale, False)
    nb = capi.required_bytes(n, nbits, 16, strategy)
    want = torch.zeros(nb, dtype=torch.uint8, device=DEV)
    capi.scaling_compress(rot, want, pool, n, nbits, 16, strategy)
    got = torch.zeros(nb, dtype=torch.uint8, device=DEV)
    capi.rht_scaling_compress(x, capi.pack_signs(sign), got, block, scale, nbits, strategy, rand_pool=pool)
    assert torch.equal(got, want)
    dec = torch.empty(n, device=DEV)
    capi.scaling_decompress(want, dec, n, nbits, 16, strategy)
    capi.rht_blocked(dec, sign, block, scale, True)
    back = torch.empty(n, device=DEV)
    capi.scaling_decompress_irht(got, sign, back, block, scale, nbits, strategy)
    assert torch.equal(back.view(torch.int32), dec.view(torch.int32))


@pytest.mark.parametrize("block", [16, 1024, 8192, 16384])
def test_matrix_core_variant_agrees_to_rounding_error(capi, block):
    """dq_rht_scaling_compress_mfma16 forms the first four stages as a matrix product: another summation order, so
    the records agree with the butterfly kernel's except for codes whose value sat on a rounding boundary"""
    n = 1 << 18
    g = torch.Generator().manual_seed(block)
    x = (torch.randn(n, generator=g) * 1e-3).to(DEV)
    sign = torch.empty(n // 32, dtype=torch.int32, device=DEV)
    capi.rand_diag_bits(sign, n, 7)
    scale = 1.0 / math.sqrt(block)
    nbytes = capi.required_bytes(n, 4, 16, 2)
    a = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    b = torch.zeros(nbytes + 16, dtype=torch.uint8, device=DEV)
    capi.rht_scaling_compress(x, sign, a, block, scale, 4, 2, seed=11, step=2)
    capi.rht_scaling_compress_mfma16(x, sign, b, block, scale, seed=11, step=2)
    assert bool((b[nbytes:] == 0).all())
    differing = float((a != b[:nbytes]).float().mean())
    assert differing < 2e-3, differing
    out_a, out_b = torch.empty_like(x), torch.empty_like(x)
    capi.scaling_decompress_irht(a, sign, out_a, block, scale, 4, 2)
    capi.scaling_decompress_irht(b[:nbytes].clone(), sign, out_b, block, scale, 4, 2)
    nm = lambda y: float(((y - x).double() ** 2).sum() / (x.double() ** 2).sum())
    assert abs(nm(out_a) - nm(out_b)) < 0.01 * nm(out_a)
    with pytest.raises(RuntimeError):
        capi.rht_scaling_compress_mfma16(x, sign, b, 8, 1.0)
