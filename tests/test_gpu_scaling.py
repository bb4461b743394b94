"""GPU parity of the scaling-quantisation entry points against the CPU oracle.

Everything here calls the HIP kernels through the C ABI (ctypes) or through the
`eden_utils` binding that sits on top of it, and compares packed bytes / decoded
bit patterns with the oracle: bit-exact, no tolerance.
"""
import numpy as np
import pytest
import torch

from helpers import BF16, F16, F32, TORCH_DT, bits_to_f32, from_bits, make_input, make_rand, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cmp_bits(name, got, want):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, name
    if got.dtype == np.float32:
        # bit patterns, except that any NaN matches any NaN
        nan = np.isnan(got) & np.isnan(want)
        got = np.where(nan, 0, got.view(np.uint32))
        want = np.where(nan, 0, want.view(np.uint32))
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, "%s: %d mismatches, first at %d: got %r want %r" % (
        name, bad.size, bad[0], got[bad[0]], want[bad[0]])


def _roundtrip(capi, oracle, dt, n, nbits, C, strategy, src_t, rand_t, tag):
    nbytes = oracle.required_bytes(n, nbits, C, strategy)
    assert capi.required_bytes(n, nbits, C, strategy) == nbytes
    src_d, rand_d = src_t.to(DEV), rand_t.to(DEV)
    enc_d = torch.full((nbytes + 7,), 0xAB, dtype=torch.uint8, device=DEV)
    capi.scaling_compress(src_d, enc_d, rand_d, n, nbits, C, strategy)
    torch.cuda.synchronize()
    enc_o = oracle.scaling_compress(to_bits(src_t), to_bits(rand_t), n, nbits, C, strategy, dt)
    enc_g = enc_d.cpu().numpy()
    _cmp_bits(tag + " compress", enc_g[:nbytes], enc_o)
    assert (enc_g[nbytes:] == 0xAB).all(), tag + " wrote past the packed stream"

    # decompress (overwrite)
    dec_d = torch.zeros(n, dtype=TORCH_DT[dt], device=DEV)
    capi.scaling_decompress(enc_d, dec_d, n, nbits, C, strategy)
    dec_o = np.zeros(n, np.float32 if dt == F32 else np.uint16)
    oracle.scaling_decompress(enc_o, dec_o, n, nbits, C, strategy, dt)
    _cmp_bits(tag + " decompress", to_bits(dec_d), dec_o)

    # decompress_add
    base_t = (src_t.float() * 0.125).to(TORCH_DT[dt])
    add_d = base_t.to(DEV)
    capi.scaling_decompress(enc_d, add_d, n, nbits, C, strategy, add=True)
    add_o = to_bits(base_t)
    oracle.scaling_decompress(enc_o, add_o, n, nbits, C, strategy, dt, add=True)
    _cmp_bits(tag + " decompress_add", to_bits(add_d), add_o)
    return enc_o


def _dec_comp(capi, oracle, dt, n, nbits, C, strategy, recv_src_t, inp_t, rand_recv_t, rand_send_t, tag):
    nbytes = oracle.required_bytes(n, nbits, C, strategy)
    recv_o = oracle.scaling_compress(to_bits(recv_src_t), to_bits(rand_recv_t), n, nbits, C, strategy, dt)
    recv_d = torch.from_numpy(recv_o).to(DEV)
    inp_d = inp_t.to(DEV)
    send_d = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    capi.scaling_dec_comp(recv_d, inp_d, send_d, rand_send_t.to(DEV), n, nbits, C, strategy)
    torch.cuda.synchronize()
    inp_o = to_bits(inp_t)
    send_o = oracle.scaling_dec_comp(recv_o, inp_o, to_bits(rand_send_t), n, nbits, C, strategy, dt)
    _cmp_bits(tag + " dec_comp send", send_d.cpu().numpy(), send_o)
    # inp: untouched by the fused path, holds the sum on the split path -- same as the oracle
    _cmp_bits(tag + " dec_comp inp", to_bits(inp_d), inp_o)

    # the reference's own invariant: fused bytes == decompress_add + compress bytes
    inp2_d = inp_t.to(DEV)
    capi.scaling_decompress(recv_d, inp2_d, n, nbits, C, strategy, add=True)
    send2_d = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    capi.scaling_compress(inp2_d, send2_d, rand_send_t.to(DEV), n, nbits, C, strategy)
    assert torch.equal(send_d, send2_d), tag + " fused != split"


@pytest.mark.parametrize("dt", [F16, BF16])
@pytest.mark.parametrize("C", [16, 32])
@pytest.mark.parametrize("nbits", [2, 4, 8])
@pytest.mark.parametrize("strategy", [0, 1, 2, 3])
def test_functional_sweep(capi, oracle, dt, C, nbits, strategy):
    """The 48-case sweep of the reference's functional test, bit-exact."""
    tdt = TORCH_DT[dt]
    n = C * (32 if strategy >= 2 else 19)
    src = make_input(n, tdt)
    rnd = make_rand(n, 1000 + nbits * 31 + C * 7 + strategy, tdt)
    tag = "dt=%d C=%d b=%d s=%d" % (dt, C, nbits, strategy)
    _roundtrip(capi, oracle, dt, n, nbits, C, strategy, src, rnd, tag)
    recv_src = (make_input(n, tdt).float() * 0.5).to(tdt)
    inp = (make_input(n, tdt).float() * -0.25).to(tdt)
    _dec_comp(capi, oracle, dt, n, nbits, C, strategy, recv_src, inp,
              make_rand(n, 2000 + nbits * 17 + C + strategy, tdt),
              make_rand(n, 3000 + nbits * 19 + C + strategy, tdt), tag)


@pytest.mark.parametrize("dt", [F16, BF16, F32])
@pytest.mark.parametrize("C", [8, 32])
@pytest.mark.parametrize("strategy", [0, 1, 2, 3])
def test_chunks_of_8_and_32_in_aligned_buffers(capi, oracle, dt, C, strategy):
    """chunk sizes 8 and 32 in 16-byte aligned buffers (the kernels that keep the chunk in registers): chunk counts
    that end inside a wave, inside a workgroup and past one, every width the chunk size allows, canaries around the
    decoded vector"""
    tdt = TORCH_DT[dt]
    for nbits in (2, 3, 4, 5, 8):
        if (C * nbits) % 8:
            continue
        for nchunks in (16, 48, 208, 256 + 80, 1024 + 16):
            n = C * nchunks
            g = torch.Generator().manual_seed(C * 1000 + nbits * 10 + strategy + nchunks)
            src = (torch.randn(n, generator=g) * 0.02).to(tdt)
            if nchunks == 48:
                src[5] = float("inf")
            if nchunks == 208:                      # NaN, -inf, a zero chunk, a chunk of tiny values, one of huge ones
                src[7], src[C + 3] = float("nan"), float("-inf")
                src[2 * C:3 * C] = 0.0
                src[3 * C:4 * C] = (torch.randn(C, generator=g) * 1e-30).to(tdt)
                src[4 * C:5 * C] = (torch.randn(C, generator=g) * (6e4 if dt == F16 else 1e30)).to(tdt)
            rnd = torch.rand(n, generator=g).to(tdt)
            tag = "dt=%d C=%d b=%d s=%d chunks=%d" % (dt, C, nbits, strategy, nchunks)
            enc_o = _roundtrip(capi, oracle, dt, n, nbits, C, strategy, src, rnd, tag)
            # the decoded vector inside a larger buffer, 16-byte aligned at both ends
            pad = 16
            buf = torch.full((n + 2 * pad,), 3.0, dtype=tdt, device=DEV)
            capi.scaling_decompress(torch.from_numpy(enc_o).to(DEV), buf[pad:pad + n], n, nbits, C, strategy)
            got = buf.float().cpu()
            assert bool((got[:pad] == 3).all()) and bool((got[pad + n:] == 3).all()), tag + " wrote outside the vector"
            inp = (torch.randn(n, generator=g) * 0.01).to(tdt)
            _dec_comp(capi, oracle, dt, n, nbits, C, strategy, src, inp, rnd, torch.rand(n, generator=g).to(tdt), tag)


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("nbits", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("strategy", [2, 3])
def test_production_shape_random(capi, oracle, dt, nbits, strategy):
    """chunk 16 / superchunk 16 on random gradients, ragged superchunk counts."""
    tdt = TORCH_DT[dt]
    g = torch.Generator().manual_seed(77 + nbits * 5 + strategy)
    for nsc in (1, 3, 4, 5, 16, 67, 1030):
        n = nsc * 256
        scale = torch.exp(torch.randn(nsc, 1, generator=g) * 3.0 - 7.0)
        src = (torch.randn(nsc, 256, generator=g) * scale).reshape(-1).to(tdt)
        rnd = torch.rand(n, generator=g).to(tdt)
        tag = "dt=%d b=%d s=%d nsc=%d" % (dt, nbits, strategy, nsc)
        _roundtrip(capi, oracle, dt, n, nbits, 16, strategy, src, rnd, tag)
        inp = (torch.randn(n, generator=g) * 2e-3).to(tdt)
        _dec_comp(capi, oracle, dt, n, nbits, 16, strategy, src, inp, rnd, torch.rand(n, generator=g).to(tdt), tag)


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("strategy", [2, 3])
def test_special_values(capi, oracle, dt, strategy):
    """zeros, denormals, huge values, inf/nan inputs, rand exactly 0 and 1."""
    tdt = TORCH_DT[dt]
    n = 256 * 8
    g = torch.Generator().manual_seed(5)
    src = torch.randn(n, generator=g) * 1e-3
    src[0:256] = 0.0
    src[256:512] *= 1e-38
    src[512:768] *= 1e35
    src[768] = float("inf")
    src[800] = float("-inf")
    src[1030] = float("nan")
    src[1280:1536] = 3.0e38
    src[1536:1552] = 0.0
    src[1792:2048] = torch.randn(256, generator=g) * 1e-3
    src[1800] = 1e30
    src = src.to(tdt)
    rnd = torch.rand(n, generator=g)
    rnd[::7] = 0.0
    rnd[3::11] = 1.0
    rnd = rnd.to(tdt)
    for nbits in (2, 4, 8):
        _roundtrip_nan_safe = _roundtrip  # codes and scale bytes never hold NaN: exact compare is valid
        _roundtrip_nan_safe(capi, oracle, dt, n, nbits, 16, strategy, src, rnd, "special b=%d" % nbits)


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("strategy", [0, 1, 2, 3])
@pytest.mark.parametrize("C", [16, 8, 32])
def test_zero_elements_with_random_values_0_and_1(capi, oracle, dt, strategy, C):
    """Ordinary magnitudes throughout (so every wave takes the estimate route), many exact zeros of either sign, and
    random values that are exactly 0 and exactly 1 on zero and non-zero elements alike: coordinate - random value is an
    integer for those zeros, the case the estimate cannot decide (ceil(-0) = 0, ceil(-1) = -1 in the reference's chain)."""
    tdt = TORCH_DT[dt]
    n = 256 * 24
    g = torch.Generator().manual_seed(77 + strategy)
    src = torch.randn(n, generator=g) * 1e-2
    src[torch.rand(n, generator=g) < 0.4] = 0.0
    src[5::13] = -0.0
    src[1024:1280] = 0.0            # whole superchunks of zeros
    src = src.to(tdt)
    rnd = torch.rand(n, generator=g)
    rnd[::3] = 0.0
    rnd[1::5] = 1.0
    rnd = rnd.to(tdt)
    for nbits in (2, 4, 5, 8):
        if (C * nbits) % 8:
            continue
        tag = "zeros dt=%d C=%d b=%d s=%d" % (dt, C, nbits, strategy)
        _roundtrip(capi, oracle, dt, n, nbits, C, strategy, src, rnd, tag)
        inp = (torch.randn(n, generator=g) * 1e-2)
        inp[torch.rand(n, generator=g) < 0.5] = 0.0
        _dec_comp(capi, oracle, dt, n, nbits, C, strategy, src, inp.to(tdt), rnd, rnd.flip(0).contiguous(), tag)


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("strategy", [0, 1, 2, 3])
@pytest.mark.parametrize("C", [16, 8, 32])
def test_estimate_route_at_the_ends_of_its_range(capi, oracle, dt, strategy, C):
    """Inputs that keep every wave on the estimate route (finite, ordinary scales, random values in [0, 1]) and sit at the
    ends of what it handles: magnitudes from 2^-95 to 2^95, chunks whose elements all equal plus or minus the chunk maximum
    (their coordinate is +-R, or just beyond when the stored scale rounds down: the clamp on either side), and random
    values 0, 1 and next to them."""
    tdt = TORCH_DT[dt]
    nsc = 24
    n = nsc * 16 * C
    g = torch.Generator().manual_seed(400 + strategy + C)
    mags = torch.tensor([2.0 ** -95, 2.0 ** -60, 2.0 ** -20, 1.0, 2.0 ** 20, 2.0 ** 60, 2.0 ** 95, 3.0e-2])
    src = torch.randn(nsc, 16, C, generator=g)
    # every third chunk: all elements at +- the same magnitude; the others: one maximum, the rest random below it
    sign = torch.where(torch.rand(nsc, 16, C, generator=g) < 0.5, -1.0, 1.0)
    flat = (torch.arange(16).view(1, 16, 1) % 3 == 0)
    src = torch.where(flat, sign * (1.0 + torch.rand(nsc, 16, 1, generator=g)), src.clamp(-3.0, 3.0) / 3.0)
    src[:, :, 0] = torch.where(flat[:, :, 0].expand(nsc, 16), src[:, :, 0], sign[:, :, 0] * 1.0)
    src = (src * mags[torch.arange(nsc) % mags.numel()].view(nsc, 1, 1)).reshape(-1)
    edge = torch.tensor([0.0, 1.0, 2.0 ** -8, 1.0 - 2.0 ** -8, 2.0 ** -20, 0.5, 0.99609375, 0.00390625])
    rnd = torch.rand(n, generator=g)
    pick = torch.rand(n, generator=g) < 0.5
    rnd = torch.where(pick, edge[torch.randint(0, edge.numel(), (n,), generator=g)], rnd)
    src, rnd = src.to(tdt), rnd.to(tdt)
    for nbits in (2, 4, 5, 8):
        if (C * nbits) % 8:
            continue
        tag = "edges dt=%d C=%d b=%d s=%d" % (dt, C, nbits, strategy)
        _roundtrip(capi, oracle, dt, n, nbits, C, strategy, src, rnd, tag)
        _dec_comp(capi, oracle, dt, n, nbits, C, strategy, src, (src.float() * -0.5).to(tdt), rnd, rnd.flip(0).contiguous(), tag)


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("strategy", [0, 1, 2, 3])
@pytest.mark.parametrize("C", [16, 8, 32])
def test_subnormal_quotients_half_way_between_two_subnormal_numbers(capi, oracle, dt, strategy, C):
    """Elements v = m 2^-150 d (m odd, d the quantisation step of their chunk) with random value 0: the quotient v / d
    is a tie between two subnormal numbers, which the division rounds to even and a product with an inexact reciprocal
    of d does not, and with a random value of 0 the code is R for a quotient of 0 and R + 1 for anything above.  Such
    a v exists when d is an even multiple of a power of two (binary32 elements) or a multiple of 2^17 (bfloat16): the
    chunk maxima are chosen so that d = q 2^k."""
    from helpers import unpack_stream
    tdt = TORCH_DT[dt]
    nsc = 40
    n = nsc * 16 * C
    g = torch.Generator().manual_seed(5150 + strategy + C)
    ks = torch.tensor([1, 2, 3, 5, 17, 18, 20, 30, 40, 60])
    qs = torch.tensor([255, 3, 5, 6, 7, 9, 10, 11, 12, 13, 14, 15, 20, 22, 100, 254])
    placed = 0
    for nbits in (2, 4, 8):
        if (C * nbits) % 8:
            continue
        R = (1 << (nbits - 1)) - 1
        amax = (qs.double() - torch.where(qs == 255, 0.0, 0.5)).view(1, 16) * (2.0 ** ks[torch.arange(nsc) % ks.numel()].double()).view(nsc, 1) * R
        src = (torch.rand(nsc, 16, C, generator=g).double() - 0.5) * amax.view(nsc, 16, 1)
        src[:, :, 0] = amax * torch.where(torch.rand(nsc, 16, generator=g) < 0.5, -1.0, 1.0)
        src = src.reshape(-1).float().to(tdt)
        enc = oracle.scaling_compress(to_bits(src), to_bits(torch.full((n,), 0.5).to(tdt)), n, nbits, C, strategy, dt)
        _, (a0, a1) = unpack_stream(enc, n, nbits, C, strategy)
        if strategy >= 2:
            step = a0.astype(np.float64) * bits_to_f32(a1, BF16).astype(np.float64).repeat(16)
        else:
            step = bits_to_f32(a0, BF16).astype(np.float64)
        vals = src.double().reshape(-1, C).clone()
        rnd = torch.rand(n // C, C, generator=g)
        for slot, m in enumerate((1, 3, 5, 7, 9, 11, 13), start=1):
            if slot >= C:
                break
            cand = torch.from_numpy(step * m * 2.0 ** -150)
            cand = torch.where(torch.rand(cand.shape, generator=g) < 0.5, -cand, cand)
            ok = (cand.float().to(tdt).double() == cand) & (cand != 0)
            vals[:, slot] = torch.where(ok, cand, vals[:, slot])
            rnd[:, slot] = torch.where(ok, torch.tensor([0.0, 0.0, 1.0, 2.0 ** -20])[torch.randint(0, 4, ok.shape, generator=g)], rnd[:, slot])
            placed += int(ok.sum())
        src2 = vals.reshape(-1).float().to(tdt)
        assert torch.equal(src2.double().reshape(-1, C)[:, 0], src.double().reshape(-1, C)[:, 0])
        tag = "ties dt=%d C=%d b=%d s=%d" % (dt, C, nbits, strategy)
        _roundtrip(capi, oracle, dt, n, nbits, C, strategy, src2, rnd.reshape(-1).to(tdt), tag)
    assert placed > (400 if dt == F32 else 40), placed


@pytest.mark.parametrize("nbits", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("strategy", [2, 3])
@pytest.mark.parametrize("C", [16, 8, 32])
def test_random_values_on_the_rounding_boundary(capi, oracle, nbits, strategy, C):
    """The kernels decide most codes from a cheap estimate of the coordinate and redo an element with the reference's
    exact chain when coordinate - random value comes close to an integer.  Here every random value is the fractional
    part of its element's coordinate (to float32 accuracy, and one or two float32 steps beside it), so every element
    sits on that boundary: bytes must still be the oracle's."""
    from helpers import unpack_stream
    if (C * nbits) % 8:
        pytest.skip("the code bytes of a chunk must be whole")
    nsc = 40
    n = nsc * 16 * C
    g = torch.Generator().manual_seed(900 + 10 * nbits + strategy)
    scale = torch.exp(torch.randn(nsc, 1, generator=g) * 2.0 - 6.0)
    src = (torch.randn(nsc, 16 * C, generator=g) * scale).reshape(-1)
    src[5::97] = 0.0
    # the quantisation steps the oracle uses: from the records of a first pass with any random values
    enc = oracle.scaling_compress(src.numpy(), np.full(n, 0.5, np.float32), n, nbits, C, strategy, F32)
    _, (q, unit) = unpack_stream(enc, n, nbits, C, strategy)
    step = q.astype(np.float64).repeat(C) * bits_to_f32(unit, BF16).astype(np.float64).repeat(16 * C)
    x = src.numpy().astype(np.float64) / step
    if strategy == 3:
        _, params = capi.mee_lookup_table(nbits)
        c, l2b = (float(v) for v in params[[1, 3]].view(np.float16).astype(np.float64))
        x = np.sign(x) * np.log2(np.abs(x) / c + 1.0) / l2b
    frac = (x - np.floor(x)).astype(np.float32)
    for shift in (0, 1, -1, 2, -2):
        rnd = frac.copy()
        for _ in range(abs(shift)):
            rnd = np.nextafter(rnd, np.float32(2.0 if shift > 0 else -1.0))
        rnd = np.clip(rnd, 0.0, 1.0).astype(np.float32)
        tag = "boundary C=%d b=%d s=%d shift=%d" % (C, nbits, strategy, shift)
        _roundtrip(capi, oracle, F32, n, nbits, C, strategy, src, torch.from_numpy(rnd), tag)
        # the fused ring step sees the same situation through its accumulated input
        if shift == 0:
            inp = torch.zeros(n)
            _dec_comp(capi, oracle, F32, n, nbits, C, strategy, src, inp, torch.from_numpy(rnd), torch.from_numpy(rnd), tag)


def _wide_source(n, tdt, seed):
    """random magnitudes over the whole exponent range of the type, plus zeros, infinities, NaN and
    values the type cannot hold without rounding to the extremes"""
    g = torch.Generator().manual_seed(seed)
    lo, hi = (-24, 15) if tdt == torch.float16 else (-60, 60)
    expo = torch.randint(lo, hi, (n // 16,), generator=g).float().repeat_interleave(16)
    src = torch.randn(n, generator=g) * torch.pow(2.0, expo) * torch.pow(2.0, torch.randint(-6, 1, (n,), generator=g).float())
    src[0:64] = 0.0
    src[100] = float("inf")
    src[333] = float("-inf")
    src[517] = float("nan")
    src[640:656] = float("nan")            # a whole chunk of NaN
    src[700:716] = 65504.0 if tdt == torch.float16 else 3.0e38
    return src.to(tdt)


@pytest.mark.parametrize("dt,strategies", [(F16, (0, 1, 2, 3)), (BF16, (0, 1)), (F32, (0, 1))])
@pytest.mark.parametrize("nbits", [2, 3, 4, 5, 6, 7, 8])
def test_tile16_shapes(capi, oracle, dt, strategies, nbits):
    """chunk 16 outside the production kernel -- binary16 elements, flat strategies: ordinary data over
    several tiles with a ragged last tile, then the special values; the ring step is the split one"""
    tdt = TORCH_DT[dt]
    for strategy in strategies:
        n = 16 * (64 * 5 + 16 * 3 + (0 if strategy >= 2 else 7))
        g = torch.Generator().manual_seed(nbits * 10 + strategy)
        src = (torch.randn(n, generator=g) * 1e-2).to(tdt)
        rnd = torch.rand(n, generator=g).to(tdt)
        tag = "tile16 dt=%d b=%d s=%d" % (dt, nbits, strategy)
        _roundtrip(capi, oracle, dt, n, nbits, 16, strategy, src, rnd, tag)
        inp = (torch.randn(n, generator=g) * 1e-2).to(tdt)
        _dec_comp(capi, oracle, dt, n, nbits, 16, strategy, src, inp, rnd, torch.rand(n, generator=g).to(tdt), tag)
        wide = _wide_source(n, tdt, nbits + strategy)
        rnd2 = torch.rand(n, generator=g)
        rnd2[::7] = 0.0
        rnd2[3::11] = 1.0
        _roundtrip(capi, oracle, dt, n, nbits, 16, strategy, wide, rnd2.to(tdt), tag + " wide")


def test_tile16_unaligned_and_mixed_pool(capi, oracle):
    """element views off the 16-byte grid, packed pointers at odd chunk offsets, bf16 pool beside fp32 elements"""
    g = torch.Generator().manual_seed(77)
    n = 16 * 151
    for tdt, dt, strategy, nbits in ((torch.float16, F16, 2, 4), (torch.float16, F16, 1, 8), (torch.bfloat16, BF16, 0, 4),
                                     (torch.float32, F32, 1, 5)):
        if strategy >= 2:
            n = 256 * 9
        src_t = (torch.randn(n, generator=g) * 1e-3).to(tdt)
        rnd_t = torch.rand(n, generator=g).to(tdt)
        nbytes = oracle.required_bytes(n, nbits, 16, strategy)
        enc_o = oracle.scaling_compress(to_bits(src_t), to_bits(rnd_t), n, nbits, 16, strategy, dt)
        big_src = torch.zeros(n + 64, dtype=tdt, device=DEV)
        big_rnd = torch.zeros(n + 64, dtype=tdt, device=DEV)
        big_src[3:3 + n] = src_t.to(DEV)
        big_rnd[1:1 + n] = rnd_t.to(DEV)
        for off in (1, 7, 16):
            buf = torch.zeros(nbytes + 32, dtype=torch.uint8, device=DEV)
            capi.scaling_compress(big_src[3:3 + n], buf[off:], big_rnd[1:1 + n], n, nbits, 16, strategy)
            got = buf.cpu().numpy()
            assert (got[:off] == 0).all() and (got[off + nbytes:] == 0).all()
            assert (got[off:off + nbytes] == enc_o).all()
            out = torch.zeros(n + 8, dtype=tdt, device=DEV)
            capi.scaling_decompress(buf[off:], out[5:5 + n], n, nbits, 16, strategy)
            dec_o = np.zeros(n, np.float32 if dt == F32 else np.uint16)
            oracle.scaling_decompress(enc_o, dec_o, n, nbits, 16, strategy, dt)
            _cmp_bits("unaligned", to_bits(out[5:5 + n]), dec_o)
            assert float(out[:5].abs().sum()) == 0.0 and float(out[5 + n:].abs().sum()) == 0.0
    # fp32 elements with a bf16 pool, flat
    src = torch.randn(n, generator=g) * 1e-3
    rnd16 = torch.rand(n, generator=g).to(torch.bfloat16)
    enc_d = torch.zeros(oracle.required_bytes(n, 4, 16, 0), dtype=torch.uint8, device=DEV)
    capi.scaling_compress(src.to(DEV), enc_d, rnd16.to(DEV), n, 4, 16, 0)
    _cmp_bits("mixed flat", enc_d.cpu().numpy(), oracle.scaling_compress(to_bits(src), to_bits(rnd16.float()), n, 4, 16, 0, F32))


def test_fp32_gradient_with_bf16_rand_pool(capi, oracle):
    """fp32 elements + bf16 random pool (DQ_RAND_BF16) == fp32 elements + the same values widened"""
    g = torch.Generator().manual_seed(21)
    n = 256 * 37
    src = torch.randn(n, generator=g) * 1e-3
    rnd16 = torch.rand(n, generator=g).to(torch.bfloat16)
    inp = torch.randn(n, generator=g) * 1e-3
    for nbits, strategy in ((4, 2), (8, 2), (4, 3), (5, 2)):
        nbytes = oracle.required_bytes(n, nbits, 16, strategy)
        enc_d = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        capi.scaling_compress(src.to(DEV), enc_d, rnd16.to(DEV), n, nbits, 16, strategy)
        enc_o = oracle.scaling_compress(to_bits(src), to_bits(rnd16.float()), n, nbits, 16, strategy, F32)
        _cmp_bits("mixed compress", enc_d.cpu().numpy(), enc_o)
        send_d = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        capi.scaling_dec_comp(enc_d, inp.to(DEV), send_d, rnd16.to(DEV), n, nbits, 16, strategy)
        send_o = oracle.scaling_dec_comp(enc_o, to_bits(inp), to_bits(rnd16.float()), n, nbits, 16, strategy, F32)
        _cmp_bits("mixed dec_comp", send_d.cpu().numpy(), send_o)


def test_unaligned_buffers(capi, oracle):
    """views with storage offsets: element pointers off the 16-byte grid, packed
    pointers at record-aligned (odd) offsets"""
    n = 256 * 9
    g = torch.Generator().manual_seed(9)
    for nbits, strategy in ((4, 2), (8, 3), (2, 2)):
        nbytes = oracle.required_bytes(n, nbits, 16, strategy)
        rec = nbytes // 9
        src_t = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
        rnd_t = torch.rand(n, generator=g).to(torch.bfloat16)
        big_src = torch.zeros(n + 64, dtype=torch.bfloat16, device=DEV)
        big_rnd = torch.zeros(n + 64, dtype=torch.bfloat16, device=DEV)
        big_src[3:3 + n] = src_t.to(DEV)
        big_rnd[16:16 + n] = rnd_t.to(DEV)
        enc_o = oracle.scaling_compress(to_bits(src_t), to_bits(rnd_t), n, nbits, 16, strategy, BF16)
        for off in (rec, 2 * rec + 0, 5 * rec):
            buf = torch.zeros(nbytes + 6 * rec, dtype=torch.uint8, device=DEV)
            capi.scaling_compress(big_src[3:3 + n], buf[off:], big_rnd[16:16 + n], n, nbits, 16, strategy)
            got = buf.cpu().numpy()
            assert (got[:off] == 0).all() and (got[off + nbytes:] == 0).all()
            assert (got[off:off + nbytes] == enc_o).all()
            out = torch.zeros(n + 8, dtype=torch.bfloat16, device=DEV)
            capi.scaling_decompress(buf[off:], out[5:5 + n], n, nbits, 16, strategy)
            dec_o = np.zeros(n, np.uint16)
            oracle.scaling_decompress(enc_o, dec_o, n, nbits, 16, strategy, BF16)
            assert (to_bits(out[5:5 + n]) == dec_o).all()
            assert float(out[:5].abs().sum()) == 0.0 and float(out[5 + n:].abs().sum()) == 0.0


def test_eden_utils_binding(eden_utils, oracle):
    """same calls as the reference's test, through the pybind module"""
    n, nbits, C, strategy = 16 * 32, 4, 16, 2
    src = make_input(n, torch.bfloat16, DEV)
    rnd = make_rand(n, 1234, torch.bfloat16, DEV)
    enc = torch.zeros(oracle.required_bytes(n, nbits, C, strategy), dtype=torch.uint8, device=DEV)
    dec = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream
    eden_utils.scaling_compress(src, enc, rnd, n, nbits, C, stream, strategy)
    eden_utils.scaling_decompress(enc, dec, n, nbits, C, stream, strategy)
    torch.cuda.synchronize()
    enc_o = oracle.scaling_compress(to_bits(src), to_bits(rnd), n, nbits, C, strategy, BF16)
    assert (enc.cpu().numpy() == enc_o).all()
    with pytest.raises(RuntimeError, match="nbits must be one of"):
        eden_utils.scaling_compress(src, enc, rnd, n, 5, C, stream, strategy)
    with pytest.raises(RuntimeError, match="input must be torch.float16 or torch.bfloat16"):
        eden_utils.scaling_compress(src.float(), enc, rnd.float(), n, nbits, C, stream, strategy)
    with pytest.raises(RuntimeError, match="output buffer is too small"):
        eden_utils.scaling_compress(src, enc[:-1], rnd, n, nbits, C, stream, strategy)
