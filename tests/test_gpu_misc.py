"""GPU parity of the superchunk, Hadamard, randDiag, bit-plane packing and
rounding entry points against the CPU oracle (bit-exact unless stated)."""
import math

import numpy as np
import pytest
import torch

from helpers import BF16, F16, F32, TORCH_DT, from_bits, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _eq(name, got, want):
    got, want = np.asarray(got), np.asarray(want)
    if got.dtype == np.float32:
        nan = np.isnan(got) & np.isnan(want)
        got = np.where(nan, 0, got.view(np.uint32))
        want = np.where(nan, 0, want.view(np.uint32))
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, "%s: %d mismatches, first at %d (%r vs %r)" % (name, bad.size, bad[0], got[bad[0]], want[bad[0]])


@pytest.mark.parametrize("dt", [F16, BF16, F32])
@pytest.mark.parametrize("n", [1, 255, 256, 257, 1000, 256 * 33, 256 * 1000 + 17])
@pytest.mark.parametrize("world", [1, 8, 3])
def test_superchunk_mean_center_and_back(capi, oracle, dt, n, world):
    tdt = TORCH_DT[dt]
    g = torch.Generator().manual_seed(n * 7 + world)
    src = (torch.randn(n, generator=g) * 1e-2 + 3e-3).to(tdt)
    nsc = (n + 255) // 256
    res_d = torch.full((nsc * 256,), 7.0, dtype=tdt, device=DEV)
    stats_d = torch.zeros(nsc * 2, dtype=torch.bfloat16, device=DEV)
    capi.superchunk_mean_center(src.to(DEV), res_d, stats_d, n, world)
    res_o, stats_o = oracle.superchunk_mean_center(to_bits(src), n, world, dt)
    _eq("residual", to_bits(res_d), res_o)
    _eq("stats", to_bits(stats_d), stats_o)
    out_d = torch.full((n + 3,), 5.0, dtype=tdt, device=DEV)
    capi.superchunk_add_mean_copy(res_d, out_d, stats_d, n)
    out_o = oracle.superchunk_add_mean_copy(res_o, stats_o, n, dt)
    _eq("add_mean", to_bits(out_d[:n]), out_o)
    assert (out_d[n:] == 5.0).all()


@pytest.mark.parametrize("dt", [F16, BF16, F32])
def test_superchunk_mean_center_wide_range_and_worlds(capi, oracle, dt):
    """every exponent (subnormal quotients, overflow to inf in fp16 squares), world sizes that are not
    powers of two (the division must stay correctly rounded), a view that is not 16-byte aligned"""
    tdt = TORCH_DT[dt]
    n = 256 * 517 + 100
    g = torch.Generator().manual_seed(31)
    expo = torch.randint(-40 if dt != F16 else -24, 30 if dt != F16 else 12, (n,), generator=g).float()
    src = (torch.randn(n, generator=g) * torch.pow(2.0, expo)).to(tdt)
    src[1000:1256] = 0.0
    nsc = (n + 255) // 256
    for world, shift in ((1, 0), (2, 0), (3, 0), (5, 3), (6, 0), (7, 0), (8, 0), (12, 0), (64, 0), (100, 8)):
        buf = torch.zeros(n + 16, dtype=tdt, device=DEV)
        view = buf[shift:shift + n]
        view.copy_(src)
        res_d = torch.full((nsc * 256,), 7.0, dtype=tdt, device=DEV)
        stats_d = torch.zeros(nsc * 2, dtype=torch.bfloat16, device=DEV)
        capi.superchunk_mean_center(view, res_d, stats_d, n, world)
        res_o, stats_o = oracle.superchunk_mean_center(to_bits(src), n, world, dt)
        _eq("residual W=%d" % world, to_bits(res_d), res_o)
        _eq("stats W=%d" % world, to_bits(stats_d), stats_o)


def test_superchunk_constant_block(capi):
    """closed form: a constant block has residual 0 and stats (c/W, 256*(c/W)^2)"""
    c, W = 0.5, 4
    src = torch.full((512,), c, dtype=torch.bfloat16, device=DEV)
    res = torch.ones(512, dtype=torch.bfloat16, device=DEV)
    stats = torch.zeros(4, dtype=torch.bfloat16, device=DEV)
    capi.superchunk_mean_center(src, res, stats, 512, W)
    assert float(res.abs().max()) == 0.0
    assert stats.float().tolist() == [c / W, 256 * (c / W) ** 2] * 2


@pytest.mark.parametrize("k", [0, 1, 2, 3, 5, 8, 10, 12, 13, 14, 15, 16, 17, 18, 19, 20, 21, 22, 23, 24])
def test_hadamard_whole_vector(capi, oracle, k):
    n = 1 << k
    g = torch.Generator().manual_seed(k)
    x = torch.randn(n, generator=g)
    x_d = x.to(DEV)
    capi.hadamard(x_d)
    _eq("fwht 2^%d" % k, x_d.cpu().numpy(), oracle.fwht(x.numpy()))


def test_hadamard_identities(capi):
    """H(e_i) = i-th Walsh row (+-1), H(1) = n e_0, H(H(x)) = n x on small integers"""
    n = 1 << 14
    e = torch.zeros(n, device=DEV)
    e[12345] = 1.0
    capi.hadamard(e)
    idx = torch.arange(n, device=DEV)
    par = torch.zeros(n, dtype=torch.int64, device=DEV)
    v = idx & 12345
    for b in range(14):
        par ^= (v >> b) & 1
    assert torch.equal(e, 1.0 - 2.0 * par.float())
    ones = torch.ones(n, device=DEV)
    capi.hadamard(ones)
    assert float(ones[0]) == n and float(ones[1:].abs().max()) == 0.0
    x = torch.randint(-8, 9, (n,), device=DEV).float()
    y = x.clone()
    capi.hadamard(y)
    capi.hadamard(y)
    assert torch.equal(y, x * n)


def test_hadamard_module_functions(eden_utils, oracle):
    n = 1 << 11
    x = torch.randn(n, device=DEV)
    ref = oracle.fwht(x.cpu().numpy())
    y = eden_utils.Hadamard(x, torch.cuda.current_stream().cuda_stream)
    assert y.data_ptr() != x.data_ptr()
    _eq("Hadamard", y.cpu().numpy(), ref)
    z = x.clone()
    eden_utils.Hadamard_inplace(z)
    _eq("Hadamard_inplace", z.cpu().numpy(), ref)
    w = x.clone()
    eden_utils.Hadamard_inplace_ptr(w.data_ptr(), n, 0)
    torch.cuda.synchronize()
    _eq("Hadamard_inplace_ptr", w.cpu().numpy(), ref)
    with pytest.raises(RuntimeError, match="power of 2"):
        eden_utils.Hadamard(torch.zeros(12, device=DEV))
    with pytest.raises(RuntimeError, match="torch.float32"):
        eden_utils.Hadamard(torch.zeros(16, device=DEV, dtype=torch.bfloat16))


@pytest.mark.parametrize("kb", [2, 4, 8, 10, 11, 12, 13, 14, 15, 16, 17, 20, 23])
@pytest.mark.parametrize("inverse", [False, True])
def test_rht_blocked(capi, oracle, kb, inverse):
    block = 1 << kb
    nblocks = 3 if kb <= 15 else (2 if kb < 23 else 1)
    n = block * nblocks
    g = torch.Generator().manual_seed(kb)
    x = torch.randn(n, generator=g) * 1e-3
    sign = (torch.randint(0, 2, (n,), generator=g) * 2 - 1).float()
    scale = 1.0 / math.sqrt(block)
    x_d = x.to(DEV)
    capi.rht_blocked(x_d, sign.to(DEV), block, scale, inverse)
    ref = oracle.rht_blocked(x.numpy(), sign.numpy(), block, np.float32(scale), inverse)
    _eq("rht", x_d.cpu().numpy(), ref)


def test_rht_roundtrip_is_identity(capi):
    """inverse(forward(x)) == x up to fp32 rounding (orthonormal transform)"""
    block, n = 1 << 12, 1 << 20
    x = torch.randn(n, device=DEV) * 1e-3
    sign = (torch.randint(0, 2, (n,), device=DEV) * 2 - 1).float()
    y = x.clone()
    s = 1.0 / math.sqrt(block)
    capi.rht_blocked(y, sign, block, s, False)
    # energy is preserved
    assert abs(float(y.double().pow(2).sum() / x.double().pow(2).sum()) - 1.0) < 1e-5
    capi.rht_blocked(y, sign, block, s, True)
    assert float((y - x).abs().max()) <= 1e-5 * float(x.abs().max())


@pytest.mark.parametrize("size", [8, 64, 100, 4096, 1000003])
@pytest.mark.parametrize("seed", [0, 1, 42, 2 ** 31])
def test_rand_diag(capi, oracle, size, seed):
    out = torch.zeros(size, device=DEV)
    capi.rand_diag(out, seed)
    _eq("rand_diag", out.cpu().numpy(), oracle.rand_diag(size, seed))


@pytest.mark.parametrize("size", [256, 768, 1024, 256 * 33, 1 << 20, 256 * 4097])
@pytest.mark.parametrize("seed", [0, 7, 2 ** 31])
def test_rand_diag_bits(capi, oracle, size, seed):
    """the diagonal generated as packed bits == the float diagonal of the oracle, packed"""
    bits = torch.full((size // 32 + 2,), 0x55555555, dtype=torch.int32, device=DEV)
    capi.rand_diag_bits(bits[:size // 32], size, seed)
    want = np.packbits(oracle.rand_diag(size, seed) < 0, bitorder="little").view(np.uint32)
    got = bits.cpu().numpy().view(np.uint32)
    assert (got[:size // 32] == want).all() and (got[size // 32:] == 0x55555555).all()
    sign = torch.empty(size, device=DEV)
    capi.rand_diag(sign, seed)
    assert torch.equal(capi.pack_signs(sign), bits[:size // 32])


@pytest.mark.parametrize("nbits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("nbins", [32, 64, 96, 1024, 1056, 100000 * 32])
def test_bit_plane_packing(capi, oracle, eden_utils, nbits, nbins):
    g = torch.Generator().manual_seed(nbits * 100 + nbins % 97)
    bins = torch.randint(0, 1 << nbits, (nbins,), generator=g, dtype=torch.int32)
    arr_o = oracle.bins_to_bits(bins.numpy(), nbits)
    arr_d = eden_utils.EdenBinsToBits(bins.to(DEV), nbits)
    assert arr_d.dtype == torch.int32 and arr_d.numel() == nbins // 32 * nbits
    _eq("bins_to_bits", arr_d.cpu().numpy().view(np.uint32), arr_o)
    back = eden_utils.EdenBitsToBins(arr_d, nbits)
    assert torch.equal(back.cpu(), bins)


@pytest.mark.parametrize("nbits", [3, 8, 9, 12, 17, 32])
def test_bit_plane_packing_wide_and_misaligned(capi, oracle, nbits):
    """planes beyond the first eight, bins with bits above nbits set (ignored), a source that is not 16-byte aligned"""
    nbins = 32 * 77
    g = torch.Generator().manual_seed(nbits)
    store = torch.randint(-2 ** 31, 2 ** 31 - 1, (nbins + 3,), generator=g, dtype=torch.int32).to(DEV)
    for off in (0, 1, 3):
        bins = store[off:off + nbins]
        arr = torch.zeros(nbins // 32 * nbits, dtype=torch.int32, device=DEV)
        capi.bins_to_bits(bins, arr, nbits)
        _eq("bins_to_bits", arr.cpu().numpy().view(np.uint32), oracle.bins_to_bits(bins.cpu().numpy(), nbits))


def test_quantization_compression(eden_utils):
    """values land on floor/ceil of t = clamp(v/div, +-max), unbiased in the mean"""
    n = 1 << 20
    v = (torch.rand(n, device=DEV) * 12.0 - 6.0)
    t = (v / 0.5).clamp(-10.0, 10.0)
    eden_utils.set_quantization_seed(123)
    q = v.clone()
    eden_utils.quantization_compression(q, 0.5, 10.0)
    assert bool(((q == t.floor()) | (q == t.floor() + 1)).all())
    assert abs(float((q - t).mean())) < 5e-3
    eden_utils.set_quantization_seed(123)
    q2 = v.clone()
    eden_utils.quantization_compression(q2, 0.5, 10.0)
    assert torch.equal(q, q2)
    q3 = v.clone()
    eden_utils.quantization_compression(q3, 0.5, 10.0)
    assert not torch.equal(q, q3)


@pytest.mark.parametrize("n", [1, 3, 4, 1021, 1 << 16])
def test_quantization_matches_oracle(capi, oracle, n):
    """dq_quantization against the oracle's restatement of cuda_hadamard.cu:607-627 on the same Philox stream"""
    g = torch.Generator().manual_seed(n)
    v = torch.rand(n, generator=g) * 30.0 - 15.0
    if n > 8:
        v[:8] = torch.tensor([0.0, 1.0, -1.0, 2.5, -2.5, 1e9, -1e9, float("inf")])
    for div, tmax, seed in ((0.5, 10.0, 123), (0.37, 100.0, 0xFEDCBA9876543210), (3.0, 0.5, 0)):
        q = v.clone().to(DEV)
        capi.quantization(q, div, tmax, seed)
        want = oracle.quantization(v.numpy(), div, tmax, seed)
        assert (q.cpu().numpy().view(np.uint32) == want.view(np.uint32)).all(), (n, div)
        # a view that starts 4 bytes into a buffer (the kernel then leaves its 16-byte accesses)
        buf = torch.full((n + 3,), 77.0, device=DEV)
        buf[1:n + 1] = v.to(DEV)
        capi.quantization(buf[1:n + 1], div, tmax, seed)
        assert (buf[1:n + 1].cpu().numpy().view(np.uint32) == want.view(np.uint32)).all(), (n, div, "unaligned")
        assert float(buf[0]) == 77.0 and bool((buf[n + 1:] == 77.0).all())


def test_quantization_compression_module_stream(eden_utils, oracle):
    """the module function draws seed, seed + golden ratio, ... from set_quantization_seed"""
    v = torch.rand(4096) * 12.0 - 6.0
    eden_utils.set_quantization_seed(123)
    for k in range(2):
        q = v.clone().to(DEV)
        eden_utils.quantization_compression(q, 0.5, 10.0)
        want = oracle.quantization(v.numpy(), 0.5, 10.0, (123 + k * 0x9E3779B97F4A7C15) & (2 ** 64 - 1))
        assert (q.cpu().numpy() == want).all()


@pytest.mark.parametrize("adt,bdt,run_bytes", [(torch.float32, torch.bfloat16, 584), (torch.bfloat16, torch.bfloat16, 328),
                                               (torch.bfloat16, None, 1096)])
def test_tile_io_floor_moves_exactly_the_bytes_of_the_codec_shape(capi, adt, bdt, run_bytes):
    """dq_tile_io_floor, the launch of the codec's shape without the arithmetic: every store carries the exclusive-or of all
    a lane loaded (so nothing it claims to read can be left out), it writes tiles * bytes per tile and not a byte more"""
    tiles = 37
    g = torch.Generator().manual_seed(run_bytes)
    a = torch.randn(1024 * tiles, generator=g).to(adt).to(DEV)
    b = torch.rand(1024 * tiles, generator=g).to(bdt).to(DEV) if bdt is not None else None
    run = torch.full((run_bytes * tiles + 64,), 0xAB, dtype=torch.uint8, device=DEV)

    def lane_words(t):          # [tiles, 64]: exclusive-or of the 32-bit words of each lane's chunk of 16 elements
        w = t.cpu().contiguous().view(torch.uint8).numpy().view(np.uint32).reshape(tiles, 64, -1)
        return np.bitwise_xor.reduce(w, axis=2)

    x = np.arange(64, dtype=np.uint32)[None, :] ^ lane_words(a)
    if b is not None:
        x = x ^ lane_words(b)
    capi.tile_io_floor(0, a, b, run, run_bytes, tiles)
    got = run.cpu().numpy()
    assert (got[run_bytes * tiles:] == 0xAB).all()
    pieces = got[:run_bytes * tiles].view(np.uint32).reshape(tiles, run_bytes // 8, 2)
    j = np.arange(run_bytes // 8)
    assert (pieces[:, :, 0] == x[:, j % 64]).all()
    assert (pieces[:, :, 1] == x[:, j % 64] + (j // 64).astype(np.uint32)[None, :]).all()

    # decoder shape: reads the run just written (and b), overwrites a
    y = np.broadcast_to(np.arange(64, dtype=np.uint32)[None, :], (tiles, 64)).copy()
    for jj in range(run_bytes // 8):
        y[:, jj % 64] ^= pieces[:, jj, 0] ^ pieces[:, jj, 1]
    if b is not None:
        y = y ^ lane_words(b)
    guard = torch.full((1024 * (tiles + 1),), 3.0, dtype=adt, device=DEV)
    capi.tile_io_floor(1, guard, b, run, run_bytes, tiles)
    out = guard.cpu().view(torch.uint8).numpy().view(np.uint32).reshape(tiles + 1, -1, 64, 4)   # 16-byte piece 64 k + lane
    k = np.arange(out.shape[1], dtype=np.uint32)[None, :, None]
    assert (out[:tiles, :, :, 0] == y[:, None, :]).all() and (out[:tiles, :, :, 1] == y[:, None, :] + 1).all()
    assert (out[:tiles, :, :, 2] == y[:, None, :] + 2).all() and (out[:tiles, :, :, 3] == y[:, None, :] + 3 + k).all()
    assert bool((guard[1024 * tiles:] == 3.0).all())
    with pytest.raises(ValueError):
        capi.tile_io_floor(0, a, b, run, run_bytes, tiles + 1)


@pytest.mark.parametrize("dt", [F16, BF16, F32])
@pytest.mark.parametrize("n", [8, 255, 256 * 9 + 5, 256 * 40 + 4])
def test_superchunk_add_mean_copy_alignments(capi, oracle, dt, n):
    """the 16-byte kernel of add_mean_copy (two-byte and four-byte elements), the kernel for what it leaves over, and views
    that are not 16-byte aligned give the oracle's bits and write nothing beyond n"""
    tdt = TORCH_DT[dt]
    g = torch.Generator().manual_seed(n)
    nsc = (n + 255) // 256
    res = (torch.randn(nsc * 256, generator=g) * 1e-2).to(tdt)
    stats = (torch.randn(nsc * 2, generator=g) * 1e-2).to(torch.bfloat16)
    want = oracle.superchunk_add_mean_copy(to_bits(res), to_bits(stats), n, dt)
    for shift_in, shift_out in ((0, 0), (1, 0), (0, 1), (4, 4)):
        rbuf = torch.zeros(nsc * 256 + 8, dtype=tdt, device=DEV)
        rview = rbuf[shift_in:shift_in + nsc * 256]
        rview.copy_(res)
        obuf = torch.full((n + 16,), 5.0, dtype=tdt, device=DEV)
        oview = obuf[shift_out:]
        capi.superchunk_add_mean_copy(rview, oview, stats.to(DEV), n)
        _eq("add_mean %d/%d" % (shift_in, shift_out), to_bits(oview[:n]), want)
        assert bool((oview[n:] == 5.0).all()) and bool((obuf[:shift_out] == 5.0).all())
