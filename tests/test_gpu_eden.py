"""EDEN Lloyd-Max quantiser / THC uniform quantiser kernels: bit-exact against the oracle; the host mirrors
against the reference's own outputs (tests/golden/eden_golden.npz) and the reference's torch op chains."""
import math
import os

import numpy as np
import pytest
import torch

from helpers import to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "eden_golden.npz"))


def _tables(nbits):
    return (torch.from_numpy(GOLD["centroids_%d" % nbits]).to(DEV), torch.from_numpy(GOLD["boundaries_%d" % nbits]).to(DEV))


@pytest.mark.parametrize("nbits", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("n", [32, 1024, 4096 * 3 + 64, 1 << 20])
def test_eden_quantize_bit_exact(capi, oracle, nbits, n):
    g = torch.Generator().manual_seed(n + nbits)
    x = torch.randn(n, generator=g) * 3e-3
    if n > 64:
        x[5] = 0.0
        x[7:40] *= 50.0                       # outliers beyond the last boundary
    cen, bnd = _tables(nbits)
    packed = torch.full((n // 32 * nbits,), -1, dtype=torch.int32, device=DEV)
    result = torch.zeros(4, device=DEV)
    work = torch.zeros(capi.eden_work_doubles(n), dtype=torch.float64, device=DEV)
    capi.eden_quantize(x.to(DEV), bnd, cen, nbits, packed, result, work)
    bins_o, res_o = oracle.eden_quantize(x.numpy(), GOLD["boundaries_%d" % nbits], GOLD["centroids_%d" % nbits], nbits)
    assert (result.cpu().numpy().view(np.uint32) == res_o.view(np.uint32)).all()
    assert (packed.cpu().numpy().view(np.uint32) == oracle.bins_to_bits(bins_o, nbits)).all()
    out = torch.zeros(n, device=DEV)
    capi.eden_dequantize(packed, n, cen, nbits, out)
    assert (out.cpu().numpy() == oracle.eden_dequantize(bins_o, GOLD["centroids_%d" % nbits])).all()


def test_eden_quantize_degenerate_norms(capi, oracle):
    """all zeros (0/0 -> NaN: torch.bucketize's lower bound sends it to the last bin) and a norm outside the fast-division range"""
    cen, bnd = _tables(4)
    for x in (torch.zeros(64), torch.full((64,), 1e-30), torch.full((64,), 3e18) * torch.randn(64).sign()):
        packed = torch.zeros(8, dtype=torch.int32, device=DEV)
        result = torch.zeros(4, device=DEV)
        work = torch.zeros(capi.eden_work_doubles(64), dtype=torch.float64, device=DEV)
        capi.eden_quantize(x.to(DEV), bnd, cen, 4, packed, result, work)
        bins_o, res_o = oracle.eden_quantize(x.numpy(), GOLD["boundaries_4"], GOLD["centroids_4"], 4)
        got, want = result.cpu().numpy(), res_o
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        assert same.all()
        assert (packed.cpu().numpy().view(np.uint32) == oracle.bins_to_bits(bins_o, 4)).all()


@pytest.mark.parametrize("case", [tuple(c) for c in GOLD["cases"]])
def test_eden_class_against_reference_outputs(capi, oracle, case):
    """Eden.compress / decompress with the reference's tables vs what the reference produced on the CPU"""
    from dynamiq_sigcomm_artifact_amd.eden import Eden
    dim, nbits, seed, nslices = (int(v) for v in case)
    cen = {nbits: torch.from_numpy(GOLD["centroids_%d" % nbits])}
    bnd = {nbits: torch.from_numpy(GOLD["boundaries_%d" % nbits])}
    eden = Eden(centroids=cen, boundaries=bnd, device=DEV)
    x = torch.from_numpy(GOLD["x_%d" % dim])
    data = eden.compress(x.to(DEV), nbits, seed)
    assert len(data) == nslices
    key = "%d_%d_%d" % (dim, nbits, seed)
    for k, d in enumerate(data):
        scale_g, orig_g, nh_g = GOLD["meta_%s_%d" % (key, k)]
        assert (d["orig_dim"], d["num_hadamard"], d["nbits"], d["seed"]) == (int(orig_g), int(nh_g), nbits, seed)
        bins = oracle.bits_to_bins(d["packed_bins"].cpu().numpy().view(np.uint32), nbits)
        bins_g = oracle.bits_to_bins(GOLD["packed_%s_%d" % (key, k)].view(np.uint32), nbits)
        assert (bins != bins_g).mean() <= 2e-3 and (np.abs(bins - bins_g) <= 1).all()
        assert abs(float(d["scale"]) - scale_g) <= 1e-4 * abs(scale_g)
    rec = eden.decompress(data).cpu()
    rec_g = torch.from_numpy(GOLD["rec_" + key])
    assert rec.shape == rec_g.shape and rec.dtype == x.dtype
    nmse = float(((rec - x) ** 2).sum() / (x ** 2).sum())
    nmse_g = float(((rec_g - x) ** 2).sum() / (x ** 2).sum())
    assert abs(nmse - nmse_g) <= 5e-3 * nmse_g
    assert float(((rec - rec_g) ** 2).sum() / (x ** 2).sum()) <= 2e-2 * nmse_g + 1e-9


def test_eden_class_own_tables_and_large_vector():
    """the computed Lloyd-Max tables give the textbook distortion D (with EDEN's unbiased scale ||x||^2 / <c, x> the
    NMSE is D / (1 - D)); a 2^22 vector goes through the multi-pass transform"""
    from dynamiq_sigcomm_artifact_amd.eden import Eden
    eden = Eden(device=DEV)
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(1 << 22, generator=g, device=DEV) * 1e-3
    from dynamiq_sigcomm_artifact_amd.eden import lloyd_max_normal, _conditional_means
    textbook = {1: 0.3634, 2: 0.1175, 4: 0.009497}     # Lloyd-Max distortion of N(0,1): Max (1960), tables I-II
    for nbits in (1, 2, 4, 8):
        c = lloyd_max_normal(nbits)
        # at the stationary point E[c(X) X] = E[c(X)^2], so D = 1 - E[c^2]; cell masses from the cdf
        from scipy.stats import norm
        b = np.concatenate(([-np.inf], (c[:-1] + c[1:]) / 2, [np.inf]))
        d = 1.0 - float(np.sum(c * c * (norm.cdf(b[1:]) - norm.cdf(b[:-1]))))
        if nbits in textbook:
            assert abs(d - textbook[nbits]) < 5e-5
        rec = eden.decompress(eden.compress(x, nbits, 7))
        nmse = float(((rec - x) ** 2).sum() / (x ** 2).sum())
        assert abs(nmse - d / (1 - d)) <= 0.02 * d, (nbits, nmse, d)
    odd = torch.randn(3000, generator=g, device=DEV).to(torch.bfloat16)
    rec = eden.decompress(eden.compress(odd, 4, 1))
    assert rec.dtype == torch.bfloat16 and rec.numel() == 3000
    assert float(((rec.float() - odd.float()) ** 2).sum() / (odd.float() ** 2).sum()) < 0.02


def _thc_torch_chain(rotated, lo, delta, levels, uniform):
    """thc_hooks.py:161-166 with bernoulli_(p) spelled (uniform < p)"""
    r = rotated.clone()
    r.sub_(lo).div_(delta)
    r.clamp_(min=0, max=levels - 1)
    floored = r.floor()
    probs = r.sub_(floored)
    floored.add_((uniform < probs).float())
    return floored.to(torch.bfloat16)


def test_thc_kernels_bit_exact(capi, oracle):
    n = 100003
    g = torch.Generator().manual_seed(2)
    rot = torch.randn(n, generator=g) * 0.01
    rot[3] = float("inf")
    rot[4] = float("-inf")
    rot[5] = float("nan")
    rot[6] = 0.0
    uni = torch.rand(n, generator=g)
    uni[::13] = 0.0
    max_norm = torch.tensor(0.3)
    lo = (-(3.2971933456919635 * max_norm / math.sqrt(1024))).reshape(1)
    for levels in (16, 31, 64):
        delta = ((-lo - lo) / (levels - 1) + 1e-23).reshape(1)
        out = torch.zeros(n, dtype=torch.bfloat16, device=DEV)
        capi.thc_quantize(rot.to(DEV), uni.to(DEV), out, lo.to(DEV), delta.to(DEV), levels)
        want = oracle.thc_quantize(rot.numpy(), uni.numpy(), float(lo), float(delta), levels)
        got = to_bits(out)
        nan = (got & 0x7fff) > 0x7f80
        assert ((got == want) | (nan & ((want & 0x7fff) > 0x7f80))).all()
        chain = _thc_torch_chain(rot.to(DEV), lo.to(DEV), delta.to(DEV), levels, uni.to(DEV))
        keep = ~torch.isnan(chain.float())
        assert torch.equal(out[keep], chain[keep])
        # decode: (sum of levels) * (delta / W) + lo
        step = (delta / 4).reshape(1)
        dec = torch.zeros(n, device=DEV)
        capi.thc_dequantize(out, dec, step.to(DEV), lo.to(DEV))
        want_d = oracle.thc_dequantize(want, float(step), float(lo))
        ok = (dec.cpu().numpy().view(np.uint32) == want_d.view(np.uint32)) | np.isnan(want_d)
        assert ok.all()
        ref = out.float().mul_(step.to(DEV)).add_(lo.to(DEV))
        assert torch.equal(dec[keep], ref[keep])


def test_thc_compressor_round_trip():
    from dynamiq_sigcomm_artifact_amd.thc import OldINCACudaHadamardCompressor
    size = 100000
    d = 1 << 17
    params = {"d": {(0, 0): d}, "size": {(0, 0): size}, "T": 3.2971933456919635, "nclients": 1, "rank": 0,
              "quantization_levels": 64, "device": DEV}
    comp = OldINCACudaHadamardCompressor(params)
    g = torch.Generator(device=DEV).manual_seed(1)
    x = (torch.randn(size, generator=g, device=DEV) * 1e-3).to(torch.bfloat16)
    norm = x.float().norm(2)
    levels = comp.compress(x, (0, 0), norm)
    assert levels.dtype == torch.bfloat16 and levels.numel() == d
    assert float(levels.float().min()) >= 0 and float(levels.float().max()) <= 63
    assert torch.equal(levels.float(), levels.float().round())
    rec = comp.decompress(levels, (0, 0), norm)
    assert rec.numel() == size
    nmse = float(((rec - x.float()) ** 2).sum() / (x.float() ** 2).sum())
    # per rotated coordinate (unit variance after scaling by sqrt(d)/||x||): uniform stochastic rounding with step
    # 2T/63 adds step^2/6, clipping at +-T adds E[(|z|-T)^2; |z|>T] = 2((1+T^2) Q(T) - T phi(T)); only size of the d
    # inverse-rotated coordinates are kept
    from scipy.stats import norm as gauss
    T = 3.2971933456919635
    expect = ((2 * T / 63) ** 2 / 6 + 2 * ((1 + T * T) * gauss.sf(T) - T * gauss.pdf(T))) * size / d
    assert abs(nmse - expect) < 0.03 * expect
    # the sum over two ranks decodes with delta / 2
    params2 = dict(params, nclients=2)
    c0, c1 = OldINCACudaHadamardCompressor(dict(params2, rank=0)), OldINCACudaHadamardCompressor(dict(params2, rank=1))
    y = (torch.randn(size, generator=g, device=DEV) * 1e-3).to(torch.bfloat16)
    big = torch.maximum(norm, y.float().norm(2))
    total = (c0.compress(x, (0, 0), big).float() + c1.compress(y, (0, 0), big).float()).to(torch.bfloat16)
    mean = c0.decompress(total, (0, 0), big)
    ref = (x.float() + y.float()) / 2
    assert float(((mean - ref) ** 2).sum() / (ref ** 2).sum()) < 0.02


def test_binding_functions(eden_utils, capi):
    n, nbits = 4096, 4
    cen, bnd = _tables(nbits)
    x = torch.randn(n, device=DEV) * 1e-3
    packed, result = eden_utils.eden_quantize(x, bnd, cen, nbits)
    packed2 = torch.empty_like(packed)
    result2 = torch.empty_like(result)
    capi.eden_quantize(x, bnd, cen, nbits, packed2, result2, torch.empty(capi.eden_work_doubles(n), dtype=torch.float64, device=DEV))
    assert torch.equal(packed, packed2) and torch.equal(result, result2)
    out = eden_utils.eden_dequantize(packed, cen, nbits)
    assert out.shape == (n,) and bool(torch.isin(out, cen).all())
    lo, delta = torch.tensor([-0.005], device=DEV), torch.tensor([0.01 / 63], device=DEV)
    u = torch.rand(n, device=DEV)
    lev = eden_utils.thc_quantize(x, u, lo, delta, 64)
    lev2 = torch.empty_like(lev)
    capi.thc_quantize(x, u, lev2, lo, delta, 64)
    assert torch.equal(lev, lev2)
    dec = torch.empty(n, device=DEV)
    eden_utils.thc_dequantize(lev, dec, delta, lo)
    assert float((dec - x).abs().max()) <= float(delta) * 1.01
    with pytest.raises(RuntimeError, match="vec size must be a positive multiple of 32"):
        eden_utils.eden_quantize(x[:100].contiguous(), bnd, cen, nbits)
    with pytest.raises(RuntimeError, match="boundaries must hold"):
        eden_utils.eden_quantize(x, bnd[:5].contiguous(), cen, nbits)


@pytest.mark.parametrize("n,block", [(64, 64), (1024, 1024), (1024, 64), (1 << 15, 1 << 15), (1 << 16, 1 << 16),
                                     (1 << 17, 1 << 17), (1 << 20, 1 << 20), (1 << 22, 1 << 22), (1 << 23, 1 << 23), (1 << 18, 1 << 12), (3 << 14, 1 << 14)])
def test_thc_quantiser_folded_into_the_transform(capi, n, block):
    """dq_thc_rht_quantize == rht_blocked + thc_quantize and dq_thc_dequantize_irht == thc_dequantize + inverse
    rht_blocked, bit for bit, for single-pass and multi-pass transforms"""
    g = torch.Generator().manual_seed(n + block)
    x = (torch.randn(n, generator=g) * 1e-2).to(DEV)
    sign = (torch.randint(0, 2, (n,), generator=g).float() * 2 - 1).to(DEV)
    uni = torch.rand(n, generator=g).to(DEV)
    scale = float(np.float32(1.0) / np.float32(np.sqrt(block)))
    norm = float(x.norm())
    T, levels = 2.5, 31
    hi = T * norm / np.sqrt(n)
    lo = torch.tensor([-hi], dtype=torch.float32, device=DEV)
    delta = torch.tensor([2 * hi / (levels - 1) + 1e-23], dtype=torch.float32, device=DEV)
    rot = x.clone()
    capi.rht_blocked(rot, sign, block, scale, False)
    want = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    capi.thc_quantize(rot, uni, want, lo, delta, levels)
    work = x.clone()
    got = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    capi.thc_rht_quantize(work, sign, uni, got, block, scale, lo, delta, levels)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert int(want.float().max()) <= levels - 1 and float(want.float().std()) > 1.0       # the quantiser did something
    # the way back, as after a direct sum over 4 ranks
    summed = (want.float() * 4).to(torch.bfloat16)
    step = delta / 4
    dec = torch.empty(n, device=DEV)
    capi.thc_dequantize(summed, dec, step, lo)
    capi.rht_blocked(dec, sign, block, scale, True)
    back = torch.full((n,), 7.0, device=DEV)
    capi.thc_dequantize_irht(summed, sign, back, block, scale, step, lo)
    assert torch.equal(back.view(torch.int32), dec.view(torch.int32))
    # the diagonal as packed bits: the same levels, the same vector back, the same rotation
    bits = capi.pack_signs(sign)
    work.copy_(x)
    got.zero_()
    capi.thc_rht_quantize(work, bits, uni, got, block, scale, lo, delta, levels)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    back.fill_(7.0)
    capi.thc_dequantize_irht(summed, bits, back, block, scale, step, lo)
    assert torch.equal(back.view(torch.int32), dec.view(torch.int32))
    rot2 = x.clone()
    capi.rht_blocked(rot2, bits, block, scale, False)
    assert torch.equal(rot2.view(torch.int32), rot.view(torch.int32))
    capi.rht_blocked(rot2, bits, block, scale, True)
    capi.rht_blocked(rot, sign, block, scale, True)
    assert torch.equal(rot2.view(torch.int32), rot.view(torch.int32))
    # buffers that are only element-aligned take the scalar paths
    if n <= 1 << 16:
        r3 = torch.zeros(n + 4, device=DEV)[1:1 + n].copy_(x)
        r4 = r3.clone()
        capi.rht_blocked(r3, bits, block, scale, False)
        capi.rht_blocked(r4, sign, block, scale, False)
        assert torch.equal(r3.view(torch.int32), r4.view(torch.int32))
        w2 = torch.zeros(n + 4, device=DEV)[1:1 + n].copy_(x)
        u2 = torch.zeros(n + 4, device=DEV)[3:3 + n].copy_(uni)
        g2 = torch.zeros(n + 4, dtype=torch.bfloat16, device=DEV)[1:1 + n]
        capi.thc_rht_quantize(w2, sign, u2, g2, block, scale, lo, delta, levels)
        assert torch.equal(g2.view(torch.int16), want.view(torch.int16))
        b2 = torch.zeros(n + 4, device=DEV)[1:1 + n]
        capi.thc_dequantize_irht(g2 * 4, sign, b2, block, scale, step, lo)
        assert torch.equal(b2.view(torch.int32), dec.view(torch.int32))


@pytest.mark.parametrize("nbits", [1, 3, 4, 8])
@pytest.mark.parametrize("n,block", [(32, 32), (96, 32), (1024, 1024), (4096 * 3, 4096), (1 << 15, 1 << 15), (1 << 16, 1 << 16),
                                     (1 << 17, 1 << 17), (1 << 20, 1 << 20), (1 << 22, 1 << 22), (1 << 23, 1 << 23), (1 << 18, 1 << 12)])
def test_eden_dequantiser_folded_into_the_inverse_transform(capi, nbits, n, block):
    """dq_eden_dequantize_irht == eden_dequantize, inverse rht_blocked, product with the scale -- bit for bit, single-pass
    and multi-pass transforms, float and packed diagonals, with and without the scale"""
    g = torch.Generator().manual_seed(n + nbits)
    cen, _ = _tables(nbits)
    bins = torch.randint(0, 1 << nbits, (n,), generator=g, dtype=torch.int32).to(DEV)
    packed = torch.empty(n // 32 * nbits, dtype=torch.int32, device=DEV)
    capi.bins_to_bits(bins, packed, nbits)
    sign = (torch.randint(0, 2, (n,), generator=g).float() * 2 - 1).to(DEV)
    scale = float(np.float32(1.0) / np.float32(np.sqrt(block)))
    eden_scale = torch.tensor([0.00123], dtype=torch.float32, device=DEV)
    want = torch.empty(n, device=DEV)
    capi.eden_dequantize(packed, n, cen, nbits, want)
    capi.rht_blocked(want, sign, block, scale, True)
    for sg in (sign, capi.pack_signs(sign), None):
        ref = want
        if sg is None:
            ref = torch.empty(n, device=DEV)
            capi.eden_dequantize(packed, n, cen, nbits, ref)
            capi.rht_blocked(ref, None, block, scale, True)
        got = torch.full((n + 8,), 7.0, device=DEV)
        capi.eden_dequantize_irht(packed, n, cen, nbits, sg, got[:n], block, scale)
        assert torch.equal(got[:n].view(torch.int32), ref.view(torch.int32)) and bool((got[n:] == 7.0).all())
        capi.eden_dequantize_irht(packed, n, cen, nbits, sg, got[:n], block, scale, post_scale=eden_scale)
        assert torch.equal(got[:n].view(torch.int32), (eden_scale * ref).view(torch.int32)) and bool((got[n:] == 7.0).all())


def test_srrcomp_utils_surface(capi, oracle):
    """the helpers srrcomp.Eden inherits from SRRCompUtils (srrcomp.py:13-167) and its _quantize (:356-361), as methods
    of the drop-in class: each equals the oracle's function or the entry point it wraps"""
    from dynamiq_sigcomm_artifact_amd.eden import Eden, SRRCompUtils
    eden = Eden(device=DEV)
    assert isinstance(eden, SRRCompUtils) and set(eden.utils) == {"cpu", "gpu"}
    assert set(eden.utils["gpu"]) == {"Hadamard", "BinsToBits", "BitsToBins"}
    with pytest.raises(Exception, match="Illegal gpuacctype"):
        SRRCompUtils("opencl")
    with pytest.raises(RuntimeError, match="device tensors only"):
        eden.utils["cpu"]["Hadamard"](torch.zeros(8))
    # randDiag: the integer hash of the reference; with torchRNG torch's own stream of +-1
    for size, seed in ((1000, 7), (4096, 123456789), (1, 0)):
        got = eden.randDiag(size, DEV, seed)
        assert got.dtype == torch.float32 and np.array_equal(got.cpu().numpy(), oracle.rand_diag(size, seed))
    coins = eden.randDiag(512, DEV, 5, torchRNG=True)
    assert set(coins.cpu().tolist()) == {-1.0, 1.0} and torch.equal(coins, eden.randDiag(512, DEV, 5, torchRNG=True))
    # Hadamard: in place, returns the flat view
    x = torch.randn(1 << 12, generator=torch.Generator().manual_seed(3))
    x_d = x.to(DEV).view(64, 64)
    y = eden.Hadamard(x_d)
    assert y.data_ptr() == x_d.data_ptr() and np.array_equal(y.cpu().numpy(), oracle.fwht(x.numpy()))
    with pytest.raises(Exception, match="power of 2"):
        eden.Hadamard(torch.zeros(12, device=DEV))
    # the packers take the int64 bins of torch.bucketize
    bins = torch.randint(0, 32, (4096,), generator=torch.Generator().manual_seed(4))
    bits = eden.EdenBinsToBits(bins.to(DEV), 5)
    assert bits.dtype == torch.int32 and np.array_equal(bits.cpu().numpy().view(np.uint32), oracle.bins_to_bits(bins.numpy().astype(np.int32), 5).view(np.uint32))
    assert torch.equal(eden.EdenBitsToBins(bits, 5).cpu(), bins.to(torch.int32))
    # _quantize: the bins and the scale of eden_quantize
    n, nbits = 8192, 4
    v = torch.randn(n, generator=torch.Generator().manual_seed(6)).to(DEV)
    q_bins, scale = eden._quantize(v, nbits)
    cen, bnd = eden._tables(nbits)
    packed = torch.empty(n // 32 * nbits, dtype=torch.int32, device=DEV)
    result = torch.empty(4, dtype=torch.float32, device=DEV)
    capi.eden_quantize(v, bnd, cen, nbits, packed, result, torch.empty(capi.eden_work_doubles(n), dtype=torch.float64, device=DEV))
    assert q_bins.dtype == torch.int64 and torch.equal(eden.EdenBinsToBits(q_bins, nbits), packed)
    assert float(scale) == float(result[2])
    # against torch's own ops away from the boundaries: at most a handful of bins differ by the rounding of the quotient
    ref = torch.bucketize(v * (n ** 0.5) / torch.norm(v, 2), bnd)
    assert int((ref != q_bins).sum()) <= 2
