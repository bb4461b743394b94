"""Every added function of the eden_utils module once, against the same call through ctypes: catches a wrong argument
order or a wrong size check in the binding layer (the kernels themselves are covered through the C ABI elsewhere)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bits_t(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def test_plan_and_mixed_bindings(capi, eden_utils):
    eu = eden_utils
    nsc, n = 300, 300 * 256 - 40
    g = torch.Generator().manual_seed(1)
    scales = torch.exp(torch.randn(nsc, 1, generator=g) * 6.0) * 1e-3
    src = (torch.randn(nsc, 256, generator=g) * scales).reshape(-1)[:n].to(torch.bfloat16).to(DEV)
    stats_a = torch.zeros(nsc, 2, dtype=torch.bfloat16, device=DEV)
    stats_b = torch.zeros_like(stats_a)
    mean_a, mean_b = torch.zeros(nsc, device=DEV), torch.zeros(nsc, device=DEV)
    capi.superchunk_stats(src, stats_a, mean_a, n, 2)
    eu.superchunk_stats(src, stats_b, mean_b, n, 2)
    assert torch.equal(bits_t(stats_a), bits_t(stats_b)) and torch.equal(mean_a, mean_b)

    order_a = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    order_b = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    q_a = torch.zeros(nsc, dtype=torch.int64, device=DEV)
    q_b = torch.zeros(nsc, dtype=torch.int64, device=DEV)
    capi.group_plan_stats(stats_a, 7.1, q_a, order_a, work)
    counts = eu.group_plan_stats(stats_b, 7.1, order_b, q_b)
    assert counts.tolist() == work[:4].tolist() and min(counts.tolist()[:3]) > 0
    assert torch.equal(order_a, order_b) and torch.equal(q_a, q_b)
    order_c = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    assert eu.group_plan(q_b, order_c).tolist() == counts.tolist() and torch.equal(order_c, order_a)

    cap = capi.mixed_required_bytes(nsc, 2)
    assert eu.mixed_required_bytes(nsc, 2) == cap
    pool = torch.rand(nsc * 256, generator=g).to(torch.bfloat16).to(DEV)
    for kw in (dict(rand_pool=pool), dict(seed=5, step=2)):
        a = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        b = torch.zeros(cap, dtype=torch.uint8, device=DEV)
        capi.mixed_compress(src, order_a, work, a, nsc, 3, center_mean=mean_a, center_world=2, n=n, ring_chunk=1,
                            ring_world=2, **kw)
        eu.mixed_compress(src, order_a, counts, b, nsc, center_mean=mean_a, center_world=2, n=n, ring_chunk=1, ring_world=2,
                          strategy=3, **kw)
        assert torch.equal(a, b) and int(a.max()) > 0
        a2, b2 = torch.zeros_like(a), torch.zeros_like(a)
        capi.mixed_compress(src, order_a, work, a2, nsc, 3, recv=a, center_mean=mean_a, center_world=2, n=n, ring_chunk=1,
                            ring_world=2, **kw)
        eu.mixed_compress(src, order_a, counts, b2, nsc, recv=a, center_mean=mean_a, center_world=2, n=n, ring_chunk=1,
                          ring_world=2, strategy=3, **kw)
        assert torch.equal(a2, b2) and not torch.equal(a2, a)
    out_a = torch.full((n,), 3.0, dtype=torch.bfloat16, device=DEV)
    out_b = torch.full((n,), 3.0, dtype=torch.bfloat16, device=DEV)
    capi.mixed_decompress(a2, out_a, order_a, work, nsc, 3, stats=stats_a, n_limit=n, ring_chunk=1, ring_world=2)
    eu.mixed_decompress(a2, out_b, order_a, counts, nsc, stats_a, n, ring_chunk=1, ring_world=2, strategy=3)
    assert torch.equal(bits_t(out_a), bits_t(out_b)) and bool((out_a != 3.0).any())
    with pytest.raises(RuntimeError, match="3 \\* nsc"):
        eu.group_plan(q_b, torch.zeros(nsc, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="mixed_required_bytes"):
        eu.mixed_compress(src, order_a, counts, torch.zeros(16, dtype=torch.uint8, device=DEV), nsc, seed=1)


def test_offset_search_bindings(capi, eden_utils):
    eu = eden_utils
    g = torch.Generator().manual_seed(4)
    stats = torch.zeros(5000, 2, dtype=torch.bfloat16, device=DEV)
    stats[:, 1] = torch.exp(torch.randn(5000, generator=g) * 4 - 6).to(torch.bfloat16).to(DEV)
    assert eu.bitrate_hist_ints() == capi.bitrate_hist_ints()
    ha = torch.zeros(capi.bitrate_hist_ints(), dtype=torch.int32, device=DEV)
    hb = torch.zeros_like(ha)
    for mode, prev in ((0, 60.0), (1, 3.0)):
        capi.norm_histogram(stats, ha)
        eu.norm_histogram(stats, hb)
        assert torch.equal(ha, hb) and int(ha.sum()) == 5000
        ra = torch.zeros(4, dtype=torch.float64, device=DEV)
        capi.bitrate_search(ha, mode, prev, 4.375, ra)
        rb = eu.bitrate_search(hb, mode, prev, 4.375)
        assert ra.tolist() == rb.tolist() and int(hb.abs().sum()) == 0
    # the plan with the offset left on the device
    nsc = 5000
    order_a = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    order_b = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    capi.group_plan_stats(stats, rb[0:1], None, order_a, work)
    counts = eu.group_plan_stats_dev_u(stats, rb[0:1], order_b)
    assert counts.tolist() == work[:4].tolist() and torch.equal(order_a, order_b)
    capi.norm_histogram(stats, ha)
    assert eu.group_plan_stats_dev_u(stats, rb[0:1], order_b, None, hb).tolist() == counts.tolist() and torch.equal(ha, hb)
    ha.zero_()
    hb.zero_()
    with pytest.raises(RuntimeError, match="float64"):
        eu.group_plan_stats_dev_u(stats, rb[0:1].float(), order_b)
    with pytest.raises(RuntimeError, match="bitrate_hist_ints"):
        eu.norm_histogram(stats, torch.zeros(100, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="mode must be"):
        eu.bitrate_search(hb, 2, 0.0, 4.0)


def test_transform_bindings(capi, eden_utils):
    eu = eden_utils
    n, block, nbits = 8192 * 2, 2048, 5
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(n, generator=g) * 1e-3).to(DEV)
    sign = (torch.randint(0, 2, (n,), generator=g).float() * 2 - 1).to(DEV)
    pool = torch.rand(n, generator=g).to(torch.bfloat16).to(DEV)
    scale = 1.0 / math.sqrt(block)
    bits_a, bits_b = capi.pack_signs(sign), eu.pack_signs(sign)
    assert torch.equal(bits_a, bits_b)
    nb = capi.required_bytes(n, nbits, 16, 3)
    for sg in (sign, bits_a, None):
        for kw in (dict(rand_pool=pool), dict(seed=3, step=4)):
            a = torch.zeros(nb, dtype=torch.uint8, device=DEV)
            b = torch.zeros(nb, dtype=torch.uint8, device=DEV)
            capi.rht_scaling_compress(x, sg, a, block, scale, nbits, 3, **kw)
            eu.rht_scaling_compress(x, sg, b, block, scale, nbits, strategy=3, **kw)
            assert torch.equal(a, b)
        ya, yb = torch.empty(n, device=DEV), torch.empty(n, device=DEV)
        capi.scaling_decompress_irht(a, sg, ya, block, scale, nbits, 3)
        eu.scaling_decompress_irht(a, sg, yb, block, scale, nbits, strategy=3)
        assert torch.equal(ya, yb)
    # THC
    uni = torch.rand(n, generator=g).to(DEV)
    lo = torch.tensor([-4e-3], device=DEV)
    delta = torch.tensor([8e-3 / 30], device=DEV)
    la = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    lb = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    capi.thc_rht_quantize(x.clone(), sign, uni, la, n, 1.0 / math.sqrt(n), lo, delta, 31)
    eu.thc_rht_quantize(x.clone(), sign, uni, lb, n, 1.0 / math.sqrt(n), lo, delta, 31)
    assert torch.equal(bits_t(la), bits_t(lb)) and float(la.float().std()) > 1.0
    ra, rb = torch.empty(n, device=DEV), torch.empty(n, device=DEV)
    capi.thc_dequantize_irht(la, sign, ra, n, 1.0 / math.sqrt(n), delta, lo)
    eu.thc_dequantize_irht(la, sign, rb, n, 1.0 / math.sqrt(n), delta, lo)
    assert torch.equal(ra, rb)
    assert float((ra - x).pow(2).sum() / x.pow(2).sum()) < 0.05
    # the diagonal as bits through the module: same levels, same vector back, same rotation; the seeded diagonal as bits
    eu.thc_rht_quantize(x.clone(), bits_a, uni, lb.zero_(), n, 1.0 / math.sqrt(n), lo, delta, 31)
    assert torch.equal(bits_t(la), bits_t(lb))
    eu.thc_dequantize_irht(la, bits_a, rb.zero_(), n, 1.0 / math.sqrt(n), delta, lo)
    assert torch.equal(ra, rb)
    assert torch.equal(eu.rht_blocked(x.clone(), bits_a, block, scale, False), eu.rht_blocked(x.clone(), sign, block, scale, False))
    assert torch.equal(eu.rand_diag_bits(n, 5, x.device), capi.pack_signs(eu.rand_diag(n, 5, x.device)))
    # EDEN's dequantiser folded into the inverse rotation
    from dynamiq_sigcomm_artifact_amd.eden import normal_centroids_and_boundaries
    cen = normal_centroids_and_boundaries(4)[0].to(DEV)
    pk = torch.randint(-2 ** 31, 2 ** 31 - 1, (n // 32 * 4,), generator=g, dtype=torch.int32).to(DEV)
    es = torch.tensor([0.5], device=DEV)
    oa = torch.empty(n, device=DEV)
    capi.eden_dequantize_irht(pk, n, cen, 4, bits_a, oa, n, 1.0 / math.sqrt(n), post_scale=es)
    assert torch.equal(oa, eu.eden_dequantize_irht(pk, cen, 4, bits_a, n, 1.0 / math.sqrt(n), es))
    with pytest.raises(RuntimeError, match="multiple of 256"):
        eu.rand_diag_bits(100, 5, x.device)
