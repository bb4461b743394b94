"""dq_group_plan_sorted (the fixed-proportion allocation of comm_hooks.py:710-721 as one launch) against
torch.argsort(descending=True, stable=True) on the device and against the oracle; the groups feed the row-list
codec, whose bytes are compared with the gather -> codec sequence the hook runs."""
import numpy as np
import pytest
import torch

from helpers import to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


EXOTIC = "NaN of either sign, -0"


def _stats(norms):
    st = torch.zeros((norms.numel(), 2), dtype=torch.bfloat16, device=DEV)
    st[:, 1] = norms.to(DEV)
    st[:, 0] = 0.25
    return st


def _norm_sets():
    g = torch.Generator().manual_seed(21)
    sets = {
        "bucket 25600 lognormal": torch.exp(torch.randn(25600, generator=g) * 3 - 8),
        "tie-heavy 25600 (12 values)": torch.exp2(torch.randint(-6, 6, (25600,), generator=g).float()),
        "all equal 4097": torch.full((4097,), 0.125),
        "all zero 25600": torch.zeros(25600),
        "one": torch.tensor([3.0]),
        "255": torch.exp(torch.randn(255, generator=g)),
        "256": torch.exp(torch.randn(256, generator=g)),
        "257": torch.exp(torch.randn(257, generator=g)),
        "65535 narrow": torch.rand(65535, generator=g) * 1e-4 + 2e-4,
        # more than one round of loads per thread with keys of either sign (the two-counters-per-word layout)
        "40001 of either sign": torch.randn(40001, generator=g) * torch.exp(torch.randn(40001, generator=g)),
    }
    sp = torch.exp(torch.randn(30011, generator=g) * 4 - 5)
    sp[::7] = 0.0
    sp[3::11] = -0.0
    sp[1::97] = float("nan")
    sp[2::131] = -1.0
    sp[5::173] = float("inf")
    sp[6::191] = float("-inf")
    sets["zeros, NaN, infinities, negatives"] = sp
    sets = {k: v.to(torch.bfloat16) for k, v in sets.items()}
    # torch documents NaN as the greatest value and equal values as ties; its CPU sort and its small device sort behave
    # so.  Its large device sort is a radix sort on the bit pattern: NaNs order by payload, a NaN with the sign bit set
    # (what the CPU's float -> bf16 conversion writes: 0xffff) goes behind -inf, and -0 may be told from +0.  The library
    # follows the documented order.  The comparison with torch on the device therefore uses one NaN pattern (0x7fc0,
    # what device arithmetic produces) and +0 only; NaNs of either sign and payload and -0 are compared with the oracle
    # (EXOTIC), which is pinned by torch's CPU sort.
    bits = sets["zeros, NaN, infinities, negatives"].view(torch.int16)
    exotic = bits.clone()
    bits[1::97] = 0x7fc0
    bits[3::11] = 0
    exotic[1::97] = torch.tensor(0xffff - 0x10000, dtype=torch.int16)
    exotic[98::194] = 0x7fff
    exotic[1::291] = 0x7fc0
    sets[EXOTIC] = exotic.view(torch.bfloat16)
    return sets


@pytest.mark.parametrize("name", sorted(_norm_sets()))
@pytest.mark.parametrize("method", ["x_5bit", "x_3bit", "x_4bit_fixed", "x_7bit"])
def test_sorted_plan_matches_argsort(capi, oracle, name, method):
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    norms = _norm_sets()[name]
    nsc = norms.numel()
    st = _stats(norms)
    thr = B.fixed_proportion_thresholds(method)
    top, mid, bottom = B.fixed_proportion_counts(nsc, thr)
    order = torch.full((3 * nsc,), -7, dtype=torch.int32, device=DEV)
    work = torch.full((capi.group_plan_work_ints(nsc),), -7, dtype=torch.int32, device=DEV)
    qb = torch.zeros(nsc, dtype=torch.int64, device=DEV)
    capi.group_plan_sorted(st, top, bottom, order, work, qbits_out=qb)
    o = order.cpu().numpy()
    assert work[:4].tolist() == [top, mid, bottom, 0]
    # the reference's own ops on the device (comm_hooks.py:710-721)
    g8, g4, g2 = B.fixed_proportion_groups(st[:, 1], thr)
    # and the oracle
    o8, o4, o2 = oracle.fixed_proportion_groups(to_bits(st.reshape(-1))[1:], top, bottom, stride=2)
    for base, cnt, g, og in ((0, top, g8, o8), (nsc, mid, g4, o4), (2 * nsc, bottom, g2, o2)):
        assert (o[base:base + cnt] == og).all(), (name, method, base)
        if name != EXOTIC:
            assert (o[base:base + cnt] == g.cpu().numpy()).all(), (name, method, base)
        assert (o[base + cnt:base + nsc] == -7).all()                      # nothing written beyond a list
    want_q = np.zeros(nsc, np.int64)
    want_q[o8], want_q[o4], want_q[o2] = 8, 4, 2
    assert (qb.cpu().numpy() == want_q).all()


def test_sorted_plan_wrapper_and_module(capi, eden_utils):
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    g = torch.Generator().manual_seed(5)
    st = _stats(torch.exp(torch.randn(1000, generator=g)).to(torch.bfloat16))
    thr = B.fixed_proportion_thresholds("dynamiQ_mee_5bit")
    order, work, counts = B.fixed_proportion_plan(st, thr)
    assert counts == (350, 450, 200) and work[:3].tolist() == [350, 450, 200]
    order2 = torch.zeros_like(order)
    w2 = eden_utils.group_plan_sorted(st, 350, 200, order2)
    assert w2.tolist() == [350, 450, 200, 0]
    for base, cnt in ((0, 350), (1000, 450), (2000, 200)):
        assert torch.equal(order[base:base + cnt], order2[base:base + cnt])
    srt = torch.argsort(st[:, 1].float(), descending=True, stable=True)
    assert torch.equal(order[:350].long(), srt[:350])


def test_sorted_plan_validation(capi):
    st = _stats(torch.ones(70000).to(torch.bfloat16))
    order = torch.zeros(3 * 70000, dtype=torch.int32, device=DEV)
    work = torch.zeros(64, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="work buffer is too small"):
        capi.group_plan_sorted(st, 10, 10, order, work)
    with pytest.raises(RuntimeError, match="top_count"):
        capi.group_plan_sorted(st[:100], 60, 60, order, work)
    with pytest.raises(RuntimeError, match="4-byte aligned"):
        capi.group_plan_sorted(st.reshape(-1)[1:201].reshape(100, 2), 10, 10, order, work)
    torch.cuda.synchronize()


@pytest.mark.parametrize("strategy", [2, 3])
@pytest.mark.parametrize("widths", [(8, 4, 2), (7, 5, 3)])
def test_groups_feed_the_row_codec(capi, oracle, strategy, widths):
    """one bucket end to end as the fixed-proportion hook runs it (one rank): groups in sorted order -> index_select ->
    compress (rand rows paired with the position in the group) -> decompress -> index_copy_, against the row-list
    kernels fed by the device plan; with the hook's widths and with the extension widths 7 / 5 / 3 in their place"""
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    nsc = 1200
    g = torch.Generator().manual_seed(8)
    scale = torch.exp(torch.randn(nsc, 1, generator=g) * 2 - 4)
    x = (torch.randn(nsc, 256, generator=g) * scale).to(torch.bfloat16).to(DEV)
    st = _stats((x.float() ** 2).sum(1).to(torch.bfloat16))
    thr = B.fixed_proportion_thresholds("m_5bit")
    order, work, counts = B.fixed_proportion_plan(st, thr)
    groups = B.fixed_proportion_groups(st[:, 1], thr)
    out = torch.zeros_like(x)
    want = torch.zeros_like(x)
    for width, base, cnt, idx in ((widths[0], 0, counts[0], groups[0]), (widths[1], nsc, counts[1], groups[1]),
                                  (widths[2], 2 * nsc, counts[2], groups[2])):
        rand = torch.rand(cnt * 256, generator=g).to(torch.bfloat16).to(DEV)
        nbytes = capi.required_bytes(cnt * 256, width, 16, strategy)
        # the hook's sequence, through the oracle
        gathered = torch.index_select(x, 0, idx).reshape(-1)
        packed_o = oracle.scaling_compress(to_bits(gathered), to_bits(rand), cnt * 256, width, 16, strategy, 1)
        dec = np.zeros(cnt * 256, np.uint16)
        oracle.scaling_decompress(packed_o, dec, cnt * 256, width, 16, strategy, 1)
        want.index_copy_(0, idx, torch.from_numpy(dec.view(np.int16)).view(torch.bfloat16).reshape(cnt, 256).to(DEV))
        # the library: no gather, rows from the plan
        rows = order[base:base + cnt]
        packed = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        capi.scaling_compress_rows(x.reshape(-1), rows, packed, rand, cnt, width, strategy)
        assert (packed.cpu().numpy() == packed_o[:nbytes]).all(), width
        capi.scaling_decompress_rows(packed, out.reshape(-1), rows, None, nsc * 256, cnt, width, strategy)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("W", [1, 2, 3])
@pytest.mark.parametrize("method,cls", [("dynamiQ_aee_5bit", "aee"), ("dynamiQ_mee_3bit", "mee"), ("dynamiQ_mee_4bit_fixed", "mee")])
def test_fixed_proportion_allreduce_device_plan_equals_op_sequence(capi, W, method, cls):
    """the whole partition of the non-dynamic hook: sort / slice / index_select / ring / index_copy_ / add-mean as the
    reference runs it against one plan launch + row-list codec calls; same random rows, so the outputs are bit-equal"""
    import types
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    from dynamiq_sigcomm_artifact_amd.compressors import Aee_Dynamic_Range_GPU_kern, Mee_Dynamic_Range_GPU_kern
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import fixed_proportion_allreduce, fixed_proportion_allreduce_grouped
    K = Aee_Dynamic_Range_GPU_kern if cls == "aee" else Mee_Dynamic_Range_GPU_kern
    # a ragged tail; one case beyond the one-launch plan (70,001 superchunks: the radix-sort path)
    n = 256 * 70000 + 77 if (W == 1 and method == "dynamiQ_aee_5bit") else 256 * 700 + 77
    g = torch.Generator().manual_seed(31 + W)
    scale = torch.exp(torch.randn((n + 255) // 256, generator=g) * 2 - 5).repeat_interleave(256)[:n]
    vecs = [(torch.randn(n, generator=g) * scale + 1e-3).to(torch.bfloat16).to(DEV) for _ in range(W)]
    thr = B.fixed_proportion_thresholds(method)
    fixed = "fixed" in method

    def comps():
        gen = torch.Generator(device=DEV).manual_seed(5)
        params = lambda r: {"d": {(0, 0): n + 256}, "world_size": W, "rank": r, "args": types.SimpleNamespace(aggregation_method=method)}
        return {q: [K(q, 16, params(r), generator=gen) for r in range(W)] for q in (8, 4, 2)}

    ref, total, idx = fixed_proportion_allreduce([v.clone() for v in vecs], thr, comps(), fixed_4bit_only=fixed)
    out, total2, order, counts = fixed_proportion_allreduce_grouped([v.clone() for v in vecs], thr, comps(), fixed_4bit_only=fixed)
    assert torch.equal(total.view(torch.int16), total2.view(torch.int16))
    nsc = (n + 255) // 256
    for gi, (cnt, ix) in enumerate(zip(counts, idx)):
        assert torch.equal(order[gi * nsc:gi * nsc + cnt].long(), ix)
    for a, b in zip(ref, out):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for r in range(1, W):
        assert torch.equal(out[0], out[r])
    exact = sum(v.double() for v in vecs) / W
    nmse = float(((out[0].double() - exact) ** 2).sum() / (exact ** 2).sum())
    assert nmse < 0.2


@pytest.mark.parametrize("nsc", [65536, 100_003, 1_000_000, 7_812_500])
@pytest.mark.parametrize("method", ["x_5bit", "x_3bit"])
def test_sorted_plan_of_a_long_bucket(capi, oracle, nsc, method):
    """Buckets beyond the one-launch plan (the reference trains with a 4000 MB DDP bucket cap: millions of superchunks)
    go through the radix sort in the work buffer: the same three lists as the oracle's stable descending sort, NaN first,
    ties by index; 7,812,500 superchunks = 2 * 10^9 elements."""
    from dynamiq_sigcomm_artifact_amd import bitrate
    g = torch.Generator().manual_seed(nsc)
    norms = torch.exp(torch.randn(nsc, generator=g) * 3 - 8)
    norms[::1001] = 0.0
    norms[5::20011] = float("nan")
    norms[7::30011] = float("inf")
    if nsc == 100_003:                         # patterns a sum of squares never takes
        norms[3::997] = -1.5
        norms[11::4999] = -0.0
    norms = norms.to(torch.bfloat16)
    bits = norms.view(torch.int16)
    bits[5::20011] = 0x7fc0
    stats = torch.zeros((nsc, 2), dtype=torch.bfloat16)
    stats[:, 1] = norms
    stats[:, 0] = 0.25
    stats_d = stats.to(DEV)
    thr = bitrate.fixed_proportion_thresholds(method)
    order, work, (n8, n4, n2) = bitrate.fixed_proportion_plan(stats_d, thr)
    assert work[:4].tolist() == [n8, n4, n2, 0]
    want = oracle.argsort_descending_stable(norms.view(torch.int16).numpy().view(np.uint16))
    o = order.cpu().numpy()
    assert np.array_equal(o[:n8], want[:n8]), "8-bit list"
    assert np.array_equal(o[nsc:nsc + n4], want[n8:n8 + n4]), "4-bit list"
    assert np.array_equal(o[2 * nsc:2 * nsc + n2], want[n8 + n4:]), "2-bit list"
    # the widths, and a second call into the same buffers
    qb = torch.zeros(nsc, dtype=torch.int64, device=DEV)
    capi.group_plan_sorted(stats_d, n8, n2, order, work, qbits_out=qb)
    q = qb.cpu().numpy()
    assert (q[want[:n8]] == 8).all() and (q[want[n8:n8 + n4]] == 4).all() and (q[want[n8 + n4:]] == 2).all()
    assert np.array_equal(order.cpu().numpy()[:n8], want[:n8])
