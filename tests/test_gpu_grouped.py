"""The codec over lists of superchunk indices (gather / scatter / mean add folded into the kernels)
against what it replaces: torch.nonzero, index_select + codec + index_copy_, superchunk_add_mean_copy
(testbed_evaluation/new_comm_hooks/comm_hooks.py:963-1019) -- byte for byte."""
import math
import types

import numpy as np
import pytest
import torch

from helpers import BF16, F32, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("nsc", [1, 5, 1023, 1024, 1025, 4096, 4097, 25600, 65535, 65536, 65537, 300001])
def test_group_plan_matches_nonzero(capi, nsc):
    g = torch.Generator().manual_seed(nsc)
    q = torch.tensor([2, 4, 8, 16])[torch.randint(0, 4 if nsc > 5 else 3, (nsc,), generator=g)].to(DEV)
    if nsc == 1023:
        q[:] = 8            # a single group
    if nsc in (25600, 65536):
        # widths that are none of 2, 4, 8 in every form: zero, odd, negative, and values whose low half reads 8, 4 or 2
        odd = torch.tensor([0, 1, 3, -8, (1 << 32) + 8, (5 << 32) + 4, -(1 << 40) + 2, 1 << 62], device=DEV)
        q[torch.randperm(nsc, generator=g)[:64].to(DEV)] = odd.repeat(8)
        q = q.view(-1)
    order = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    for rep in range(3):        # the same work buffer serves call after call
        if rep:
            q = q.roll(rep * 37 + 1)
            order.fill_(-1)
        capi.group_plan(q, order, work)
        counts = work[:4].tolist()
        want = [torch.nonzero(q == w).view(-1) for w in (8, 4, 2)]
        assert counts[:3] == [w.numel() for w in want] and counts[3] == nsc - sum(w.numel() for w in want)
        for g in range(3):      # one region of nsc entries per width; nothing written beyond a group
            region = order[g * nsc:(g + 1) * nsc].cpu()
            assert torch.equal(region[:counts[g]], want[g].cpu().to(torch.int32))
            assert bool((region[counts[g]:] == -1).all())


def test_group_plan_stats_all_bf16_norms(capi, oracle):
    """widths computed in the kernel == the oracle's restatement of the allocation rule for EVERY bf16 norm
    pattern and a sweep of offsets; torch's own op sequence on the device agrees as well"""
    from dynamiq_sigcomm_artifact_amd import bitrate
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    norms = pats.view(torch.bfloat16)
    nsc = norms.numel()
    stats = torch.zeros(nsc, 2, dtype=torch.bfloat16)
    stats[:, 1] = norms
    stats_d = stats.to(DEV)
    order = torch.empty(3 * nsc, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    qout = torch.empty(nsc, dtype=torch.int64, device=DEV)
    finite = torch.isfinite(norms.float())
    for u in (-10.0, 0.0, 3.3, 7.25, 10.38818359375, 11.0, 13.7, 25.0, 60.0):
        capi.group_plan_stats(stats_d, u, qout, order, work)
        want = oracle.dynamic_bitrate_qbits(to_bits(norms), u)
        got = qout.cpu().numpy()
        assert (got == want).all(), (u, np.nonzero(got != want)[0][:10], got[got != want][:10], want[got != want][:10])
        counts = work[:4].tolist()
        assert counts == [int((want == 8).sum()), int((want == 4).sum()), int((want == 2).sum()), 0]
        order_h = order.cpu().numpy()
        for g, w in enumerate((8, 4, 2)):
            idx = np.nonzero(want == w)[0]
            assert (order_h[g * nsc:g * nsc + idx.size] == idx).all()
        t = bitrate.dynamic_bitrate_qbits(stats_d[:, 1], u).cpu()
        assert int((t[finite] != qout.cpu()[finite]).sum()) == 0, u


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("nbits,strategy", [(2, 2), (4, 2), (8, 3), (5, 3)])
def test_rows_entry_points_match_gather_codec_scatter(capi, dt, nbits, strategy):
    nsc, n_valid = 1037, 1037 * 256 - 77
    g = torch.Generator().manual_seed(nbits * 7 + strategy)
    full = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
    peer = (torch.randn(nsc * 256, generator=g) * 1e-2).to(dt).to(DEV)
    stats = torch.randn(nsc, 2, generator=g).mul(1e-2).to(torch.bfloat16).to(DEV)
    rows = torch.randperm(nsc, generator=g)[:701].sort().values.to(torch.int32).to(DEV)
    nrows = rows.numel()
    rnd = torch.rand(nrows * 256, generator=g).to(torch.bfloat16).to(DEV)
    if dt == torch.float32 and nbits == 2:
        rnd = rnd.float()       # same-dtype pool as well as the mixed one
    nbytes = capi.required_bytes(nrows * 256, nbits, 16, strategy)
    idx = rows.long()

    # reference sequence
    grp = full.view(-1, 256).index_select(0, idx).reshape(-1).contiguous()
    enc_ref = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    capi.scaling_compress(grp, enc_ref, rnd, nrows * 256, nbits, 16, strategy)
    grp2 = peer.view(-1, 256).index_select(0, idx).reshape(-1).contiguous()
    send_ref = torch.zeros_like(enc_ref)
    capi.scaling_dec_comp(enc_ref, grp2, send_ref, rnd, nrows * 256, nbits, 16, strategy)
    dec = torch.empty_like(grp)
    capi.scaling_decompress(send_ref, dec, nrows * 256, nbits, 16, strategy)
    res = torch.zeros_like(full)
    res.view(-1, 256).index_copy_(0, idx, dec.view(-1, 256))
    out_ref = torch.full((n_valid,), 7.0, dtype=dt, device=DEV)
    capi.superchunk_add_mean_copy(res, out_ref, stats, n_valid)

    # folded
    enc = torch.zeros_like(enc_ref)
    capi.scaling_compress_rows(full, rows, enc, rnd, nrows, nbits, strategy)
    assert torch.equal(enc, enc_ref)
    send = torch.zeros_like(enc_ref)
    peer_before = peer.clone()
    capi.scaling_dec_comp_rows(enc, peer, rows, send, rnd, nrows, nbits, strategy)
    assert torch.equal(send, send_ref) and torch.equal(peer, peer_before)
    out = torch.full((n_valid + 300,), 7.0, dtype=dt, device=DEV)
    capi.scaling_decompress_rows(send, out, rows, stats, n_valid, nrows, nbits, strategy)
    sel = torch.zeros(nsc * 256, dtype=torch.bool, device=DEV)
    sel.view(-1, 256)[idx] = True
    sel = sel[:n_valid]
    assert torch.equal(to_bits_t(out[:n_valid][sel]), to_bits_t(out_ref[sel]))
    assert bool((out[:n_valid][~sel] == 7.0).all()) and bool((out[n_valid:] == 7.0).all())    # nothing else touched

    # without stats, scatter into a residual-sized buffer; rows == None is the identity list
    plain = torch.zeros_like(full)
    capi.scaling_decompress_rows(send, plain, rows, None, nsc * 256, nrows, nbits, strategy)
    assert torch.equal(to_bits_t(plain), to_bits_t(res))
    ident = torch.empty_like(dec)
    capi.scaling_decompress_rows(send, ident, None, None, nrows * 256, nrows, nbits, strategy)
    assert torch.equal(to_bits_t(ident), to_bits_t(dec))
    # an element buffer that is only 2-byte aligned takes the per-lane store path
    if dt == torch.bfloat16:
        shifted = torch.zeros(nsc * 256 + 8, dtype=dt, device=DEV)[1:1 + nsc * 256]
        capi.scaling_decompress_rows(send, shifted, rows, stats, n_valid, nrows, nbits, strategy)
        assert torch.equal(to_bits_t(shifted[:n_valid][sel]), to_bits_t(out_ref[sel]))
        assert bool((shifted[n_valid:] == 0).all())


def to_bits_t(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def _tensors(n, W, seed):
    g = torch.Generator().manual_seed(seed)
    blocks = (n + 2559) // 2560
    scale = torch.exp(torch.randn(blocks, generator=g) * 4.0 + math.log(1e-3)).repeat_interleave(2560)[:n]
    return [(torch.randn(n, generator=g) * scale).to(torch.bfloat16).to(DEV) for _ in range(W)]


def _compressors(cls, W, n, seed):
    out = {}
    for q in (2, 4, 8):
        out[q] = []
        for r in range(W):
            params = {"d": {(0, 0): n * 4}, "world_size": W, "rank": r,
                      "args": types.SimpleNamespace(aggregation_method="dynamiQ")}
            gen = torch.Generator(device=DEV).manual_seed(seed * 100 + q * 10 + r)
            out[q].append(cls(q, 16, params, generator=gen))
    return out


@pytest.mark.parametrize("W", [1, 2, 5])
@pytest.mark.parametrize("method", ["aee", "mee"])
def test_grouped_pipeline_equals_reference_sequence(eden_utils, W, method):
    from dynamiq_sigcomm_artifact_amd import bitrate
    from dynamiq_sigcomm_artifact_amd.compressors import Aee_Dynamic_Range_GPU_kern, Mee_Dynamic_Range_GPU_kern
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import dynamic_bitrate_allreduce, dynamic_bitrate_allreduce_grouped
    cls = Aee_Dynamic_Range_GPU_kern if method == "aee" else Mee_Dynamic_Range_GPU_kern
    n = 256 * 2111 + 19            # a ragged tail: the last superchunk is mostly padding
    vecs = _tensors(n, W, 3)
    # u from the reduced norms, as the hook does at its first compressed round (comm_hooks.py:94-114)
    nsc = (n + 255) // 256
    norms = torch.zeros(nsc, dtype=torch.bfloat16, device=DEV)
    for v in vecs:
        st = torch.empty(nsc, 2, dtype=torch.bfloat16, device=DEV)
        eden_utils.superchunk_mean_center(v, torch.empty(nsc * 256, dtype=v.dtype, device=DEV), st, n, W)
        norms += st[:, 1]
    u, _, _ = bitrate.dynamic_bitrate_binary_search_u([norms], 4.375)
    a_out, a_stats, a_q = dynamic_bitrate_allreduce([v.clone() for v in vecs], u, _compressors(cls, W, n, 1))
    b_out, b_stats, b_q = dynamic_bitrate_allreduce_grouped([v.clone() for v in vecs], u, _compressors(cls, W, n, 1))
    assert torch.equal(a_q, b_q) and len({int(x) for x in a_q.unique().tolist()}) == 3
    assert torch.equal(to_bits_t(a_stats), to_bits_t(b_stats))
    for r in range(W):
        assert torch.equal(to_bits_t(a_out[r]), to_bits_t(b_out[r])), r
    for r in range(1, W):
        assert torch.equal(to_bits_t(b_out[0]), to_bits_t(b_out[r]))
    c_out, _, c_q = dynamic_bitrate_allreduce_grouped([v.clone() for v in vecs], u, _compressors(cls, W, n, 1),
                                                      device_qbits=True)
    assert torch.equal(c_q, a_q) and torch.equal(to_bits_t(c_out[0]), to_bits_t(a_out[0]))
    ref = torch.stack([v.double() for v in vecs]).mean(0)
    nmse = float(((b_out[0].double() - ref) ** 2).sum() / (ref ** 2).sum())
    assert nmse < 0.2


@pytest.mark.parametrize("nsc,shift", [(70000, 0), (4099, 1), (65536, 1)])
def test_group_plan_stats_two_launch_paths(capi, oracle, nsc, shift):
    """more than 64 tiles, and a stats buffer that is only 2-byte aligned, take the two-launch path: same result"""
    g = torch.Generator().manual_seed(nsc)
    norms = torch.exp(torch.randn(nsc, generator=g) * 6.0).to(torch.bfloat16)
    buf = torch.zeros(2 * nsc + 2, dtype=torch.bfloat16)
    stats = buf[shift:shift + 2 * nsc].view(nsc, 2)
    stats[:, 1] = norms
    stats_d = buf.to(DEV)[shift:shift + 2 * nsc].view(nsc, 2)
    assert stats_d.data_ptr() % 4 == 2 * shift
    order = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    qout = torch.empty(nsc, dtype=torch.int64, device=DEV)
    u = 7.1
    capi.group_plan_stats(stats_d, u, qout, order, work)
    want = oracle.dynamic_bitrate_qbits(to_bits(norms), u)
    assert (qout.cpu().numpy() == want).all()
    counts = work[:4].tolist()
    assert counts == [int((want == 8).sum()), int((want == 4).sum()), int((want == 2).sum()), 0] and min(counts[:3]) > 0
    order_h = order.cpu().numpy()
    for gi, w in enumerate((8, 4, 2)):
        idx = np.nonzero(want == w)[0]
        assert (order_h[gi * nsc:gi * nsc + idx.size] == idx).all()
        assert (order_h[gi * nsc + idx.size:(gi + 1) * nsc] == -1).all()


@pytest.mark.parametrize("u_on_device", [False, True])
@pytest.mark.parametrize("nsc,shift", [(5000, 0), (5000, 2), (65537, 0), (70000, 0), (70001, 0), (70002, 2), (200003, 0), (1048576 + 1029, 0)])
def test_group_plan_stats_long_buckets(capi, oracle, nsc, shift, u_on_device):
    """more than 64 tiles with 16-byte aligned statistics: the first launch counts a group of tiles per workgroup, four
    superchunks per load, and leaves the thresholds and the totals of its group; the second reads those.  Ragged
    ends, negative, NaN and infinite norms, u as a number and from device memory, and (shift 2) the statistics 4 bytes off,
    which takes the older pair of kernels; 5,000 superchunks: the same inputs through the one-launch kernel, with its
    four-per-load recount and (shift 2) without: all against the width rule of the oracle"""
    g = torch.Generator().manual_seed(nsc + shift)
    norms = torch.exp(torch.randn(nsc, generator=g) * 6.0).to(torch.bfloat16)
    special = torch.randperm(nsc, generator=g)[:400]
    norms[special[:100]] = -norms[special[:100]]
    norms[special[100:200]] = float("nan")
    norms[special[200:300]] = float("inf")
    norms[special[300:400]] = 0.0
    norms[nsc - 1] = float("nan")                      # in the ragged last quad where there is one
    buf = torch.zeros(2 * nsc + 8, dtype=torch.bfloat16)
    stats = buf[shift:shift + 2 * nsc].view(nsc, 2)
    stats[:, 1] = norms
    stats[:, 0] = torch.randn(nsc, generator=g).to(torch.bfloat16)   # the means in the low halves must not matter
    stats_d = buf.to(DEV)[shift:shift + 2 * nsc].view(nsc, 2)
    assert stats_d.data_ptr() % 16 == (2 * shift) % 16
    order = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work = torch.full((capi.group_plan_work_ints(nsc),), -5, dtype=torch.int32, device=DEV)
    qout = torch.empty(nsc, dtype=torch.int64, device=DEV)
    u = 7.1
    capi.group_plan_stats(stats_d, torch.tensor([u], dtype=torch.float64, device=DEV) if u_on_device else u, qout, order, work)
    want = oracle.dynamic_bitrate_qbits(to_bits(norms), u)
    assert (qout.cpu().numpy() == want).all()
    counts = work[:4].tolist()
    assert counts == [int((want == 8).sum()), int((want == 4).sum()), int((want == 2).sum()), 0] and min(counts[:3]) > 0
    order_h = order.cpu().numpy()
    for gi, w in enumerate((8, 4, 2)):
        idx = np.nonzero(want == w)[0]
        assert (order_h[gi * nsc:gi * nsc + idx.size] == idx).all()
        assert (order_h[gi * nsc + idx.size:(gi + 1) * nsc] == -1).all()
    # without the width output, and once more into the same work buffer (nothing of a plan may depend on what an earlier one left)
    order2 = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    capi.group_plan_stats(stats_d, u, None, order2, work)
    assert torch.equal(order, order2) and work[:4].tolist() == counts


@pytest.mark.parametrize("nsc", [30000, 70000])
def test_group_plan_stats_thresholds_kept_in_the_work_buffer(capi, oracle, nsc):
    """with u in device memory the plan (one launch, or the pair for long buckets) leaves the thresholds it searched for in
    work[4..6] and a later launch on the same buffer takes them from there when u has the same bits: same plans with and
    without, after a change of u, and with anything else in those words (zeros, noise, the right u beside a broken seal, the
    entry of another u)"""
    g = torch.Generator().manual_seed(5)
    norms = torch.exp(torch.randn(nsc, generator=g) * 6.0).to(torch.bfloat16)
    norms[torch.randperm(nsc, generator=g)[:50]] = float("nan")
    stats = torch.zeros((nsc, 2), dtype=torch.bfloat16)
    stats[:, 1] = norms
    stats_d = stats.to(DEV)
    order = torch.empty(3 * nsc, dtype=torch.int32, device=DEV)

    def plan(u_dev, work):
        order.fill_(-1)
        q = torch.empty(nsc, dtype=torch.int64, device=DEV)
        capi.group_plan_stats(stats_d, u_dev, q, order, work)
        return q.cpu().numpy(), order.clone(), work[:4].tolist()

    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    u_dev = torch.tensor([7.1], dtype=torch.float64, device=DEV)
    for u in (7.1, 7.1, 3.25, 3.25, 7.1, 60.0, -10.0, 7.1):
        u_dev.fill_(u)
        q, o, c = plan(u_dev, work)
        want = oracle.dynamic_bitrate_qbits(to_bits(norms), u)
        assert (q == want).all(), u
        kept = work[4:8].cpu().numpy().view(np.uint32)
        assert kept[0] == np.float32(u).view(np.uint32) and kept[2] == kept[0] ^ kept[1] ^ 0x9e3779b9, u
        # the same through a fresh buffer (a search) and through one whose words 4..7 hold other things
        for fill in ("zeros", "noise", "broken seal", "other u"):
            w2 = torch.zeros_like(work)
            if fill == "noise":
                w2[4:8] = torch.randint(-2 ** 31, 2 ** 31 - 1, (4,), generator=g, dtype=torch.int64).to(torch.int32).to(DEV)
            elif fill == "broken seal":
                w2[4:8] = work[4:8]
                w2[5] += 1
            elif fill == "other u":
                w2[4:8] = work[4:8]
                w2[4] += 1
            q2, o2, c2 = plan(u_dev, w2)
            assert (q2 == want).all() and torch.equal(o2, o) and c2 == c, (u, fill)
