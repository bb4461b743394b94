"""The search for the offset u on a histogram of the norm patterns (dq_norm_histogram, dq_bitrate_search) against the
oracle's restatement of comm_hooks.py:73-139 over the norms themselves, and against the reference's torch op sequence
run on the device.  Every result is compared with ==: counts are integers and the search runs in IEEE double."""
import numpy as np
import pytest
import torch

from helpers import to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MAXP = 0x7f80


def _stats(norms):
    """bf16 [nsc, 2] statistics with the given norm column"""
    st = torch.zeros((norms.numel(), 2), dtype=torch.bfloat16, device=DEV)
    st[:, 1] = norms.to(DEV)
    st[:, 0] = 0.25
    return st


def _norm_sets():
    g = torch.Generator().manual_seed(3)
    sets = {
        "lognormal": [torch.exp(torch.randn(25600, generator=g) * 3 - 8).to(torch.bfloat16)],
        "three buckets": [torch.exp(torch.randn(n, generator=g) * s - 6).to(torch.bfloat16)
                          for n, s in ((5000, 5.0), (1, 1.0), (70001, 0.5))],
        "narrow": [(torch.rand(4096, generator=g) * 1e-4 + 2e-4).to(torch.bfloat16)],
        "one value": [torch.full((300,), 1.0).to(torch.bfloat16)],
    }
    special = torch.exp(torch.randn(2000, generator=g) * 4 - 5).to(torch.bfloat16)
    special[::7] = 0.0
    special[1::97] = float("nan")
    special[2::131] = -1.0
    special[3::211] = -0.0
    sets["zeros, NaN, negative"] = [special]
    return sets


def test_norm_histogram_counts(capi):
    norms = _norm_sets()["zeros, NaN, negative"][0].clone()
    norms[5] = float("inf")
    norms[6] = float("-inf")
    hist = torch.zeros(capi.bitrate_hist_ints(), dtype=torch.int32, device=DEV)
    capi.norm_histogram(_stats(norms), hist)
    capi.norm_histogram(_stats(norms[:100]), hist)          # accumulates
    pat = np.concatenate([to_bits(norms), to_bits(norms[:100])]).astype(np.int64)
    nan = (pat & 0x7fff) > MAXP
    bins = np.where(nan, MAXP + 1, np.where(pat > MAXP, 0, pat))
    want = np.bincount(bins, minlength=hist.numel())
    assert (hist.cpu().numpy() == want).all()
    assert want[MAXP] == 2 and want[MAXP + 1] > 0           # +inf (in both calls), NaN


@pytest.mark.parametrize("name", list(_norm_sets().keys()))
def test_search_equals_the_oracle_on_the_norms(capi, oracle, name):
    from dynamiq_sigcomm_artifact_amd.bitrate import NormHistogram
    norms_list = _norm_sets()[name]
    bits_list = [to_bits(t) for t in norms_list]
    h = NormHistogram(DEV)
    for target in (1.375, 2.375, 3.375, 4.375, 5.375, 7.375, 9.0):
        for t in norms_list:
            h.add(_stats(t))
        assert h.count == sum(t.numel() for t in norms_list)
        got = h.binary_search_u(target)
        want = oracle.dynamic_bitrate_binary_search_u(bits_list, target)
        assert got == tuple(want), (name, target, got, want)
        assert int(h.hist.abs().sum()) == 0 and h.count == 0          # consumed
        for prev in (want[0], want[0] + 6.0, want[0] - 3.5, 60.0, -10.0, 100.0, -50.0):
            for t in norms_list:
                h.add(_stats(t))
            got = h.adjust_u(prev, target)
            want2 = oracle.dynamic_bitrate_adjust_u(bits_list, prev, target)
            assert got == tuple(want2), (name, target, prev, got, want2)


def test_search_equals_the_torch_op_sequence_on_the_device():
    """the reference's own functions as mirrored in bitrate.py, on device tensors (the scalar u enters the add in
    binary32 there, as in the reference's CUDA run)"""
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    g = torch.Generator().manual_seed(9)
    norms_list = [torch.exp(torch.randn(n, generator=g) * 4 - 7).to(torch.bfloat16).to(DEV) for n in (30000, 777)]
    h = B.NormHistogram(DEV)
    for target in (2.375, 4.375, 6.375):
        for t in norms_list:
            h.add(_stats(t))
        got = h.binary_search_u(target)
        want = B.dynamic_bitrate_binary_search_u(norms_list, target)
        assert got == tuple(want), (target, got, want)
        for prev in (want[0] + 5.0, want[0] - 2.0):
            for t in norms_list:
                h.add(_stats(t))
            assert h.adjust_u(prev, target) == tuple(B.dynamic_bitrate_adjust_u(norms_list, prev, target))


def test_closed_forms_and_the_empty_histogram():
    """all norms 1.0: log2 = 0, so the width is 2 below u = 4, 4 below 8 (bf16(u) = 7.96875 already rounds to 8 bits), 8
    from there on, and the bisection can be followed by hand"""
    from dynamiq_sigcomm_artifact_amd.bitrate import NormHistogram
    h = NormHistogram(DEV)
    ones = _stats(torch.ones(1000).to(torch.bfloat16))
    h.add(ones)
    assert h.binary_search_u(4.0) == (7.5, 4.0, 0.0)              # probes 60, 25, 7.5
    h.add(ones)
    assert h.binary_search_u(3.0) == (7.5, 4.0, -1.0)             # unreachable: the first probe at distance 1 is kept
    h.add(ones)
    assert h.adjust_u(60.0, 4.0) == (56.0, 8.0, -4.0)             # one step of the deficit, same sign: returned
    h.add(ones)
    assert h.adjust_u(7.0, 4.0) == (7.0, 4.0, 0.0)
    assert float(h.result[3]) == 1.0                              # one probe
    # nothing added: the average is 0.0 everywhere, the starting candidate stays the best
    assert h.binary_search_u(4.375) == (60.0, 0.0, 4.375)
    assert float(h.result[3]) == 33.0


def test_pipeline_feeds_the_histogram(oracle):
    """a step of three buckets through the single-pass all-reduce with the histogram attached: the u for the next step
    equals the oracle's search over the reduced norms of the three buckets"""
    from dynamiq_sigcomm_artifact_amd.bitrate import NormHistogram
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import dynamic_bitrate_allreduce_single_pass
    g = torch.Generator().manual_seed(21)
    h = NormHistogram(DEV)
    reduced = []
    for nsc, W in ((40, 2), (7, 1), (130, 3)):
        scales = torch.exp(torch.randn(nsc, 1, generator=g) * 4.0) * 1e-3
        vecs = [(torch.randn(nsc, 256, generator=g) * scales).reshape(-1).to(torch.bfloat16).to(DEV) for _ in range(W)]
        _, total, _ = dynamic_bitrate_allreduce_single_pass(vecs, 7.0, norm_histogram=h)
        reduced.append(to_bits(total[:, 1].contiguous()))
    assert h.count == 177
    counted = h.hist.clone()
    got = h.adjust_u(7.0, 4.375)
    assert got == tuple(oracle.dynamic_bitrate_adjust_u(reduced, 7.0, 4.375))
    # the same step with u in device memory: the plan launches fill the histogram themselves, same counts, same outputs
    g = torch.Generator().manual_seed(21)
    u_dev = torch.tensor([7.0], dtype=torch.float64, device=DEV)
    h2 = NormHistogram(DEV)
    for nsc, W in ((40, 2), (7, 1), (130, 3)):
        scales = torch.exp(torch.randn(nsc, 1, generator=g) * 4.0) * 1e-3
        vecs = [(torch.randn(nsc, 256, generator=g) * scales).reshape(-1).to(torch.bfloat16).to(DEV) for _ in range(W)]
        outs_a, _, plan_a = dynamic_bitrate_allreduce_single_pass(vecs, u_dev, norm_histogram=h2)
        outs_b, _, plan_b = dynamic_bitrate_allreduce_single_pass(vecs, 7.0)
        assert plan_a.tolist() == plan_b.tolist() and all(torch.equal(a, b) for a, b in zip(outs_a, outs_b))
    assert h2.count == 177 and torch.equal(h2.hist, counted)


@pytest.mark.parametrize("nsc", [3000, 70000])
def test_plan_reads_the_offset_from_device_memory(capi, nsc):
    """search -> plan with nothing read back: the plan kernels (one launch and, beyond 65536 superchunks, two) take u from
    the search's result tensor and give the widths, counts and order of the call that gets the same u as a number"""
    from dynamiq_sigcomm_artifact_amd.bitrate import NormHistogram
    g = torch.Generator().manual_seed(nsc)
    stats = _stats(torch.exp(torch.randn(nsc, generator=g) * 4 - 6).to(torch.bfloat16))
    h = NormHistogram(DEV)
    h.add(stats)
    capi.bitrate_search(h.hist, 0, 0.0, 4.375, h.result)             # no read-back here
    order_a = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    order_b = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work_a = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    work_b = torch.zeros_like(work_a)
    q_a = torch.zeros(nsc, dtype=torch.int64, device=DEV)
    q_b = torch.zeros_like(q_a)
    capi.group_plan_stats(stats, h.result[0:1], q_a, order_a, work_a)
    u = float(h.result[0])
    capi.group_plan_stats(stats, u, q_b, order_b, work_b)
    assert torch.equal(q_a, q_b) and torch.equal(order_a, order_b) and work_a[:4].tolist() == work_b[:4].tolist()
    assert sorted(work_a[:3].tolist())[1] > 0                        # at least two widths in use
    with pytest.raises(RuntimeError, match="float64"):
        capi.group_plan_stats(stats, torch.zeros(1, device=DEV), None, order_a, work_a)


def test_steps_chained_on_the_device(capi, oracle):
    """four training steps with drifting norms: the correction of every step starts from the u the previous search left
    in device memory, the plans read it from there, nothing is read back until the end -- and the final triple is the
    one the oracle's functions give when chained on the host"""
    from dynamiq_sigcomm_artifact_amd.bitrate import NormHistogram
    g = torch.Generator().manual_seed(33)
    h = NormHistogram(DEV)
    target = 4.375
    steps = [[torch.exp(torch.randn(n, generator=g) * 3 - 7 + 0.8 * k).to(torch.bfloat16) for n in (9000, 400)] for k in range(4)]
    want = None
    for k, norms_list in enumerate(steps):
        for t in norms_list:
            h.add(_stats(t))
        h.launch_search(0 if k == 0 else 1, 0.0 if k == 0 else h.result[0:1], target)
        bits = [to_bits(t) for t in norms_list]
        want = (oracle.dynamic_bitrate_binary_search_u(bits, target) if k == 0
                else oracle.dynamic_bitrate_adjust_u(bits, want[0], target))
        # a plan of the next step reading u from the device
        nsc = norms_list[0].numel()
        order = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
        work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
        q = torch.zeros(nsc, dtype=torch.int64, device=DEV)
        capi.group_plan_stats(_stats(norms_list[0]), h.result[0:1], q, order, work)
        assert (q.cpu().numpy() == oracle.dynamic_bitrate_qbits(bits[0], want[0])).all()
    assert tuple(h.result[:3].tolist()) == tuple(want)


@pytest.mark.parametrize("nsc", [1, 1000, 25600, 65536, 70000])
def test_plan_launch_fills_the_histogram(capi, nsc):
    """the histogram workgroup of the plan launch (and the separate launch beyond 65536 superchunks) counts what
    norm_histogram counts, and leaves the plan as it is"""
    g = torch.Generator().manual_seed(nsc)
    norms = torch.exp(torch.randn(nsc, generator=g) * 4 - 6).to(torch.bfloat16)
    if nsc > 10:
        norms[3], norms[5], norms[7] = float("nan"), -1.0, float("inf")
    stats = _stats(norms)
    u = torch.tensor([7.3, 0, 0, 0], dtype=torch.float64, device=DEV)
    want = torch.full((capi.bitrate_hist_ints(),), 5, dtype=torch.int32, device=DEV)      # accumulates on top
    got = want.clone()
    capi.norm_histogram(stats, want)
    order_a = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    order_b = torch.full((3 * nsc,), -1, dtype=torch.int32, device=DEV)
    work_a = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=DEV)
    work_b = torch.zeros_like(work_a)
    capi.group_plan_stats(stats, u[0:1], None, order_a, work_a, hist=got)
    capi.group_plan_stats(stats, 7.3, None, order_b, work_b)
    assert torch.equal(got, want) and int(got.sum()) == 5 * got.numel() + nsc
    assert torch.equal(order_a, order_b) and work_a[:4].tolist() == work_b[:4].tolist()
    # a number for u and a histogram: the same counts through a launch of its own
    again = torch.full_like(got, 5)
    capi.group_plan_stats(stats, 7.3, None, order_b, work_b, hist=again)
    assert torch.equal(again, want)


def test_search_and_pipeline_on_a_side_stream(capi):
    """the search's read-back waits for the stream it was launched on, and the pipeline puts its torch ops (statistics
    sum, exchange copies) on the stream of its kernels: a side stream given as a torch stream or as a raw handle gives
    the results of the current stream"""
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import dynamic_bitrate_allreduce_single_pass
    g = torch.Generator().manual_seed(17)
    norms = torch.exp(torch.randn(25600, generator=g) * 3 - 8).to(torch.bfloat16)
    st = _stats(norms)
    h = B.NormHistogram(DEV)
    h.add(st)
    want = h.binary_search_u(4.375)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    for s in (side, side.cuda_stream):
        h.add(st, stream=s)
        assert h.binary_search_u(4.375, stream=s) == want
    vecs = [(torch.randn(256 * 300 + 17, generator=g) * 1e-2).to(torch.bfloat16).to(DEV) for _ in range(3)]
    ref, total, counts = dynamic_bitrate_allreduce_single_pass(vecs, want[0], seed=3)
    torch.cuda.synchronize()
    outs, total2, counts2 = dynamic_bitrate_allreduce_single_pass(vecs, want[0], seed=3, stream=side)
    side.synchronize()
    assert counts.tolist() == counts2.tolist()
    for a, b in zip(ref, outs):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
