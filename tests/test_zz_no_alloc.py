"""dq_eden_quantize_static: the entry point that allocates nothing (its per-tile partial sums live in a
static device array inside the library).  Checked through the C ABI against dq_eden_quantize, bit for bit,
on two calls in a row, the second with a smaller input, so that what the first call left in the shared
array cannot leak into the second."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "eden_golden.npz"))


def _pair(capi, n, nbits, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(n, generator=g) * 3e-3).to(DEV)
    cen = torch.from_numpy(GOLD["centroids_%d" % nbits]).to(DEV)
    bnd = torch.from_numpy(GOLD["boundaries_%d" % nbits]).to(DEV)
    words = n // 32 * nbits
    packed_a = torch.full((words + 8,), -1, dtype=torch.int32, device=DEV)   # 8 canary words behind the output
    packed_b = torch.full((words + 8,), -1, dtype=torch.int32, device=DEV)
    res_a = torch.zeros(4, device=DEV)
    res_b = torch.zeros(4, device=DEV)
    work = torch.zeros(capi.eden_work_doubles(n), dtype=torch.float64, device=DEV)
    torch.cuda.synchronize()
    capi.eden_quantize(x, bnd, cen, nbits, packed_a, res_a, work)
    capi.eden_quantize_static(x, bnd, cen, nbits, packed_b, res_b)
    torch.cuda.synchronize()
    return packed_a.cpu().numpy(), res_a.cpu().numpy(), packed_b.cpu().numpy(), res_b.cpu().numpy(), words


def test_static_scratch_matches_caller_scratch_twice_second_smaller(capi):
    assert capi.lib().dq_eden_quantize_static_max_n() == 1 << 28
    for n, nbits, seed in ((4096 * 37 + 96, 4, 11), (4096 * 5 + 32, 5, 12)):
        pa, ra, pb, rb, words = _pair(capi, n, nbits, seed)
        assert (ra.view(np.uint32) == rb.view(np.uint32)).all(), (n, ra, rb)
        assert (pa[:words] == pb[:words]).all(), n
        assert (pb[words:] == -1).all(), n
        assert np.isfinite(rb).all() and rb[0] > 0 and rb[2] > 0


def test_static_scratch_allocates_nothing_and_replays_from_a_graph(capi):
    """a warmed call leaves the device's free-memory counter where it was, and the call captured into a HIP graph on one
    stream gives the eager result on every replay (other work and synchronisations between the replays)"""
    n, nbits = 4096 * 9 + 64, 4
    g = torch.Generator().manual_seed(21)
    x = (torch.randn(n, generator=g) * 3e-3).to(DEV)
    cen = torch.from_numpy(GOLD["centroids_%d" % nbits]).to(DEV)
    bnd = torch.from_numpy(GOLD["boundaries_%d" % nbits]).to(DEV)
    words = n // 32 * nbits
    eager = torch.zeros(words, dtype=torch.int32, device=DEV)
    res_eager = torch.zeros(4, device=DEV)
    capi.eden_quantize_static(x, bnd, cen, nbits, eager, res_eager)           # warm-up: the library is loaded and set up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        capi.eden_quantize_static(x, bnd, cen, nbits, eager, res_eager)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before

    packed = torch.zeros(words, dtype=torch.int32, device=DEV)
    res = torch.zeros(4, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            capi.eden_quantize_static(x, bnd, cen, nbits, packed, res, stream=side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for k in range(3):
        packed.fill_(-1)              # a fill kernel, not a memset node
        res.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(packed, eager), k
        assert torch.equal(res.view(torch.int32), res_eager.view(torch.int32)), k
        y = (x * 2.0).sum()           # the program's own eager work between the replays
        torch.cuda.synchronize()
        assert torch.isfinite(y)


def test_static_scratch_rejects_oversize_and_bad_arguments(capi):
    L = capi.lib()
    one = torch.zeros(64, device=DEV)
    pk = torch.zeros(64, dtype=torch.int32, device=DEV)
    args = lambda n, nbits: (one.data_ptr(), n, one.data_ptr(), one.data_ptr(), nbits, pk.data_ptr(), one.data_ptr(), 0, None)
    assert L.dq_eden_quantize_static(*args((1 << 28) + 32, 4)) != 0          # beyond the static array: refused before any launch
    assert b"static scratch" in L.dq_last_error()
    assert L.dq_eden_quantize_static(*args(48, 4)) != 0                      # not a multiple of 32
    assert L.dq_eden_quantize_static(*args(64, 9)) != 0
    torch.cuda.synchronize()
