"""One bucket partition of DynamiQ's dynamic-bitrate all-reduce, with the W ranks
simulated in one GPU's HBM -- the host-side mirror of
``compress_and_reduce_and_decompress`` in
testbed_evaluation/new_comm_hooks/comm_hooks.py:932-1024:

  superchunk_mean_center -> (stats all-reduce) -> per-superchunk q in {2,4,8} ->
  per bit width: gather the superchunks of that width, compressed ring
  all-reduce, scatter back -> superchunk_add_mean_copy.

The stats all-reduce, a collective in the reference, is a sequential bf16 sum
over the simulated ranks here; with one rank the ring degenerates to
compress -> decompress of the rank's own chunk (ring_rdma.py:606-621 with
size == 1).
"""
import torch

from . import bitrate
from .compressors import superchunk_add_mean_copy, superchunk_mean_center
from .ring_sim import ring_allreduce

SUPERCHUNK = 256


def dynamic_bitrate_allreduce(rank_vecs, u, compressors, out=None):
    """rank_vecs: list of W equal-length 1-D tensors (fp16/bf16).  compressors:
    {2: [c_rank0, ...], 4: [...], 8: [...]}.  Returns (result tensors per rank,
    reduced stats, qbits)."""
    W = len(rank_vecs)
    n = rank_vecs[0].numel()
    nsc = (n + SUPERCHUNK - 1) // SUPERCHUNK
    dev, dt = rank_vecs[0].device, rank_vecs[0].dtype
    residuals = [torch.empty(nsc * SUPERCHUNK, dtype=dt, device=dev) for _ in range(W)]
    stats = [torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev) for _ in range(W)]
    for r in range(W):
        superchunk_mean_center(rank_vecs[r], residuals[r], stats[r], n, W, SUPERCHUNK)
    total = stats[0].clone()
    for r in range(1, W):
        total.add_(stats[r])
    norms = total[:, 1]
    qbits = bitrate.dynamic_bitrate_qbits(norms, u)

    res2d = [res.view(-1, SUPERCHUNK) for res in residuals]
    for q in (8, 4, 2):
        idx = torch.nonzero(qbits == q, as_tuple=False).view(-1)
        if idx.numel() == 0:
            continue
        groups = [torch.index_select(res2d[r], 0, idx).reshape(-1) for r in range(W)]
        comps = compressors[q]
        if W == 1:
            c = comps[0]
            send = c.create_tensor(groups[0], torch.uint8)
            c.compression(groups[0], send)
            c.decompression(send, groups[0])
        else:
            ring_allreduce(groups, comps, align=SUPERCHUNK)
        for r in range(W):
            res2d[r].index_copy_(0, idx, groups[r].view(-1, SUPERCHUNK))

    outs = out if out is not None else [torch.empty(n, dtype=dt, device=dev) for _ in range(W)]
    for r in range(W):
        superchunk_add_mean_copy(residuals[r], outs[r], total, n, SUPERCHUNK)
    return outs, total, qbits
