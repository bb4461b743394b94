"""The compressed ring all-reduce of DynamiQ with all W ranks simulated in the
HBM of one GPU.

The step order is the reference's
(testbed_evaluation/new_comm_hooks/ring_rdma.py:590-631): the vector is split
into W chunks aligned to the superchunk size; reduce-scatter = compress the own
chunk, then W-2 x (decode the received record stream, add the local chunk,
re-quantise: ``dec_compression``); the owner runs one more ``dec_compression``
and decodes its own ``send`` buffer back into the owner chunk, so every rank ends
with the same quantised value; all-gather = W-1 x decode.  The exchange between
neighbours, which is a network transfer in the reference, is a device-to-device
copy of the packed buffer here -- there is no inter-GPU traffic in this build.

Ranks advance in lock step (rank 0..W-1 per step), which is what a real ring
does concurrently; every rank owns its compressor object and therefore its own
random-pool offsets, exactly as separate processes would.
"""
import torch


def _align_up(x, a):
    return (x + a - 1) // a * a


def split_chunks(vec, world_size, align):
    """ring_rdma.py:590-595"""
    chunk_size = (vec.numel() + world_size - 1) // world_size
    chunk_size = _align_up(chunk_size, align)
    return [vec[chunk_size * i: min(chunk_size * (i + 1), vec.numel())] for i in range(world_size)]


def ring_allreduce(rank_vecs, compressors, align=256):
    """In-place compressed ring all-reduce (sum) over ``rank_vecs`` (one tensor per
    simulated rank, equal sizes) with one compressor object per rank.  Returns the
    list of tensors; afterwards they all hold the same quantised sum."""
    W = len(rank_vecs)
    assert W == len(compressors) and W >= 2
    chunks = [split_chunks(v, W, align) for v in rank_vecs]
    send = [c.create_tensor(chunks[r][0], torch.uint8) for r, c in enumerate(compressors)]
    recv = [c.create_tensor(chunks[r][0], torch.uint8) for r, c in enumerate(compressors)]

    def exchange(src_bufs, dst_bufs):
        # rank r sends to r+1 and receives from r-1 (ring_rdma.py:617)
        for r in range(W):
            dst_bufs[(r + 1) % W].copy_(src_bufs[r])

    # reduce-scatter
    for step in range(W - 1):
        for r in range(W):
            if step == 0:
                compressors[r].compression(chunks[r][r], send[r])
            else:
                compressors[r].dec_compression(recv[r], chunks[r][(r - step + W) % W], send[r])
        exchange(send, recv)

    for r in range(W):
        owner = chunks[r][(r + 1) % W]
        compressors[r].dec_compression(recv[r], owner, send[r])
        compressors[r].decompression(send[r], owner)

    # all-gather
    bufs = [send, recv]
    for step in range(W - 1):
        exchange(bufs[step & 1], bufs[(step ^ 1) & 1])
        for r in range(W):
            compressors[r].decompression(bufs[(step ^ 1) & 1][r], chunks[r][(r - step + W) % W])
    return rank_vecs


def split_rows(rows, world_size):
    """the ring chunks of a group of superchunks: split_chunks() on its 256 * len(rows) elements"""
    per = (rows.numel() * 256 + world_size - 1) // world_size
    per = _align_up(per, 256) // 256
    return [rows[per * i: min(per * (i + 1), rows.numel())] for i in range(world_size)]


def ring_allreduce_rows(rank_residuals, rows, compressors, rank_outputs, stats, n_limit):
    """The same schedule for one bit-width group without materialising the group tensor: ``rows`` (int32)
    lists the group's superchunks; every rank reads them from its full residual buffer and the decoded
    result lands, mean added, in the rank's output buffer.  Byte-identical to index_select ->
    ring_allreduce -> index_copy_ -> superchunk_add_mean_copy on those superchunks."""
    W = len(rank_residuals)
    assert W == len(compressors) and W >= 2
    chunks = split_rows(rows, W)
    nbytes = compressors[0].compressed_numel(chunks[0].numel() * 256)
    dev = rank_residuals[0].device
    send = [torch.zeros(nbytes, dtype=torch.uint8, device=dev) for _ in range(W)]
    recv = [torch.zeros(nbytes, dtype=torch.uint8, device=dev) for _ in range(W)]

    def exchange(src_bufs, dst_bufs):
        for r in range(W):
            dst_bufs[(r + 1) % W].copy_(src_bufs[r])

    for step in range(W - 1):
        for r in range(W):
            if step == 0:
                compressors[r].compression_rows(rank_residuals[r], chunks[r], send[r])
            else:
                compressors[r].dec_compression_rows(recv[r], rank_residuals[r], chunks[(r - step + W) % W], send[r])
        exchange(send, recv)

    for r in range(W):
        owner = chunks[(r + 1) % W]
        compressors[r].dec_compression_rows(recv[r], rank_residuals[r], owner, send[r])
        compressors[r].decompression_rows(send[r], rank_outputs[r], owner, stats, n_limit)

    bufs = [send, recv]
    for step in range(W - 1):
        exchange(bufs[step & 1], bufs[(step ^ 1) & 1])
        for r in range(W):
            compressors[r].decompression_rows(bufs[(step ^ 1) & 1][r], rank_outputs[r], chunks[(r - step + W) % W],
                                              stats, n_limit)
    return rank_outputs
