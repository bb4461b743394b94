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
from . import load_eden_utils
from .ring_sim import ring_allreduce, ring_allreduce_rows

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


def dynamic_bitrate_allreduce_grouped(rank_vecs, u, compressors, out=None, work=None, device_qbits=False):
    """Same inputs, same results (bit for bit) as dynamic_bitrate_allreduce, with the gather, the scatter
    and the final mean add folded into the codec kernels: one device-side partition of the superchunk
    indices by width (a single 16-byte read-back for the three group sizes, in place of three
    torch.nonzero), no group tensors, no index_select / index_copy_ / superchunk_add_mean_copy passes.

    device_qbits=True also computes the bit widths inside the partition call (the rule of
    bitrate.dynamic_bitrate_qbits with the library's fixed-polynomial log2 in place of torch.log2; the two
    agree except where a log2 value lies within a few binary32 ulps of a bf16 rounding boundary)."""
    eu = load_eden_utils()
    W = len(rank_vecs)
    n = rank_vecs[0].numel()
    nsc = (n + SUPERCHUNK - 1) // SUPERCHUNK
    dev, dt = rank_vecs[0].device, rank_vecs[0].dtype
    if work is None:
        work = {}
    key = (nsc, dt, W)
    if work.get("key") != key:
        work["key"] = key
        work["residuals"] = [torch.empty(nsc * SUPERCHUNK, dtype=dt, device=dev) for _ in range(W)]
        work["stats"] = [torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev) for _ in range(W)]
        work["order"] = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
    residuals, stats, order = work["residuals"], work["stats"], work["order"]
    stream = torch.cuda.current_stream().cuda_stream
    for r in range(W):
        superchunk_mean_center(rank_vecs[r], residuals[r], stats[r], n, W, SUPERCHUNK)
    total = stats[0] if W == 1 else stats[0].clone()
    for r in range(1, W):
        total.add_(stats[r])
    if device_qbits:
        qbits = work.get("qbits")
        if qbits is None or qbits.numel() != nsc:
            qbits = work["qbits"] = torch.empty(nsc, dtype=torch.int64, device=dev)
        counts = eu.group_plan_stats(total, float(u), order, qbits, stream).tolist()
    else:
        qbits = bitrate.dynamic_bitrate_qbits(total[:, 1], u)
        counts = eu.group_plan(qbits, order, stream).tolist()
    assert counts[3] == 0, "bit widths outside {2, 4, 8}"

    outs = out if out is not None else [torch.empty(n, dtype=dt, device=dev) for _ in range(W)]
    for g, (q, cnt) in enumerate(zip((8, 4, 2), counts[:3])):
        if cnt == 0:
            continue
        rows = order[g * nsc:g * nsc + cnt]          # every width has a region of nsc entries
        comps = compressors[q]
        if W == 1:
            c = comps[0]
            send = work.get(("send", q))
            need = c.compressed_numel(cnt * SUPERCHUNK)
            if send is None or send.numel() < need:
                send = work[("send", q)] = torch.empty(need, dtype=torch.uint8, device=dev)
            c.compression_rows(residuals[0], rows, send)
            c.decompression_rows(send, outs[0], rows, total, n)
        else:
            ring_allreduce_rows(residuals, rows, comps, outs, total, n)
    return outs, total, qbits


def fixed_proportion_allreduce(rank_vecs, thresholds, compressors, out=None, fixed_4bit_only=False):
    """One bucket partition of the non-dynamic hook, ``P2P_dynamiQ_hook``'s ``compress_and_reduce_and_decompress``
    (comm_hooks.py:682-786), as the reference's op sequence: mean-centre, reduce the statistics, sort the norms
    (stable, descending), gather the first / middle / last share as the 8- / 4- / 2-bit groups **in sorted order**, one
    compressed ring per group, scatter back, add the means.  ``fixed_4bit_only`` is the "fixed" method: only the 4-bit
    group (everything, thresholds {4: 1, 8: 0, 2: 0}) is communicated (:768-772)."""
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
    groups_idx = bitrate.fixed_proportion_groups(total[:, 1], thresholds)
    res2d = [res.view(-1, SUPERCHUNK) for res in residuals]
    for q, idx in zip((8, 4, 2), groups_idx):
        if idx.numel() == 0 or (fixed_4bit_only and q != 4):
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
    return outs, total, groups_idx


def fixed_proportion_allreduce_grouped(rank_vecs, thresholds, compressors, out=None, fixed_4bit_only=False):
    """The same all-reduce, bit for bit, with the sort, the slices, the gathers, the scatters and the final mean add
    replaced by one launch of the device plan (group_plan_sorted) and the row-list codec calls; the group sizes follow
    from the fractions on the host, so nothing is read back."""
    eu = load_eden_utils()
    W = len(rank_vecs)
    n = rank_vecs[0].numel()
    nsc = (n + SUPERCHUNK - 1) // SUPERCHUNK
    dev, dt = rank_vecs[0].device, rank_vecs[0].dtype
    residuals = [torch.empty(nsc * SUPERCHUNK, dtype=dt, device=dev) for _ in range(W)]
    stats = [torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev) for _ in range(W)]
    for r in range(W):
        superchunk_mean_center(rank_vecs[r], residuals[r], stats[r], n, W, SUPERCHUNK)
    total = stats[0] if W == 1 else stats[0].clone()
    for r in range(1, W):
        total.add_(stats[r])
    counts = bitrate.fixed_proportion_counts(nsc, thresholds)
    order = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
    eu.group_plan_sorted(total, counts[0], counts[2], order, None, torch.cuda.current_stream().cuda_stream)
    outs = out if out is not None else [torch.empty(n, dtype=dt, device=dev) for _ in range(W)]
    if fixed_4bit_only:
        # the groups that are not communicated keep their local residual: copy it through first
        for r in range(W):
            superchunk_add_mean_copy(residuals[r], outs[r], total, n, SUPERCHUNK)
    for g, (q, cnt) in enumerate(zip((8, 4, 2), counts)):
        if cnt == 0 or (fixed_4bit_only and q != 4):
            continue
        rows = order[g * nsc:g * nsc + cnt]
        comps = compressors[q]
        if W == 1:
            c = comps[0]
            send = torch.empty(c.compressed_numel(cnt * SUPERCHUNK), dtype=torch.uint8, device=dev)
            c.compression_rows(residuals[0], rows, send)
            c.decompression_rows(send, outs[0], rows, total, n)
        else:
            ring_allreduce_rows(residuals, rows, comps, outs, total, n)
    return outs, total, order, counts


def dynamic_bitrate_allreduce_single_pass(rank_vecs, u, strategy=2, seed=0, out=None, work=None, stream=None,
                                          norm_histogram=None):
    """The same all-reduce with every stage kept on the device: no residual buffers (the centring is folded
    into the codec's loads), no group tensors, no per-width launches and no read-back of the group sizes --
    a fixed sequence of launches per bucket (statistics, plan, and one codec launch per ring step for all
    three bit widths), which can be captured once and replayed as a graph.

    Per rank: superchunk_stats -> (stats sum) -> group_plan_stats -> ring over mixed_compress /
    mixed_decompress.  The bit widths follow the device rule of group_plan_stats; the rounding randomness is
    the in-kernel stream keyed by (seed + rank, ring step, index of the chunk in the vector), so results are
    reproducible but not those of dynamic_bitrate_allreduce, whose random values come from the pool.

    u: the offset of the width rule, a number or a float64 device tensor (e.g. result[0:1] of the offset search: then
    nothing of the step is read back).
    norm_histogram: a bitrate.NormHistogram that collects the reduced norms of the step's buckets for the search of
    the next step's u (comm_hooks.py:962, 904-931).

    Returns (result tensors per rank, reduced stats, device int32 tensor [n8, n4, n2, other])."""
    from . import capi
    W = len(rank_vecs)
    n = rank_vecs[0].numel()
    nsc = (n + SUPERCHUNK - 1) // SUPERCHUNK
    dev, dt = rank_vecs[0].device, rank_vecs[0].dtype
    if work is None:
        work = {}
    key = ("single_pass", nsc, dt, W)
    if work.get("key") != key:
        work.clear()
        work["key"] = key
        cap = capi.mixed_required_bytes(nsc, W)
        work["stats"] = [torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev) for _ in range(W)]
        work["mean"] = [torch.empty(nsc, dtype=torch.float32, device=dev) for _ in range(W)]
        work["total"] = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
        work["order"] = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
        work["plan"] = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=dev)
        work["send"] = [torch.zeros(cap, dtype=torch.uint8, device=dev) for _ in range(W)]
        work["recv"] = [torch.zeros(cap, dtype=torch.uint8, device=dev) for _ in range(W if W > 1 else 0)]
    stats, mean, order, plan = work["stats"], work["mean"], work["order"], work["plan"]
    send, recv = work["send"], work["recv"]
    # one stream for the kernels and for the torch ops between them (the statistics sum, the exchange copies):
    # resolved once per bucket, not once per launch
    torch_stream = capi.torch_stream(stream, dev)
    stream = torch_stream.cuda_stream
    for r in range(W):
        capi.superchunk_stats(rank_vecs[r], stats[r], mean[r], n, W, stream=stream)
    if W == 1:
        total = stats[0]
    else:
        total = work["total"]
        with torch.cuda.stream(torch_stream):
            total.copy_(stats[0])
            for r in range(1, W):
                total.add_(stats[r])
    # with u on the device the histogram is filled by a few more workgroups of the plan launch, otherwise by a launch of its own
    capi.group_plan_stats(total, u if isinstance(u, torch.Tensor) else float(u), None, order, plan, stream=stream,
                          hist=None if norm_histogram is None else norm_histogram.hist)
    if norm_histogram is not None:
        norm_histogram.count += nsc
    outs = out if out is not None else [torch.empty(n, dtype=dt, device=dev) for _ in range(W)]

    def encode(r, chunk, step, received=None):
        capi.mixed_compress(rank_vecs[r], order, plan, send[r], nsc, strategy, seed=seed + r, step=step, recv=received,
                            center_mean=mean[r], center_world=W, n=n, ring_chunk=chunk, ring_world=W, stream=stream)

    def decode(r, packed, chunk):
        capi.mixed_decompress(packed, outs[r], order, plan, nsc, strategy, stats=total, n_limit=n, ring_chunk=chunk,
                              ring_world=W, stream=stream)

    if W == 1:
        encode(0, 0, 0)
        decode(0, send[0], 0)
        return outs, total, plan[:4]

    def exchange(src_bufs, dst_bufs):
        with torch.cuda.stream(torch_stream):
            for r in range(W):
                dst_bufs[(r + 1) % W].copy_(src_bufs[r])

    # reduce-scatter: W - 1 steps, then the owner's step; all-gather of the owners' streams
    for step in range(W - 1):
        for r in range(W):
            encode(r, (r - step + W) % W, step, None if step == 0 else recv[r])
        exchange(send, recv)
    for r in range(W):
        encode(r, (r + 1) % W, W - 1, recv[r])
        decode(r, send[r], (r + 1) % W)
    bufs = [send, recv]
    for step in range(W - 1):
        exchange(bufs[step & 1], bufs[(step ^ 1) & 1])
        for r in range(W):
            decode(r, bufs[(step ^ 1) & 1][r], (r - step + W) % W)
    return outs, total, plan[:4]


def pick_streams(device, want, tries=16):
    """`want` streams that run side by side with each other and with the caller's current stream; returns (streams, ok).
    The runtime maps the streams of a process onto a few hardware queues when they are first used, and a queue works
    through what it is given in order, whichever stream it came from.  Two streams on one queue take turns; and with the
    caller's stream on the queue of one of them, an event that orders the *next* piece of work after the caller's
    (recorded on the caller's stream) completes only after the piece enqueued just before it -- either way two buckets
    "in flight" run as slowly as on one stream (measured: 31 against 18.5 us per 25 MB bucket).  Which streams share a
    queue depends on what else the process has used, so candidates are taken from torch's pool until `want` of them
    overlap with each other and with the current stream (capi.streams_overlap, about a millisecond per pair); if the
    pool does not yield that many, the set is filled up and ok is False."""
    from . import capi
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    apart = [torch.cuda.current_stream(device).cuda_stream]
    chosen = []
    while len(chosen) < want and tries > 0:
        tries -= 1
        cand = torch.cuda.Stream(device=device)
        if cand.cuda_stream not in apart and all(capi.streams_overlap(h, cand.cuda_stream, index) for h in apart):
            chosen.append(cand)
            apart.append(cand.cuda_stream)
    ok = len(chosen) == want
    while len(chosen) < want:
        chosen.append(torch.cuda.Stream(device=device))
    return chosen, ok


class SinglePassBuckets(object):
    """The single-pass dynamic-bitrate path for a stream of buckets on one rank (a ring of one: statistics, widths,
    partition, encode, decode, mean add -- what dynamic_bitrate_allreduce_single_pass does for W = 1), shaped for
    25 MB buckets, where the four kernels of a bucket take about as long as four host calls and every launch waits
    for the one before:

      * one host call per bucket (capi.dynamic_bitrate_bucket) instead of four (``run``);
      * eager buckets of the first of the ``streams`` slots run on the caller's own stream (``inline_first``): handing a
        bucket to another stream costs an event record, a wait and a dearer first launch behind it -- measured 17 us of
        host time against 13 us for the four kernels themselves;
      * ``streams`` buckets are in flight at a time, each on a stream of its own with scratch of its own (statistics,
        means, plan, packed stream): the latency-bound statistics and plan launches of one bucket overlap the codec
        launches of its neighbour.  The streams are chosen so that they do run side by side (``pick_streams``);
      * with ``graphs=True``, ``run_all`` records a whole step's buckets once -- one graph per stream -- and replays
        them: one graph launch per stream and step instead of one host call per bucket.  DDP hands the hook the same
        bucket views on every step, so the list of (source, output) pairs is the natural key; a replay reads whatever
        the sources hold then.  (A graph per bucket was measured and is slower than the eager call: launching a graph
        costs the host more than one call that enqueues four kernels.)

    The offset u of the width rule is read from device memory when the plan runs (``set_u`` or a float64 tensor of the
    caller's, e.g. the result of the offset search), and the rounding stream of the encoder is (seed, bucket ordinal *
    2^32 + the step counter in device memory, one copy per stream): ``begin_step`` advances the counters once per
    training step, so a replayed launch draws fresh random values on every step.

    run(x, out) enqueues a bucket and returns at once; join() makes the caller's current stream wait for everything
    enqueued so far.  The caller must not overwrite x or read out before join()."""

    def __init__(self, device, strategy=2, seed=0, streams=2, graphs=True, u=None, norm_histogram=None, inline_first=True):
        from . import capi
        self.capi = capi
        self.device = torch.device(device)
        self.strategy, self.seed, self.graphs, self.inline_first = strategy, int(seed), graphs, bool(inline_first)
        self.streams, self.side_by_side = pick_streams(self.device, max(1, int(streams)))
        self.scratch = [dict() for _ in self.streams]
        self.pending = [False] * len(self.streams)
        # one step counter per stream, advanced on that stream: no hand-over between streams at a step boundary
        self.step_devs = [torch.zeros(1, dtype=torch.int64, device=self.device) for _ in self.streams]
        self.u_dev = u if isinstance(u, torch.Tensor) else torch.full((1,), 60.0 if u is None else float(u), dtype=torch.float64,
                                                                     device=self.device)
        self.hist = norm_histogram
        ready = torch.cuda.Event()
        ready.record(torch.cuda.current_stream(self.device))
        for st in self.streams:
            st.wait_event(ready)         # the counters and u are initialised on the caller's stream
        self.cache = {}          # (x.data_ptr(), out.data_ptr(), n, dtype) -> _entry(); ("step", keys) -> [graphs, uses]
        self._enqueue = capi.lib().dq_dynamic_bitrate_bucket
        self._order = capi.lib().dq_stream_order_after
        self.ordinals = {}       # (x.data_ptr(), n) -> ordinal of the bucket in the random stream
        self.superchunks = 0

    # ---- once per training step ----------------------------------------------------------------------------
    def set_u(self, u):
        """the offset of the width rule for the buckets enqueued from now on (a number; a tensor was given at construction)"""
        cur = torch.cuda.current_stream(self.device)
        for k, st in enumerate(self.streams):
            if self.pending[k]:
                cur.wait_stream(st)
        self.u_dev.fill_(float(u))
        self._fence = torch.cuda.Event()
        self._fence.record(cur)
        for st in self.streams:
            st.wait_event(self._fence)

    def begin_step(self):
        """advance the step counter of the rounding stream: one small kernel per stream and training step, enqueued on
        that stream, so it is ordered with the stream's buckets and nothing waits for another stream"""
        for k, (st, counter) in enumerate(zip(self.streams, self.step_devs)):
            if k == 0 and self.inline_first:
                # slot 0 runs on the caller's stream when eager and on its worker stream when recorded: its counter is
                # advanced on the caller's stream, after whatever the worker stream still has of the previous step (a
                # recorded step orders the worker streams after the caller's before it starts)
                if self.pending[0]:
                    cur = torch.cuda.current_stream(self.device)
                    cur.wait_stream(st)
                    self.pending[0] = False
                counter.add_(1)
            else:
                with torch.cuda.stream(st):
                    counter.add_(1)

    # ---- per bucket ---------------------------------------------------------------------------------------------
    def _scratch(self, k, nsc):
        sc = self.scratch[k]
        if sc.get("nsc", 0) < nsc:
            capi, dev = self.capi, self.device
            sc["nsc"] = nsc
            sc["stats"] = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
            sc["mean"] = torch.empty(nsc, dtype=torch.float32, device=dev)
            sc["order"] = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
            sc["work"] = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=dev)
            sc["packed"] = torch.zeros(capi.mixed_required_bytes(nsc, 1), dtype=torch.uint8, device=dev)
            for name in ("stats", "mean", "order", "work", "packed"):
                sc[name].record_stream(self.streams[k])     # allocated on the caller's stream, used on this one
            # scratch of another size invalidates what was recorded against the old buffers
            for key in [key for key, entry in self.cache.items() if key[0] == "step" or entry[3] == k]:
                del self.cache[key]
        return sc

    def _entry(self, x, out, n, key):
        """descriptor of a bucket seen for the first time (or again after its stream's scratch grew)"""
        import ctypes
        capi = self.capi
        nsc = (n + 255) // 256
        # a source keeps its ordinal, and with it its stream and its recorded launches, from step to step
        ordinal = self.ordinals.setdefault((key[0], n), len(self.ordinals))
        k = ordinal % len(self.streams)
        sc = self._scratch(k, nsc)
        desc, dev = capi.bucket_descriptor(x, n, sc["stats"][:nsc], sc["mean"], sc["order"], sc["work"], sc["packed"],
                                           strategy=self.strategy, out=out, u=self.u_dev,
                                           hist=None if self.hist is None else self.hist.hist, seed=self.seed,
                                           step=ordinal << 32, step_dev=self.step_devs[k])
        # (descriptor, its reference for the call, device, stream index, superchunks, the stream's handle)
        entry = (desc, ctypes.byref(desc), dev, k, nsc, ctypes.c_void_p(self.streams[k].cuda_stream))
        self.cache[key] = entry
        return entry

    def run(self, x, out):
        """enqueue one bucket: out = decode(encode(x)) with the widths of its reduced norms; returns the index of the
        stream it went to.  The hot path of an eager caller: two library calls (order the worker stream after the
        caller's, enqueue the bucket's four kernels) and one dictionary look-up."""
        n = x.numel()
        key = (x.data_ptr(), out.data_ptr(), n, x.dtype)
        entry = self.cache.get(key)
        if entry is None:
            entry = self._entry(x, out, n, key)
        _, ref, dev, k, nsc, handle = entry
        cur = torch.cuda.current_stream(self.device).cuda_stream
        if k == 0 and self.inline_first:
            # the first bucket of every round of `streams` goes to the caller's own stream: nothing to order, and ordering a
            # worker stream after the caller's costs the host more than enqueueing the bucket's four kernels does
            if self.pending[0]:                 # (a recorded step ran on the worker stream of this slot)
                if self._order(cur, self.streams[0].cuda_stream, dev):
                    raise RuntimeError(self.capi.lib().dq_last_error().decode())
                self.pending[0] = False
            if self._enqueue(ref, 15, dev, cur):
                raise RuntimeError(self.capi.lib().dq_last_error().decode())
        else:
            if self._order(handle, cur, dev) or self._enqueue(ref, 15, dev, handle):
                raise RuntimeError(self.capi.lib().dq_last_error().decode())
            self.pending[k] = True
        if self.hist is not None:
            self.hist.count += nsc
        self.superchunks += nsc
        return k

    def run_all(self, pairs):
        """enqueue a whole step's buckets, [(x, out), ...].  A list that has been seen before (the same tensors in the
        same order: DDP's buckets) is replayed from one recorded graph per stream -- one graph launch per stream and
        step instead of one host call per bucket; the first time it runs bucket by bucket, the second time it records."""
        key = tuple((x.data_ptr(), o.data_ptr(), x.numel(), x.dtype) for x, o in pairs)
        entry = self.cache.get(("step", key))
        cur = torch.cuda.current_stream(self.device)
        if entry is None or not self.graphs:
            for x, o in pairs:
                self.run(x, o)
            if entry is None:
                self.cache[("step", key)] = [None, 1]
            return
        graphs, uses = entry
        if graphs is None:
            # per stream: the buckets that go to it, in order, recorded as one graph
            share = [[] for _ in self.streams]
            for (x, o), bkey in zip(pairs, key):
                item = self.cache.get(bkey)
                if item is None:                # (cannot happen after a first eager pass with unchanged scratch)
                    self.run(x, o)
                    item = self.cache[bkey]
                share[item[3]].append(item)
            self.join()
            graphs = []
            for k, st in enumerate(self.streams):
                if not share[k]:
                    graphs.append(None)
                    continue
                g = torch.cuda.CUDAGraph()
                with torch.cuda.stream(st):
                    with torch.cuda.graph(g, stream=st):
                        for item in share[k]:
                            if self._enqueue(item[1], 15, item[2], item[5]):
                                raise RuntimeError(self.capi.lib().dq_last_error().decode())
                graphs.append(g)
            entry[0] = graphs
        # one event for all streams, recorded before the first replay: an event recorded on the caller's stream between
        # two replays could complete only after the first of them (see pick_streams)
        fence = torch.cuda.Event()
        fence.record(cur)
        for k, st in enumerate(self.streams):
            if graphs[k] is not None:
                st.wait_event(fence)
        for k, st in enumerate(self.streams):
            if graphs[k] is None:
                continue
            with torch.cuda.stream(st):
                graphs[k].replay()
            self.pending[k] = True
        entry[1] = uses + 1
        total = sum((x.numel() + 255) // 256 for x, _ in pairs)
        if self.hist is not None:
            self.hist.count += total
        self.superchunks += total

    def counts(self, k):
        """device int32 tensor [n8, n4, n2, other] of the last bucket that ran on stream k"""
        return self.scratch[k]["work"][:4]

    def join(self):
        """the caller's current stream waits for everything enqueued so far"""
        cur = torch.cuda.current_stream(self.device).cuda_stream
        index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        for k, st in enumerate(self.streams):
            if self.pending[k]:
                if self._order(cur, st.cuda_stream, index):
                    raise RuntimeError(self.capi.lib().dq_last_error().decode())
                self.pending[k] = False
