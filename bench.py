#!/usr/bin/env python3
"""Benchmark of the eden_utils compression hot path on one MI355X.

A step = scaling_compress followed by scaling_decompress of one 25 MB DDP
bucket (6,553,600 fp32 gradient elements, Student-t(3) * 1e-3 with 0.1 % of the
entries multiplied by 100), hierarchical AEE (strategy 2), chunk 16, 4-bit
codes, bf16 random pool -- the 25 MB bucket configuration the headline metric
is quoted on.  Inputs are resident in HBM before the timed region; the calls go
through the C ABI of libdynamiq_eden.so.

Prints ONE JSON line.  Headline figures are HBM figures: `value` is fp32
gradient bytes (4 * N) per second of compress + decompress with the step
walking a ring of distinct bucket sets (source, random pool, packed stream,
output) whose footprint exceeds 512 MB, so that every launch streams from and
to memory; `value_cache_assisted` is the same step replaying ONE bucket's
buffers (69 MB, which the 256 MB Infinity Cache serves in part).  `roofline`
prices the dominant kernel (compress) at its algorithmic bytes
(4 + 2 + (q + 0.5625) / 8 per element) against the 8 TB/s HBM peak: `frac` on
the ring of buckets, `frac_cache_assisted` on the replayed bucket.  Every
duration is the median over `--reps` replays of a HIP graph that holds
`--steps` launches, between two events on the stream the graph runs on (the
host's per-call cost is not part of the figure; `eager_ms_per_step` has it).
`roofline.traffic` comes from profiles/hbm_traffic.json (rocprofv3 --pmc
readings of this script, scaled by the copy-kernel calibration), null when the
file has no entry for the kernel and workload.

`configs` holds one entry per cell of the other baseline configurations, each
timed the same way (ring of buffer sets where a set is smaller than the cache)
with a sample of its output compared with the oracle: the 25 MB bucket for
fp32 / bf16 sources x 4 / 8 bits x AEE / MEE; the ring step of the 8 x 124 M
ring on a 15,555,072-element chunk at 5 bits and as the dynamic {2, 4, 8} mix;
the single-pass dynamic-bitrate path per 25 MB bucket of a Llama-3-8B shaped
set; 2^30 fp32 elements: compress / decompress / fused ring step at 2, 4, 5, 8
bits and the transform fused with the codec for blocks 2^10 .. 2^15 x four
widths; and the six rows of the reference's own microbenchmark
(cuda_kernels/tests/benchmark_scaling_quantization.py:60-112).

`cpu_baseline` times the reference's CPU-runnable path for the headline
workload -- the hierarchical chunk quantiser as a torch op sequence
(cpu_baselines.py) -- on all host cores; `cpu_scalar_port` is the scalar C
oracle on one core and `cpu_rht_path` EDEN's torch round trip
(srrcomp.py:293-353) on 2^20 elements.
"""
import argparse
import json
import math
import os
import statistics
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
OVERHEAD_BITS = 0.5625  # hierarchical scale bytes per element, in bits
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
COLD_FOOTPRINT = 640e6   # bytes a ring of buffer sets must exceed


def packed_bytes_per_element(nbits):
    return (nbits + OVERHEAD_BITS) / 8.0


def make_bucket(n, seed, device):
    """Student-t(nu=3) * 1e-3 with 0.1 % outliers * 100, generated on the device."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    z = torch.randn(n, generator=g, device=device)
    chi = torch.randn(3, n, generator=g, device=device).square_().sum(0)
    x = z / torch.sqrt(chi / 3.0) * 1e-3
    idx = torch.randint(0, n, (max(1, n // 1000),), generator=g, device=device)
    x[idx] *= 100.0
    return x.contiguous()


# ---- timing ------------------------------------------------------------------------------------------------

def replay_ms(fn, iters, reps=5, warm=1):
    """per-call device times in ms, one per replay: `iters` calls of fn recorded into one HIP graph on a side stream,
    replayed `warm` times untimed and `reps` times between two events on that stream"""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    out = []
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(iters):
                fn()
        for _ in range(warm):
            graph.replay()
        side.synchronize()
        for _ in range(reps):
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record(side)
            graph.replay()
            end.record(side)
            end.synchronize()
            out.append(start.elapsed_time(end) / iters)
    torch.cuda.current_stream().wait_stream(side)
    return out


def median_ms(fn, iters, reps=5):
    return statistics.median(replay_ms(fn, iters, reps))


def eager_ms(fn, iters):
    """the same with one host call per launch (what a Python caller sees)"""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / iters


class Ring(object):
    """cycles through a list of argument tuples: every call of the timed function gets the next one"""

    def __init__(self, items):
        self.items, self.at = items, 0

    def next(self):
        self.at = (self.at + 1) % len(self.items)
        return self.items[self.at]


def frac(bytes_per_launch, ms):
    return bytes_per_launch / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS


def nmse(x, xhat):
    x = x.double()
    return float(((xhat.double() - x) ** 2).sum() / (x ** 2).sum())


def load_traffic(key):
    """HBM bytes per launch measured with rocprofv3 --pmc for `key`, or None"""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    entry = table.get(key)
    return None if entry is None else entry.get("bytes")


# ---- oracle checks of samples (the checker, not the product) -------------------------------------------------

def host_bits(t):
    t = t.cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy().copy()
    return t.view(torch.int16).numpy().view(np.uint16).copy()


def sample_matches_oracle(O, src, rand, packed, out, nbits, strategy, m):
    """compress + decompress of the first m elements (tiles are independent) against the oracle"""
    odt = O.F32 if src.dtype == torch.float32 else O.BF16
    src_h = host_bits(src[:m])
    rand_h = host_bits(rand[:m].float() if src.dtype == torch.float32 else rand[:m])
    enc_o = O.scaling_compress(src_h, rand_h, m, nbits, 16, strategy, odt)
    nb = O.required_bytes(m, nbits, 16, strategy)
    ok = bool((packed[:nb].cpu().numpy() == enc_o).all())
    if out is not None:
        dec_o = np.zeros(m, src_h.dtype)
        O.scaling_decompress(enc_o, dec_o, m, nbits, 16, strategy, odt)
        ok = ok and bool((host_bits(out[:m]).view(np.uint8) == dec_o.view(np.uint8)).all())
    return ok


# ---- the other configurations ----------------------------------------------------------------------------------

def config2_entries(capi, O, dev, n, steps, reps, sets):
    """the 25 MB bucket: fp32 and bf16 sources, 4 and 8 bits, AEE and MEE, on a ring of `sets` bucket sets"""
    out = []
    base = [make_bucket(n, 100 + k, dev) for k in range(sets)]
    g = torch.Generator(device=dev).manual_seed(7)
    rands = [torch.rand(n, generator=g, device=dev).to(torch.bfloat16) for _ in range(sets)]
    for src_name in ("fp32", "bf16"):
        srcs = base if src_name == "fp32" else [b.to(torch.bfloat16) for b in base]
        outs = [torch.empty_like(s) for s in srcs]
        sbytes = srcs[0].element_size()
        for nbits in (4, 8):
            for strategy in (2, 3):
                nb = capi.required_bytes(n, nbits, 16, strategy)
                packs = [torch.zeros(nb, dtype=torch.uint8, device=dev) for _ in range(sets)]
                ring = Ring(list(zip(srcs, rands, packs, outs)))

                def comp():
                    s, r, p, _ = ring.next()
                    capi.scaling_compress(s, p, r, n, nbits, 16, strategy)

                def dec():
                    _, _, p, o = ring.next()
                    capi.scaling_decompress(p, o, n, nbits, 16, strategy)

                def both():
                    s, r, p, o = ring.next()
                    capi.scaling_compress(s, p, r, n, nbits, 16, strategy)
                    capi.scaling_decompress(p, o, n, nbits, 16, strategy)

                for _ in range(sets):
                    both()
                torch.cuda.synchronize()
                tc, td, ts = median_ms(comp, steps, reps), median_ms(dec, steps, reps), median_ms(both, steps, reps)
                cb = (sbytes + 2 + packed_bytes_per_element(nbits)) * n
                db = (sbytes + packed_bytes_per_element(nbits)) * n
                s0, r0, p0, o0 = ring.items[0]
                out.append({
                    "workload": "config 2: 25 MB bucket, %s source, %d-bit %s, bf16 rand_pool; ring of %d bucket sets"
                                % (src_name, nbits, "AEE" if strategy == 2 else "MEE", sets),
                    "compress_us": round(tc * 1e3, 2), "decompress_us": round(td * 1e3, 2), "step_us": round(ts * 1e3, 2),
                    "compress_frac": round(frac(cb, tc), 4), "decompress_frac": round(frac(db, td), 4),
                    "GBps_fp32_in": round(4.0 * n / (ts * 1e-3) / 1e9, 1),
                    "nmse": float("%.4g" % nmse(base[0], o0)),
                    "bit_exact_vs_oracle": sample_matches_oracle(O, s0, r0, p0, o0, nbits, strategy, 1 << 18),
                })
                del packs, ring
        del outs
    return out


def config3_entries(capi, O, dev, steps, reps):
    """the fused ring step (decode the received chunk, add the local chunk, re-encode) of the 8 x 124,439,808 ring on one
    15,555,072-element bf16 chunk at the 5 bits the configuration states, and the same step of the dynamic {2, 4, 8}
    mix (one launch for the three widths, centring on load, in-kernel rounding stream)"""
    from dynamiq_sigcomm_artifact_amd import bitrate
    out = []
    n = 15555072
    sets = max(3, int(COLD_FOOTPRINT // (n * 4 + 2 * int(n * packed_bytes_per_element(5)))) + 1)
    g = torch.Generator(device=dev).manual_seed(11)
    inps = [(torch.randn(n, generator=g, device=dev) * 3e-3).to(torch.bfloat16) for _ in range(sets)]
    rands = [torch.rand(n, generator=g, device=dev).to(torch.bfloat16) for _ in range(sets)]
    peer = (torch.randn(n, generator=g, device=dev) * 7e-4).to(torch.bfloat16)
    for strategy in (2, 3):
        nbits = 5
        nb = capi.required_bytes(n, nbits, 16, strategy)
        recvs = [torch.zeros(nb, dtype=torch.uint8, device=dev) for _ in range(sets)]
        sends = [torch.zeros(nb, dtype=torch.uint8, device=dev) for _ in range(sets)]
        for k in range(sets):
            capi.scaling_compress(peer, recvs[k], rands[(k + 1) % sets], n, nbits, 16, strategy)
        ring = Ring(list(zip(recvs, inps, sends, rands)))

        def fused():
            rv, ip, sd, rd = ring.next()
            capi.scaling_dec_comp(rv, ip, sd, rd, n, nbits, 16, strategy)

        for _ in range(sets):
            fused()
        torch.cuda.synchronize()
        tf = median_ms(fused, max(4, steps // 2), reps)
        fb = (2 + 2 + 2 * packed_bytes_per_element(nbits)) * n
        rv, ip, sd, rd = ring.items[0]
        m = 1 << 18
        send_o = O.scaling_dec_comp(rv[:O.required_bytes(m, nbits, 16, strategy)].cpu().numpy(), host_bits(ip[:m]),
                                    host_bits(rd[:m]), m, nbits, 16, strategy, O.BF16)
        out.append({
            "workload": "config 3: fused ring step on a 15,555,072-element bf16 ring chunk, 5-bit %s, bf16 rand_pool; ring of "
                        "%d buffer sets" % ("AEE" if strategy == 2 else "MEE", sets),
            "us": round(tf * 1e3, 2), "frac": round(frac(fb, tf), 4), "GBps_bf16_in": round(2.0 * n / (tf * 1e-3) / 1e9, 1),
            "bit_exact_vs_oracle": bool((sd[:send_o.size].cpu().numpy() == send_o).all()),
        })
        del recvs, sends, ring
    del rands
    # the dynamic mix: one rank vector of 8 ring chunks; the step of ring chunk c reads the chunk's superchunks of the
    # vector (2 B/element), their means, the received stream, and writes the stream of the same layout
    W = 8
    nfull = 124439808
    nsc = nfull // 256
    sig = [10.0 ** (-4.0 + 2.0 * k / 7.0) for k in range(W)]
    vec = torch.empty(nfull, dtype=torch.bfloat16, device=dev)
    stats = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
    mean = torch.empty(nsc, dtype=torch.float32, device=dev)
    total = None
    for r in range(W):       # the reduced statistics of eight ranks; the last rank's vector stays as the local operand
        vec.copy_((torch.randn(nfull, generator=g, device=dev) * sig[r]).to(torch.bfloat16))
        capi.superchunk_stats(vec, stats, mean, nfull, W)
        total = stats.clone() if total is None else total.add_(stats)
    u, avg, _ = bitrate.dynamic_bitrate_binary_search_u([total[:, 1]], 4.375)
    order = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
    plan = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=dev)
    capi.group_plan_stats(total, float(u), None, order, plan)
    counts = plan[:3].tolist()
    code_bits = (8 * counts[0] + 4 * counts[1] + 2 * counts[2]) / float(nsc)
    cap = capi.mixed_required_bytes(nsc, W)
    for strategy in (2, 3):
        recv = [torch.zeros(cap, dtype=torch.uint8, device=dev) for _ in range(W)]
        send = [torch.zeros(cap, dtype=torch.uint8, device=dev) for _ in range(W)]
        for c in range(W):
            capi.mixed_compress(vec, order, plan, recv[c], nsc, strategy, seed=5, step=0, center_mean=mean, center_world=W,
                                n=nfull, ring_chunk=c, ring_world=W)
        ring = Ring(list(range(W)))

        def mixed_step():
            c = ring.next()
            capi.mixed_compress(vec, order, plan, send[c], nsc, strategy, seed=6, step=1, recv=recv[c], center_mean=mean,
                                center_world=W, n=nfull, ring_chunk=c, ring_world=W)

        for _ in range(W):
            mixed_step()
        torch.cuda.synchronize()
        tm = median_ms(mixed_step, max(4, steps // 2), reps)
        per_chunk = nfull / W
        mb = (2 + 4.0 / 256 + 2 * (code_bits + OVERHEAD_BITS) / 8.0) * per_chunk
        # sample: the 4-bit run of ring chunk 0 against the oracle's mean-centre + compress + dec_comp on the same rows
        rows = order[nsc:nsc + min(1024, -(-counts[1] // W))].cpu().numpy().astype(np.int64)
        ok = None
        if rows.size:
            sub = host_bits(vec.view(-1, 256)[torch.from_numpy(rows).to(dev)]).reshape(-1)
            res, _ = O.superchunk_mean_center(sub, sub.size, W, O.BF16)
            u0 = (O.philox_uniform_rows(rows, 5, 0).view(np.uint32) >> 16).astype(np.uint16)
            u1 = (O.philox_uniform_rows(rows, 6, 1).view(np.uint32) >> 16).astype(np.uint16)
            first = O.scaling_compress(res, u0, sub.size, 4, 16, strategy, O.BF16)
            second = O.scaling_dec_comp(first, res.copy(), u1, sub.size, 4, 16, strategy, O.BF16)
            off = min(-(-counts[0] // W), counts[0]) * 274          # the 8-bit run of chunk 0 comes first
            ok = bool((send[0][off:off + second.size].cpu().numpy() == second).all())
        out.append({
            "workload": "config 3: fused ring step of the dynamic {2,4,8} mix (%.2f code bits, target 4.375) on the ring chunks of a "
                        "124,439,808-element bf16 rank vector (15.5 M elements per step), %s, centring on load, in-kernel "
                        "rounding stream; the 8 chunks in turn" % (code_bits, "AEE" if strategy == 2 else "MEE"),
            "us": round(tm * 1e3, 2), "frac": round(frac(mb, tm), 4), "GBps_bf16_in": round(2.0 * per_chunk / (tm * 1e-3) / 1e9, 1),
            "bit_exact_vs_oracle": ok,
        })
        del recv, send
    return out


def llama_buckets(dev, count, n=6553600):
    """`count` consecutive 25 MB buckets of a Llama-3-8B shaped gradient set (per-layer tensors in parameter order,
    per-tensor scale log-normal(ln 1e-3, 1.5)), bf16"""
    shapes = [4096 * 4096, 1024 * 4096, 1024 * 4096, 4096 * 4096, 14336 * 4096, 14336 * 4096, 4096 * 14336, 4096, 4096]
    gc = torch.Generator().manual_seed(4)
    g = torch.Generator(device=dev).manual_seed(4)
    out, cur, fill, k = [], torch.empty(n, device=dev), 0, 0
    while len(out) < count:
        left = shapes[k % len(shapes)]
        k += 1
        scale = math.exp(float(torch.randn(1, generator=gc)) * 1.5 + math.log(1e-3))
        while left and len(out) < count:
            m = min(left, n - fill)
            cur[fill:fill + m] = torch.randn(m, generator=g, device=dev) * scale
            fill += m
            left -= m
            if fill == n:
                out.append(cur.to(torch.bfloat16))
                cur, fill = torch.empty(n, device=dev), 0
    return out


def config4_entries(capi, O, dev, reps):
    """the single-pass dynamic-bitrate path per 25 MB bucket through the package's pipeline object: statistics, widths,
    partition, encode (centring on load), decode (mean add) -- eager with one host call per bucket, and recorded with one,
    two and three buckets in flight"""
    from dynamiq_sigcomm_artifact_amd import bitrate
    from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import SinglePassBuckets
    out = []
    n, nb = 6553600, 96         # (a step of the configuration has 1,146 buckets; 96 distinct ones are 2.5 GB of sources and outputs)
    xs = llama_buckets(dev, nb, n)
    outs = [torch.empty_like(x) for x in xs]
    nsc = n // 256
    stats = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
    norms = []
    for x in xs:
        capi.superchunk_stats(x, stats, None, n, 1)
        norms.append(stats[:, 1].clone())
    u, avg, _ = bitrate.dynamic_bitrate_binary_search_u(norms, 4.375)
    pairs = list(zip(xs, outs))
    for streams, graphs, whole in ((1, False, False), (2, False, False), (1, True, True), (2, True, True), (3, True, True)):
        pipe = SinglePassBuckets(dev, strategy=2, seed=3, streams=streams, graphs=graphs, u=u)

        def step():
            pipe.begin_step()
            if whole:
                pipe.run_all(pairs)
            else:
                for x, o in pairs:
                    pipe.run(x, o)
            pipe.join()

        for _ in range(3):          # the first use of a bucket runs eagerly, the second records
            step()
        torch.cuda.synchronize()
        # `rounds` training steps back to back between two events, the host free to run ahead of the device as it is in a
        # training loop (one synchronisation per measurement, not per step)
        ts, rounds = [], 8
        for _ in range(reps):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(rounds):
                step()
            e.record()
            e.synchronize()
            ts.append(s.elapsed_time(e) / (nb * rounds))
        per = statistics.median(ts)
        entry = {
            "workload": "config 4: single-pass dynamic-bitrate path (u = %.2f, %.2f code bits) per 25 MB bf16 bucket of a "
                        "Llama-3-8B shaped set, steps of %d distinct buckets back to back, %s, %d bucket(s) in flight; host calls included"
                        % (u, avg, nb, "one recorded graph per stream and step" if graphs else "eager, one host call per bucket, the first bucket of every round on the caller's own stream", streams),
            "us_per_bucket": round(per * 1e3, 2), "GBps_bf16_in": round(2.0 * n / (per * 1e-3) / 1e9, 1),
        }
        if not graphs and streams == 1:
            # the output of the first bucket against the oracle chain on a sample of its superchunks
            x = xs[0]
            res, st = O.superchunk_mean_center(host_bits(x), n, 1, O.BF16)
            qb = O.dynamic_bitrate_qbits(st[1::2].copy(), u)
            rows = np.nonzero(qb == 4)[0][:512]
            ok = None
            if rows.size:
                uni = (O.philox_uniform_rows(rows, 3, 3 + 8 * reps).view(np.uint32) >> 16).astype(np.uint16)
                enc = O.scaling_compress(res.reshape(-1, 256)[rows].reshape(-1).copy(), uni, rows.size * 256, 4, 16, 2, O.BF16)
                dec = np.zeros(rows.size * 256, np.uint16)
                O.scaling_decompress(enc, dec, dec.size, 4, 16, 2, O.BF16)
                want = O.superchunk_add_mean_copy(dec, st.reshape(-1, 2)[rows].reshape(-1).copy(), dec.size, O.BF16)
                got = host_bits(outs[0].view(-1, 256)[torch.from_numpy(rows).to(dev)]).reshape(-1)
                ok = bool((got == want).all())
            entry["bit_exact_vs_oracle"] = ok
        out.append(entry)
        del pipe
    return out


def config5_entries(capi, O, dev, reps, n=1 << 30):
    out = []
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(n, generator=g, device=dev) * 1e-3
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    dst = torch.empty_like(x)
    m = 1 << 16
    for nbits in (2, 4, 5, 8):
        nb = capi.required_bytes(n, nbits, 16, 2)
        packed = torch.zeros(nb, dtype=torch.uint8, device=dev)
        send = torch.zeros(nb, dtype=torch.uint8, device=dev)
        capi.scaling_compress(x, packed, rand, n, nbits, 16, 2)
        capi.scaling_decompress(packed, dst, n, nbits, 16, 2)
        torch.cuda.synchronize()
        tc = median_ms(lambda: capi.scaling_compress(x, packed, rand, n, nbits, 16, 2), 3, reps)
        td = median_ms(lambda: capi.scaling_decompress(packed, dst, n, nbits, 16, 2), 3, reps)
        tf = median_ms(lambda: capi.scaling_dec_comp(packed, x, send, rand, n, nbits, 16, 2), 3, reps)
        pb = packed_bytes_per_element(nbits)
        out.append({
            "workload": "config 5: 2^30 fp32 N(0, 1e-3^2), %d-bit AEE, bf16 rand_pool" % nbits,
            "compress_us": round(tc * 1e3, 1), "decompress_us": round(td * 1e3, 1), "fused_ring_step_us": round(tf * 1e3, 1),
            "compress_frac": round(frac((4 + 2 + pb) * n, tc), 4), "decompress_frac": round(frac((4 + pb) * n, td), 4),
            "fused_frac": round(frac((4 + 2 + 2 * pb) * n, tf), 4),
            "compress_GBps_fp32_in": round(4.0 * n / (tc * 1e-3) / 1e9, 1),
            "nmse": float("%.4g" % nmse(x[:1 << 24], dst[:1 << 24])),
            "bit_exact_vs_oracle": sample_matches_oracle(O, x, rand, packed, dst, nbits, 2, m),
        })
        del packed, send
    del rand
    # the randomized Hadamard transform fused with the codec: packed Rademacher signs (one bit per element), in-kernel
    # rounding stream; the rotated vector never reaches memory
    sign = torch.empty(n // 32, dtype=torch.int32, device=dev)
    # The first vector-ALU-bound measurements after a stretch of memory-bound work run on a GPU that is still raising its
    # clock (whichever cell comes first reads 15-20 % slow): one measurement of the first cell is taken and thrown away.
    settle = torch.zeros(capi.required_bytes(n, 2, 16, 2), dtype=torch.uint8, device=dev)
    capi.rand_diag_bits(sign, n, 1 << 10)
    for _ in range(2):
        median_ms(lambda: capi.rht_scaling_compress(x, sign, settle, 1 << 10, 1.0 / 32.0, 2, 2, seed=1, step=0), 2, reps)
    del settle
    for kb in (10, 11, 12, 13, 14, 15):
        block = 1 << kb
        scale = 1.0 / math.sqrt(block)
        capi.rand_diag_bits(sign, n, block)
        for nbits in (2, 4, 5, 8):
            nb = capi.required_bytes(n, nbits, 16, 2)
            packed = torch.zeros(nb, dtype=torch.uint8, device=dev)
            tc = median_ms(lambda: capi.rht_scaling_compress(x, sign, packed, block, scale, nbits, 2, seed=1, step=0), 2, reps)
            td = median_ms(lambda: capi.scaling_decompress_irht(packed, sign, dst, block, scale, nbits, 2), 2, reps)
            pb = packed_bytes_per_element(nbits)
            # sample: the first two blocks against the oracle's sign flip + transform + compress (+ decompress + inverse)
            ms = max(2 * block, 1 << 12)
            bits = sign[:ms // 32].cpu().numpy().view(np.uint32)
            sg = np.where((bits[:, None] >> np.arange(32, dtype=np.uint32)) & 1, -1.0, 1.0).astype(np.float32).reshape(-1)
            y_o = O.rht_blocked(x[:ms].cpu().numpy(), sg, block, np.float32(scale))
            uni = O.philox_uniform(ms, 1, 0)
            enc_o = O.scaling_compress(y_o, uni, ms, nbits, 16, 2, O.F32)
            ok = bool((packed[:enc_o.size].cpu().numpy() == enc_o).all())
            dec_o = np.zeros(ms, np.float32)
            O.scaling_decompress(enc_o, dec_o, ms, nbits, 16, 2, O.F32)
            z_o = O.rht_blocked(dec_o, sg, block, np.float32(scale), inverse=True)
            ok = ok and bool((dst[:ms].cpu().numpy().view(np.uint32) == z_o.view(np.uint32)).all())
            out.append({
                "workload": "config 5: 2^30 fp32, randomized Hadamard transform (blocks of 2^%d, packed signs) fused with the "
                            "%d-bit AEE codec, in-kernel rounding stream" % (kb, nbits),
                "compress_us": round(tc * 1e3, 1), "decompress_us": round(td * 1e3, 1),
                "compress_frac": round(frac((4 + 0.125 + pb) * n, tc), 4), "decompress_frac": round(frac((4 + 0.125 + pb) * n, td), 4),
                "roundtrip_GBps_fp32_in": round(4.0 * n / ((tc + td) * 1e-3) / 1e9, 1),
                "bit_exact_vs_oracle": ok,
            })
            del packed
    return out


def reference_table_entries(capi, O, dev, reps, n=16 * 16 * 65536 * 16):
    """cuda_kernels/tests/benchmark_scaling_quantization.py:60-112: bf16, chunk 16, 268,435,456 elements, 2 / 4 / 8 bits x
    strategy 2 / 3; compress, decompress, the ring step as two calls and fused (the reference times eager launches; here
    the launches are replayed from a graph so that only device time is counted)"""
    out = []
    idx = torch.arange(n, dtype=torch.float32, device=dev)
    values = torch.sin(idx * 0.017) * 1.7 + torch.cos(idx * 0.0071) * 0.3
    values += (idx.remainder(7) - 3.0) * 0.013
    src = values.to(torch.bfloat16).contiguous()
    del idx, values
    inp = (src.float() * -0.25).to(torch.bfloat16).contiguous()
    inp_split = inp.clone()
    g = torch.Generator(device=dev).manual_seed(2026)
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    decoded = torch.empty_like(src)
    for nbits in (2, 4, 8):
        for strategy in (2, 3):
            nb = capi.required_bytes(n, nbits, 16, strategy)
            enc = torch.zeros(nb, dtype=torch.uint8, device=dev)
            send = torch.zeros(nb, dtype=torch.uint8, device=dev)
            capi.scaling_compress(src, enc, rand, n, nbits, 16, strategy)
            capi.scaling_decompress(enc, decoded, n, nbits, 16, strategy)
            torch.cuda.synchronize()
            ok = sample_matches_oracle(O, src, rand, enc, decoded, nbits, strategy, 1 << 16)
            tc = median_ms(lambda: capi.scaling_compress(src, enc, rand, n, nbits, 16, strategy), 4, reps)
            td = median_ms(lambda: capi.scaling_decompress(enc, decoded, n, nbits, 16, strategy), 4, reps)

            def split():
                capi.scaling_decompress(enc, inp_split, n, nbits, 16, strategy, add=True)
                capi.scaling_compress(inp_split, send, rand, n, nbits, 16, strategy)

            ts = median_ms(split, 3, reps)
            tf = median_ms(lambda: capi.scaling_dec_comp(enc, inp, send, rand, n, nbits, 16, strategy), 3, reps)
            pb = packed_bytes_per_element(nbits)
            out.append({
                "workload": "reference microbenchmark row: bf16, chunk 16, 268,435,456 elements, %d bits, strategy %d" % (nbits, strategy),
                "compress_ms": round(tc, 4), "decompress_ms": round(td, 4), "split_dec_comp_ms": round(ts, 4),
                "fused_dec_comp_ms": round(tf, 4),
                "compress_frac": round(frac((4 + pb) * n, tc), 4), "decompress_frac": round(frac((2 + pb) * n, td), 4),
                "split_frac": round(frac((pb + 4) * n + (4 + pb) * n, ts), 4), "fused_frac": round(frac((4 + 2 * pb) * n, tf), 4),
                "bit_exact_vs_oracle": ok,
            })
            inp_split.copy_(inp)
            del enc, send
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--reps", type=int, default=7, help="replays of the recorded steps; the median is reported")
    ap.add_argument("--n", type=int, default=6553600, help="gradient elements in the bucket")
    ap.add_argument("--nbits", type=int, default=4)
    ap.add_argument("--strategy", type=int, default=2, help="2 = hierarchical AEE, 3 = hierarchical MEE")
    ap.add_argument("--src", choices=["fp32", "bf16"], default="fp32")
    ap.add_argument("--rand", choices=["pool", "philox"], default="pool",
                    help="pool: the reference's rand_pool tensor (default); philox: uniform values drawn in the kernel")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of each cpu_baseline leg (0 = skip)")
    ap.add_argument("--cold-sets", type=int, default=-1,
                    help="distinct bucket sets (source, random pool, packed, output) the headline walks; default: as many "
                         "as make up 640 MB, at least 10")
    ap.add_argument("--configs", default="2,3,4,5,ref",
                    help="which of the other configurations go into `configs` (comma separated: 2, 3, 4, 5, ref; 'none' = "
                         "headline only, e.g. under a profiler)")
    ap.add_argument("--no-check", action="store_true", help="skip the oracle parity check of a sample")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain elementwise fp32 copy kernel (out = -in) of the same element count, "
                         "4*N bytes read + 4*N bytes written per launch, so that rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE readings can be scaled")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py measures one GPU's share of the path; --gpus must be 1 "
              "(no collectives, sharding or multi-rank code is part of this build)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)

    from dynamiq_sigcomm_artifact_amd import capi
    capi.lib()  # fail loudly when the HIP library is missing

    t_start = time.perf_counter()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n = args.n // 256 * 256
    nbits, strategy, C = args.nbits, args.strategy, 16
    steps, reps = max(1, args.steps), max(1, args.reps)
    sbytes = 4 if args.src == "fp32" else 2
    nb = capi.required_bytes(n, nbits, C, strategy)
    set_bytes = n * sbytes + n * 2 + nb + n * sbytes
    nsets = args.cold_sets if args.cold_sets > 0 else max(10, -(-int(COLD_FOOTPRINT) // set_bytes))

    x32 = make_bucket(n, 0, dev)
    sets = []
    for k in range(nsets):
        xk = x32 if k == 0 else make_bucket(n, k, dev)
        gk = torch.Generator(device=dev)
        gk.manual_seed(1000 + k)
        sk = xk if args.src == "fp32" else xk.to(torch.bfloat16)
        sets.append((sk, torch.rand(n, generator=gk, device=dev).to(torch.bfloat16),
                     torch.zeros(nb, dtype=torch.uint8, device=dev), torch.empty_like(sk)))
    src, rand, packed, out = sets[0]
    ring = Ring(sets)

    def compress_one(s_, p_, r_):
        if args.rand == "philox":
            capi.scaling_compress_philox(s_, p_, n, nbits, C, strategy, 2026, 0)
        else:
            capi.scaling_compress(s_, p_, r_, n, nbits, C, strategy)

    def compress():
        compress_one(src, packed, rand)

    def decompress():
        capi.scaling_decompress(packed, out, n, nbits, C, strategy)

    def step():
        compress()
        decompress()

    def compress_ring():
        s_, r_, p_, _ = ring.next()
        compress_one(s_, p_, r_)

    def decompress_ring():
        _, _, p_, o_ = ring.next()
        capi.scaling_decompress(p_, o_, n, nbits, C, strategy)

    def step_ring():
        s_, r_, p_, o_ = ring.next()
        compress_one(s_, p_, r_)
        capi.scaling_decompress(p_, o_, n, nbits, C, strategy)

    for _ in range(max(args.warmup, nsets)):
        step_ring()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # ---- timed region: `steps` steps per replay, `reps` replays, the median ----
    step_hbm = replay_ms(step_ring, steps, reps)
    ms_per_step = statistics.median(step_hbm)
    comp_hbm_ms = median_ms(compress_ring, steps, reps)
    dec_hbm_ms = median_ms(decompress_ring, steps, reps)
    step_cached = replay_ms(step, steps, reps)
    ms_cached = statistics.median(step_cached)
    comp_ms = median_ms(compress, steps, reps)
    dec_ms = median_ms(decompress, steps, reps)
    torch.cuda.synchronize()

    # ---- what launches of these shapes cost with the arithmetic taken away: the same tiles, the same accesses, over the same
    #      ring (the packed buffers of the ring hold meaningless bytes afterwards; every later use writes them first) ----
    floor_tiles = n // 1024
    run_bytes = nb * 1024 // n if strategy in (2, 3) and n % 1024 == 0 and nbits in (2, 3, 4, 5, 6, 7, 8) else 0
    comp_floor_ms = dec_floor_ms = None
    if run_bytes and run_bytes % 8 == 0:
        def compress_floor():
            s_, r_, p_, _ = ring.next()
            capi.tile_io_floor(0, s_, r_ if args.rand == "pool" else None, p_, run_bytes, floor_tiles)

        def decompress_floor():
            _, _, p_, o_ = ring.next()
            capi.tile_io_floor(1, o_, None, p_, run_bytes, floor_tiles)

        comp_floor_ms = median_ms(compress_floor, steps, reps)
        dec_floor_ms = median_ms(decompress_floor, steps, reps)
        torch.cuda.synchronize()

    t0 = time.perf_counter()
    eager_ms_per_step = eager_ms(step_ring, steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    value = 4.0 * n / (ms_per_step * 1e-3) / 1e9

    comp_bytes = (sbytes + (2 if args.rand == "pool" else 0) + packed_bytes_per_element(nbits)) * n
    dec_bytes = (sbytes + packed_bytes_per_element(nbits)) * n

    if args.pmc_calibration:
        cal_src = torch.empty(n, dtype=torch.float32, device=dev).normal_()
        cal_dst = torch.empty_like(cal_src)
        for _ in range(5):
            torch.neg(cal_src, out=cal_dst)
        torch.cuda.synchronize()

    # ---- quality: NMSE of the round trip ----
    step()
    torch.cuda.synchronize()
    quality = nmse(x32, out)

    # ---- parity of a sample against the oracle (the checker, not the product) ----
    bit_exact = None
    cpu_scalar = None
    O = None
    if not args.no_check or args.cpu_seconds > 0 or args.configs != "none":
        import oracle as O
    if O is not None:
        odt = O.F32 if args.src == "fp32" else O.BF16
        m = min(n, 1 << 20)
        src_h = host_bits(src[:m])
        if args.rand == "philox":
            uni = O.philox_uniform(m, 2026, 0)
            rand_h = uni if args.src == "fp32" else (uni.view(np.uint32) >> 16).astype(np.uint16)   # k/256 is exact in bf16
        else:
            rand_h = host_bits(rand[:m].float() if args.src == "fp32" else rand[:m])
        if not args.no_check:
            enc_o = O.scaling_compress(src_h, rand_h, m, nbits, C, strategy, odt)
            dec_o = np.zeros(m, src_h.dtype)
            O.scaling_decompress(enc_o, dec_o, m, nbits, C, strategy, odt)
            nbm = O.required_bytes(m, nbits, C, strategy)
            bit_exact = bool((packed[:nbm].cpu().numpy() == enc_o).all() and (host_bits(out[:m]) == dec_o).all())
        if args.cpu_seconds > 0:
            count, spent = 0, 0.0
            dec_o = np.zeros(m, src_h.dtype)
            while spent < args.cpu_seconds / 2 and count < 64:
                t1 = time.perf_counter()
                enc_o = O.scaling_compress(src_h, rand_h, m, nbits, C, strategy, odt)
                O.scaling_decompress(enc_o, dec_o, m, nbits, C, strategy, odt)
                spent += time.perf_counter() - t1
                count += 1
            cpu_scalar = {
                "value": round(4.0 * m * count / spent / 1e9, 4),
                "unit": "GB/s",
                "cores": 1,
                "kind": "port",
                "sample": "first %d elements of the same bucket, %d compress+decompress round trips of the scalar C oracle"
                          % (m, count),
            }

    # ---- the other configurations ----
    del ring
    del sets[1:]
    torch.cuda.empty_cache()
    configs, skipped = [], []
    wanted = [] if args.configs == "none" else [c.strip() for c in args.configs.split(",") if c.strip()]
    builders = {
        "2": lambda: config2_entries(capi, O, dev, 6553600, min(steps, 24), min(reps, 5), 16),
        "3": lambda: config3_entries(capi, O, dev, min(steps, 16), min(reps, 5)),
        "4": lambda: config4_entries(capi, O, dev, min(reps, 5)),
        "5": lambda: config5_entries(capi, O, dev, min(reps, 5)),
        "ref": lambda: reference_table_entries(capi, O, dev, min(reps, 5)),
    }
    for name in wanted:
        if name not in builders:
            skipped.append({"config": name, "reason": "unknown"})
            continue
        try:
            t_cfg = time.perf_counter()
            configs.extend(builders[name]())
            print("bench: configuration %s took %.1f s" % (name, time.perf_counter() - t_cfg), file=sys.stderr, flush=True)
        except torch.cuda.OutOfMemoryError as err:
            skipped.append({"config": name, "reason": "out of device memory: %s" % str(err)[:80]})
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    configs_seconds = time.perf_counter() - t_start

    # ---- the reference's CPU-runnable path for this workload on all host cores: the hierarchical chunk quantiser as a
    #      torch op sequence of the shape of the reference's own torch implementation (csrc/logic.py:225-296) ----
    cpu = None
    cpu_rht = None
    if args.cpu_seconds > 0:
        import cpu_baselines as CB
        xc, rc = x32.cpu(), torch.rand(n)
        if strategy == 2:
            sec, count = CB.median_seconds(lambda: CB.hier_roundtrip(xc, rc, nbits), args.cpu_seconds)
            cpu = {
                "value": round(4.0 * n / sec / 1e9, 3),
                "unit": "GB/s",
                "cores": torch.get_num_threads(),
                "kind": "port",
                "sample": "the whole bucket (%d fp32 elements), median of %d compress+decompress round trips of the "
                          "hierarchical chunk-16 quantiser as torch CPU ops (output equal to the oracle's, tests/test_cpu_baselines.py)"
                          % (n, count),
            }
        else:
            cpu = cpu_scalar
        # EDEN's rotate -> Lloyd-Max quantise -> bit planes -> back (srrcomp.py:293-353), the CPU path of the 2^20 configuration
        from dynamiq_sigcomm_artifact_amd.eden import normal_centroids_and_boundaries
        d1 = 1 << 20
        cen, bnd = normal_centroids_and_boundaries(4)
        cen, bnd = cen.float(), bnd.float()
        g1 = torch.Generator().manual_seed(0)
        x1 = torch.randn(d1, generator=g1) * 1e-3
        sec, count = CB.median_seconds(lambda: CB.rht_roundtrip(x1.clone(), 4, 0, cen, bnd), args.cpu_seconds / 2, max_reps=5)
        cpu_rht = {
            "value": round(4.0 * d1 / sec / 1e9, 4),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "2^20 fp32 N(0, 1e-3^2), median of %d EDEN compress+decompress round trips at 4 bits as torch CPU ops "
                      "(randDiag, Hadamard / sqrt(n), bucketize, EdenBinsToBits and back)" % count,
        }

    comp_gbs = comp_bytes / (comp_hbm_ms * 1e-3) / 1e9
    comp_gbs_cached = comp_bytes / (comp_ms * 1e-3) / 1e9
    dec_gbs = dec_bytes / (dec_hbm_ms * 1e-3) / 1e9
    kernel_name = "hier16_compress_kernel"
    traffic_key = "%s|%s|%dbit|strategy%d|%d|%s" % (kernel_name, args.src, nbits, strategy, n, args.rand)
    workload = {
        "workload": "one 25 MB DDP bucket: %d %s gradient elements, Student-t(3)*1e-3 with 0.1%% outliers x100; "
                    "%d-bit hierarchical %s compress + decompress, chunk 16, %s; the step walks a ring of %d distinct bucket "
                    "sets (%.0f MB), every launch streams from and to HBM"
                    % (n, args.src, nbits, "AEE" if strategy == 2 else "MEE",
                       "bf16 rand_pool" if args.rand == "pool" else "in-kernel Philox rounding", nsets, set_bytes * nsets / 1e6),
        "elements": n,
        "nbits": nbits,
        "strategy": strategy,
        "chunk_size": C,
        "source_dtype": args.src,
        "packed_bytes": int(nb),
        "bucket_sets": nsets,
        "configs": configs,
    }
    result = {
        "metric": "compress+decompress GB/s (fp32 grad in) on 1 MI355X, % of HBM peak; NMSE",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": workload,
        "roofline": {
            "bound": "hbm",
            "kernel": kernel_name,
            "achieved": round(comp_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(comp_gbs / HBM_PEAK_GBS, 4),
            "frac_is": "ring of %d distinct bucket sets, every launch streams from and to HBM; frac_cache_assisted replays one "
                       "bucket's buffers (part of its traffic is served by the 256 MB Infinity Cache)" % nsets,
            "frac_cache_assisted": round(comp_gbs_cached / HBM_PEAK_GBS, 4),
            "achieved_cache_assisted": round(comp_gbs_cached, 1),
            "traffic": load_traffic(traffic_key),
            "traffic_key": traffic_key,
            "algorithmic_bytes_per_launch": int(comp_bytes),
            "avg_launch_ms": round(comp_hbm_ms, 5),
            "avg_launch_ms_cache_assisted": round(comp_ms, 5),
            "timing": "median of %d replays of a HIP graph of %d launches" % (reps, steps),
            "io_floor": None if comp_floor_ms is None else {
                "avg_launch_ms": round(comp_floor_ms, 5),
                "frac": round(comp_bytes / (comp_floor_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "kernel_over_floor": round(comp_hbm_ms / comp_floor_ms, 3),
                "what": "dq_tile_io_floor: a kernel of the same launch shape (one wave per tile of 1,024 elements) that reads and "
                        "writes the same bytes of the same ring with the same access pattern and computes nothing, timed the same way",
            },
        },
        "kernels": {
            "compress": {"ms": round(comp_hbm_ms, 5), "algorithmic_GBps": round(comp_gbs, 1), "frac_hbm": round(comp_gbs / HBM_PEAK_GBS, 4),
                         "ms_cache_assisted": round(comp_ms, 5),
                         "io_floor_ms": None if comp_floor_ms is None else round(comp_floor_ms, 5)},
            "decompress": {"ms": round(dec_hbm_ms, 5), "algorithmic_GBps": round(dec_gbs, 1), "frac_hbm": round(dec_gbs / HBM_PEAK_GBS, 4),
                           "ms_cache_assisted": round(dec_ms, 5),
                           "io_floor_ms": None if dec_floor_ms is None else round(dec_floor_ms, 5)},
        },
        "frac_hbm_roundtrip": round((comp_bytes + dec_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "ms_per_step_replays": [round(t, 5) for t in step_hbm],
        "value_cache_assisted": round(4.0 * n / (ms_cached * 1e-3) / 1e9, 2),
        "ms_per_step_cache_assisted": round(ms_cached, 5),
        "nmse": quality,
        "bit_exact_vs_oracle": bit_exact,
        "eager_ms_per_step": round(eager_ms_per_step, 5),
        "host_wall_ms_per_step": round(wall_ms, 5),
        "configs": configs,
        "configs_skipped": skipped,
        "configs_seconds": round(configs_seconds, 1),
        "cpu_baseline": cpu,
        "cpu_scalar_port": cpu_scalar,
        "cpu_rht_path": cpu_rht,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
