#!/usr/bin/env python3
"""Runs the synthetic workloads of the build's baseline configurations on one GPU
and prints one JSON line per measurement (NMSE, GB/s, fraction of the 8 TB/s HBM
peak).  ``python evaluate.py --config 1|2|3|4|5``.  A measurement tool beside
``bench.py``; the library does not import it.

  1  2^20 fp32 N(0,1e-3^2): blocked randomized Hadamard + quantise + pack and back
  2  25 MB bucket, Student-t with outliers: 4/8-bit round trips, fp32 and bf16
  3  8 simulated ranks x 124,439,808 elements: compressed ring all-reduce
  4  Llama-3-8B shaped gradient set in 25 MB buckets: dynamic {2,4,8}-bit allocation
  5  2^30 fp32: compress / decompress / fused sweep, and the blocked transform
``--kernels`` times every entry point of the library on one 25 MB bucket.
``--reference-benchmark`` prints the table of the reference's own microbenchmark
(cuda_kernels/tests/benchmark_scaling_quantization.py:60-112: bf16, chunk 16, 268,435,456 elements,
2/4/8 bits x strategy 2/3, eager launches through the eden_utils module) with the fraction of the HBM peak.

Timings: 10 warm-up launches, then 50 launches replayed from a HIP graph between two
events (cuda_kernels/tests/benchmark_scaling_quantization.py:41-57 times eager launches;
the graph keeps the host's per-call cost out of the figure).
"""
import argparse
import json
import math
import os
import sys
import types

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import cpu_baselines                                                                       # noqa: E402
from dynamiq_sigcomm_artifact_amd import bitrate, capi                                     # noqa: E402
from dynamiq_sigcomm_artifact_amd.compressors import Aee_Dynamic_Range_GPU_kern, Mee_Dynamic_Range_GPU_kern   # noqa: E402
from dynamiq_sigcomm_artifact_amd.dynamiq_pipeline import (dynamic_bitrate_allreduce,     # noqa: E402
                                                           dynamic_bitrate_allreduce_grouped,
                                                           dynamic_bitrate_allreduce_single_pass, pick_streams)
from dynamiq_sigcomm_artifact_amd.ring_sim import ring_allreduce, split_chunks             # noqa: E402

HBM_PEAK = 8000.0  # GB/s
OV = 0.5625        # scale overhead, bits per element


def _time_us(fn, warmup=10, iters=50):
    """average device time of one fn() in microseconds: `iters` launches recorded into one HIP graph and
    replayed between two events, so the host's per-call cost (several microseconds through ctypes) does
    not sit between the launches"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(iters):
                fn()
    graph.replay()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    graph.replay()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) / iters * 1e3


def _nmse(x, xhat):
    x = x.double()
    return float(((xhat.double() - x) ** 2).sum() / (x ** 2).sum())


def _emit(**kw):
    print(json.dumps(kw), flush=True)


def _student_bucket(n, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    z = torch.randn(n, generator=g, device=dev)
    chi = torch.randn(3, n, generator=g, device=dev).square_().sum(0)
    x = z / torch.sqrt(chi / 3.0) * 1e-3
    idx = torch.randint(0, n, (max(1, n // 1000),), generator=g, device=dev)
    x[idx] *= 100.0
    return x.contiguous()


def config1(dev):
    n = 1 << 20
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(n, generator=g, device=dev) * 1e-3
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    sign = torch.empty(n, device=dev)
    capi.rand_diag(sign, 0)
    sign_bits = capi.pack_signs(sign)
    for kb in (10, 11, 12, 13, 14, 15, 20):
        B = 1 << kb
        scale = 1.0 / math.sqrt(B)
        for nbits in (4, 5, 8):
            y = x.clone()
            capi.rht_blocked(y, sign, B, scale, False)
            packed = torch.zeros(capi.required_bytes(n, nbits, 16, 2), dtype=torch.uint8, device=dev)
            capi.scaling_compress(y, packed, rand, n, nbits, 16, 2)
            z = torch.empty_like(y)
            capi.scaling_decompress(packed, z, n, nbits, 16, 2)
            capi.rht_blocked(z, sign, B, scale, True)
            plain = torch.empty_like(x)
            packed2 = torch.zeros_like(packed)
            capi.scaling_compress(x, packed2, rand, n, nbits, 16, 2)
            capi.scaling_decompress(packed2, plain, n, nbits, 16, 2)
            t_rht = _time_us(lambda: capi.rht_blocked(y, sign, B, scale, False))
            line = dict(config=1, block=B, nbits=nbits, nmse_rht=_nmse(x, z), nmse_no_rht=_nmse(x, plain),
                        rht_us=round(t_rht, 2), rht_GBps=round(8.0 * n / t_rht / 1e3, 1))
            if kb <= 15:
                # the same round trip with the transform fused into the codec: same bytes, two launches instead of four
                fused = torch.zeros_like(packed)
                capi.rht_scaling_compress(x, sign_bits, fused, B, scale, nbits, 2, rand_pool=rand)
                zf = torch.empty_like(x)
                capi.scaling_decompress_irht(fused, sign_bits, zf, B, scale, nbits, 2)
                t4 = _time_us(lambda: (capi.rht_blocked(y, sign, B, scale, False),
                                       capi.scaling_compress(y, packed, rand, n, nbits, 16, 2),
                                       capi.scaling_decompress(packed, z, n, nbits, 16, 2),
                                       capi.rht_blocked(z, sign, B, scale, True)))
                t2 = _time_us(lambda: (capi.rht_scaling_compress(x, sign_bits, fused, B, scale, nbits, 2, rand_pool=rand),
                                       capi.scaling_decompress_irht(fused, sign_bits, zf, B, scale, nbits, 2)))
                y2 = x.clone()
                capi.rht_blocked(y2, sign, B, scale, False)
                capi.scaling_compress(y2, packed, rand, n, nbits, 16, 2)
                line.update(fused_bytes_equal=bool(torch.equal(fused, packed)), nmse_fused=_nmse(x, zf),
                            roundtrip_4_launches_us=round(t4, 2), roundtrip_fused_us=round(t2, 2),
                            roundtrip_fused_GBps_fp32_in=round(4.0 * n / t2 / 1e3, 1))
            _emit(**line)
    # the reference-legal path for this configuration: EDEN (whole-vector rotation, Lloyd-Max bins, bit planes)
    from dynamiq_sigcomm_artifact_amd.eden import Eden
    eden = Eden(device=dev)
    for nbits in (4, 5, 8):
        data = eden.compress(x, nbits, 0)
        rec = eden.decompress(data)
        cen, bnd = eden._tables(nbits)
        y = x.clone()
        capi.rht_blocked(y, sign, n, 1.0 / math.sqrt(n), False)
        packed = torch.empty(n // 32 * nbits, dtype=torch.int32, device=dev)
        result = torch.empty(4, device=dev)
        work = torch.empty(capi.eden_work_doubles(n), dtype=torch.float64, device=dev)
        out = torch.empty(n, device=dev)
        tq = _time_us(lambda: capi.eden_quantize(y, bnd, cen, nbits, packed, result, work))
        td = _time_us(lambda: capi.eden_dequantize(packed, n, cen, nbits, out))
        _emit(config=1, path="eden", nbits=nbits, nmse=_nmse(x, rec), slices=len(data), quantize_us=round(tq, 2),
              dequantize_us=round(td, 2), quantize_GBps=round((8.0 + nbits / 8.0) * n / tq / 1e3, 1),
              dequantize_GBps=round((4.0 + nbits / 8.0) * n / td / 1e3, 1))


def config2(dev):
    n = 6553600
    x32 = _student_bucket(n, dev)
    g = torch.Generator(device=dev).manual_seed(1)
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    for src_name, src in (("fp32", x32), ("bf16", x32.to(torch.bfloat16))):
        sb = src.element_size()
        for strategy in (2, 3):
            for nbits in (4, 8):
                packed = torch.zeros(capi.required_bytes(n, nbits, 16, strategy), dtype=torch.uint8, device=dev)
                out = torch.empty_like(src)
                capi.scaling_compress(src, packed, rand, n, nbits, 16, strategy)
                capi.scaling_decompress(packed, out, n, nbits, 16, strategy)
                tc = _time_us(lambda: capi.scaling_compress(src, packed, rand, n, nbits, 16, strategy))
                td = _time_us(lambda: capi.scaling_decompress(packed, out, n, nbits, 16, strategy))
                pb = (nbits + OV) / 8
                _emit(config=2, source=src_name, strategy=strategy, nbits=nbits, nmse=_nmse(x32, out),
                      compress_us=round(tc, 2), decompress_us=round(td, 2),
                      roundtrip_GBps_of_fp32_input=round(4.0 * n / (tc + td) / 1e3, 1),
                      compress_frac_hbm=round((sb + 2 + pb) * n / tc / 1e3 / HBM_PEAK, 4),
                      decompress_frac_hbm=round((sb + pb) * n / td / 1e3 / HBM_PEAK, 4))
    # the flat quantiser (strategy 0) next to the same quantiser written as torch CPU ops: two independent
    # implementations of one formula, different random draws
    for nbits in (4, 8):
        packed = torch.zeros(capi.required_bytes(n, nbits, 16, 0), dtype=torch.uint8, device=dev)
        out = torch.empty_like(x32)
        capi.scaling_compress(x32, packed, rand, n, nbits, 16, 0)
        capi.scaling_decompress(packed, out, n, nbits, 16, 0)
        cpu_nmse = _cpu_torch_line(x32, nbits)
        gpu_nmse = _nmse(x32, out)
        _emit(config=2, source="fp32", strategy=0, nbits=nbits, nmse=gpu_nmse, nmse_cpu_torch=cpu_nmse,
              nmse_ratio=round(gpu_nmse / cpu_nmse, 4))


_torch_cpu_roundtrip = cpu_baselines.flat_roundtrip


def _cpu_torch_line(x32, nbits):
    """median of 5 round trips on torch's intra-op thread pool (its size follows OMP_NUM_THREADS), one warm-up"""
    import time
    threads = torch.get_num_threads()
    xc = x32.cpu()
    rc = torch.rand(xc.numel())
    _torch_cpu_roundtrip(xc, rc, nbits)
    ts = []
    for _ in range(5):
        t0 = time.perf_counter()
        out = _torch_cpu_roundtrip(xc, rc, nbits)
        ts.append(time.perf_counter() - t0)
    ts.sort()
    nmse = _nmse(xc, out)
    _emit(config=2, path="cpu torch op sequence (csrc/logic.py:225-296)", nbits=nbits, threads=threads,
          roundtrip_ms=round(ts[2] * 1e3, 2), roundtrip_GBps_of_fp32_input=round(4.0 * xc.numel() / ts[2] / 1e9, 3),
          nmse=nmse)
    return nmse


def _params(d, W, r):
    return {"d": {(0, 0): d}, "world_size": W, "rank": r, "args": types.SimpleNamespace(aggregation_method="dynamiQ")}


def config3(dev, n=124439808, W=8):
    g = torch.Generator(device=dev).manual_seed(0)
    sig = torch.pow(10.0, torch.rand(W, generator=g, device=dev) * 2.0 - 4.0)   # log-uniform [1e-4, 1e-2]
    npad = (n + 255) // 256 * 256
    exact = torch.zeros(npad, dtype=torch.float64, device=dev)
    grads = []
    for r in range(W):
        x = torch.zeros(npad, device=dev)
        x[:n] = torch.randn(n, generator=g, device=dev) * sig[r]
        exact += x.double()
        grads.append(x.to(torch.bfloat16))          # the DDP hook hands bf16 buckets to the compressor
        del x
    for nbits in (4, 5, 8):
        for cls, name in ((Aee_Dynamic_Range_GPU_kern, "aee"), (Mee_Dynamic_Range_GPU_kern, "mee")):
            gen = torch.Generator(device=dev).manual_seed(7)
            comps = [cls(nbits, 16, _params(npad, W, r), generator=gen) for r in range(W)]
            vecs = [x.clone() for x in grads]
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            ring_allreduce(vecs, comps)
            e.record()
            e.synchronize()
            ms = s.elapsed_time(e)
            same = all(torch.equal(vecs[0], v) for v in vecs[1:])
            # one fused reduce-scatter step of one rank on its ring chunk
            chunk = split_chunks(vecs[0], W, 256)[0]
            m = chunk.numel()
            recv = comps[0].create_tensor(chunk, torch.uint8)
            send = comps[0].create_tensor(chunk, torch.uint8)
            comps[0].compression(chunk, recv)
            t = _time_us(lambda: comps[0].dec_compression(recv, chunk, send), 5, 25)
            pb = (nbits + OV) / 8
            _emit(config=3, world=W, elements_per_rank=n, nbits=nbits, method=name, nmse_vs_fp64_sum=_nmse(exact, vecs[0]),
                  ranks_identical=same, ring_total_ms=round(ms, 3), step_elements=m, step_us=round(t, 2),
                  step_GBps_algorithmic=round((2 + 2 + 2 * pb) * m / t / 1e3, 1),
                  step_frac_hbm=round((2 + 2 + 2 * pb) * m / t / 1e3 / HBM_PEAK, 4))
            del vecs, comps
    # "5 bits" as the dynamic {2, 4, 8} mix (target 5 - 0.625 code bits): mean-centre, allocate, one grouped ring per width
    target = 5.0 - bitrate.DYNAMIC_BITRATE_HEADROOM
    from dynamiq_sigcomm_artifact_amd.compressors import superchunk_mean_center
    nsc = npad // 256
    norms = torch.zeros(nsc, dtype=torch.bfloat16, device=dev)
    res = torch.empty(npad, dtype=torch.bfloat16, device=dev)
    st = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
    for r in range(W):
        superchunk_mean_center(grads[r], res, st, npad, W, 256)
        norms += st[:, 1]
    del res, st
    u, avg_bits, _ = bitrate.dynamic_bitrate_binary_search_u([norms], target)
    for cls, name in ((Aee_Dynamic_Range_GPU_kern, "aee"), (Mee_Dynamic_Range_GPU_kern, "mee")):
        gen = torch.Generator(device=dev).manual_seed(7)
        comps = {q: [cls(q, 16, _params(npad, W, r), generator=gen) for r in range(W)] for q in (2, 4, 8)}
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        outs, _, qbits = dynamic_bitrate_allreduce_grouped(grads, u, comps)
        e.record()
        e.synchronize()
        same = all(torch.equal(outs[0], v) for v in outs[1:])
        _emit(config=3, world=W, elements_per_rank=n, nbits="dynamic{2,4,8}", method=name, pipeline="grouped", u=u,
              avg_code_bits=float(qbits.float().mean()), nmse_vs_fp64_mean=_nmse(exact / W, outs[0]),
              ranks_identical=same, pipeline_total_ms=round(s.elapsed_time(e), 3))
        del outs, comps
        # the same all-reduce with one codec launch per ring step for the three widths and no residual buffers
        work = {}
        strategy = 2 if name == "aee" else 3
        for timed in (False, True):             # the first call allocates the stream buffers
            s.record()
            outs, _, counts = dynamic_bitrate_allreduce_single_pass(grads, u, strategy=strategy, seed=7, work=work)
            e.record()
            e.synchronize()
        c = counts.tolist()
        same = all(torch.equal(outs[0], v) for v in outs[1:])
        _emit(config=3, world=W, elements_per_rank=n, nbits="dynamic{2,4,8}", method=name, pipeline="single_pass", u=u,
              avg_code_bits=(8 * c[0] + 4 * c[1] + 2 * c[2]) / max(1, sum(c[:3])), nmse_vs_fp64_mean=_nmse(exact / W, outs[0]),
              ranks_identical=same, pipeline_total_ms=round(s.elapsed_time(e), 3))
        del outs, work


LLAMA3_8B = [("embed", 128256 * 4096)] + [
    (name, numel) for _ in range(32) for name, numel in (
        ("q", 4096 * 4096), ("k", 1024 * 4096), ("v", 1024 * 4096), ("o", 4096 * 4096),
        ("gate", 14336 * 4096), ("up", 14336 * 4096), ("down", 4096 * 14336))]


def _llama_buckets(dev, bucket=6553600, limit=None):
    """yields fp32 buckets of the flattened gradient set; per-tensor scale log-normal(ln 1e-3, 1.5)"""
    g = torch.Generator(device=dev).manual_seed(0)
    gs = torch.Generator().manual_seed(1)
    scales = torch.exp(torch.randn(len(LLAMA3_8B), generator=gs) * 1.5 + math.log(1e-3)).tolist()
    buf = torch.empty(bucket, device=dev)
    fill, count = 0, 0
    for (name, numel), sc in zip(LLAMA3_8B, scales):
        left = numel
        while left > 0:
            take = min(left, bucket - fill)
            buf[fill:fill + take] = torch.randn(take, generator=g, device=dev) * sc
            fill += take
            left -= take
            if fill == bucket:
                yield buf
                count += 1
                if limit and count >= limit:
                    return
                fill = 0
    if fill:
        yield buf[:fill // 256 * 256]


def _offset_search_lines(dev, norms_list, target, u_ref):
    """the once-per-step search for u over the norms of every bucket: the reference's torch op sequence (one pass over
    all norms and one read-back per probe) against the histogram of norm patterns (one small launch per bucket while the
    step runs, one launch and one read-back for the search)"""
    import time
    stats = []
    for t in norms_list:
        st = torch.zeros((t.numel(), 2), dtype=torch.bfloat16, device=dev)
        st[:, 1] = t
        stats.append(st)
    hist = bitrate.NormHistogram(dev)

    def wall(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            out = fn()
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        return best * 1e3, out

    def hist_search(mode, prev):
        for st in stats:
            hist.add(st)
        return hist.binary_search_u(target) if mode == 0 else hist.adjust_u(prev, target)

    nsc = sum(t.numel() for t in norms_list)
    for name, ref_fn, mode, prev in (
            ("bisection (first compressed step)", lambda: bitrate.dynamic_bitrate_binary_search_u(norms_list, target), 0, 0.0),
            ("correction from u + 1.5 (later steps)", lambda: bitrate.dynamic_bitrate_adjust_u(norms_list, u_ref + 1.5, target),
             1, u_ref + 1.5)):
        ms_ref, want = wall(ref_fn)
        ms_hist, got = wall(lambda: hist_search(mode, prev))
        _emit(config=4, pipeline="offset search: " + name, buckets=len(norms_list), superchunks=nsc,
              torch_op_sequence_ms=round(ms_ref, 3), histogram_ms=round(ms_hist, 3), probes=int(hist.result[3]),
              same_result=bool(tuple(want) == tuple(got)), u=got[0])
    add_us = _time_us(lambda: hist.add(stats[0]))
    hist.hist.zero_()
    # an empty histogram never meets the tolerance: all 33 probes, the longest the search launch can take
    search_us = _time_us(lambda: capi.bitrate_search(hist.hist, 0, 0.0, target, hist.result))
    _emit(config=4, pipeline="offset search: device time", histogram_add_us_per_bucket=round(add_us, 2),
          search_launch_us_33_probes=round(search_us, 2))


def config4(dev, limit=None):
    target = 5.0 - bitrate.DYNAMIC_BITRATE_HEADROOM
    from dynamiq_sigcomm_artifact_amd.compressors import superchunk_mean_center
    # pass 1: norms of every superchunk -> u
    norms_list = []
    for b in _llama_buckets(dev, limit=limit):
        x = b.to(torch.bfloat16)
        n = x.numel()
        res = torch.empty(n, dtype=torch.bfloat16, device=dev)
        st = torch.empty((n // 256, 2), dtype=torch.bfloat16, device=dev)
        superchunk_mean_center(x, res, st, n, 1, 256)
        norms_list.append(st[:, 1].clone())
    u, avg_bits, delta = bitrate.dynamic_bitrate_binary_search_u(norms_list, target)
    _offset_search_lines(dev, norms_list, target, u)
    # pass 2: quantise, with the reference's op sequence and with the gather/scatter folded into the kernels
    # an untimed pass of the op sequence first: its index_select / nonzero results have a different size in every
    # bucket, and the first pass pays the allocator for each of them
    gen = torch.Generator(device=dev).manual_seed(3)
    warm = {q: [Aee_Dynamic_Range_GPU_kern(q, 16, _params(6553600 * 8, 1, 0), generator=gen)] for q in (2, 4, 8)}
    for b in _llama_buckets(dev, limit=limit):
        dynamic_bitrate_allreduce([b.to(torch.bfloat16)], u, warm)
    del warm
    for cls, name in ((Aee_Dynamic_Range_GPU_kern, "aee"), (Mee_Dynamic_Range_GPU_kern, "mee")):
        for pipe_name, pipe in (("sequence", dynamic_bitrate_allreduce), ("grouped", dynamic_bitrate_allreduce_grouped),
                                ("grouped+device_qbits", dynamic_bitrate_allreduce_grouped)):
            gen = torch.Generator(device=dev).manual_seed(3)
            comps = {q: [cls(q, 16, _params(6553600 * 8, 1, 0), generator=gen)] for q in (2, 4, 8)}
            kw = {} if pipe_name == "sequence" else {"work": {}, "device_qbits": pipe_name.endswith("device_qbits")}
            num = den = 0.0
            bits = elems = 0
            check = 0
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            times = []
            for b in _llama_buckets(dev, limit=limit):
                x = b.to(torch.bfloat16)
                s.record()
                outs, _, qbits = pipe([x], u, comps, **kw)
                e.record()
                e.synchronize()
                times.append((s.elapsed_time(e), x.numel()))
                num += float(((outs[0].double() - b.double()) ** 2).sum())
                den += float((b.double() ** 2).sum())
                bits += int(qbits.sum())
                elems += qbits.numel()
                check ^= int(outs[0].view(torch.int16).to(torch.int64).sum()) & 0xFFFFFFFF
            timed = times[3:] if len(times) > 3 else times       # the first buckets pay the one-time allocations
            gpu_ms = sum(t for t, _ in timed)
            _emit(config=4, method=name, pipeline=pipe_name, buckets=len(times), elements=elems * 256, target_avg_bits=target,
                  u=u, search_avg_bits=avg_bits, achieved_avg_code_bits=bits / elems,
                  achieved_bits_with_scales=bits / elems + OV, nmse=num / den, output_checksum=check,
                  ms_per_25MB_bucket=round(gpu_ms / len(timed), 4),
                  pipeline_GBps_of_bf16_input=round(2.0 * sum(m for _, m in timed) / (gpu_ms * 1e-3) / 1e9, 1))
        # everything on the device, one launch for the three widths; eager, then captured once and replayed
        strategy = 2 if name == "aee" else 3
        for graphed in (False, True):
            work, graph, src, out = {}, None, None, None
            num = den = 0.0
            bits = elems = 0
            check = 0
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            times = []
            for b in _llama_buckets(dev, limit=limit):
                x = b.to(torch.bfloat16)
                if graphed and src is None:
                    src, out = torch.empty_like(x), [torch.empty_like(x)]
                    src.copy_(x)
                    dynamic_bitrate_allreduce_single_pass([src], u, strategy=strategy, seed=3, out=out, work=work)
                    torch.cuda.synchronize()
                    side = torch.cuda.Stream()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.stream(side):
                        with torch.cuda.graph(graph, stream=side):
                            _, _, counts = dynamic_bitrate_allreduce_single_pass([src], u, strategy=strategy, seed=3, out=out,
                                                                                 work=work, stream=side.cuda_stream)
                if graphed and x.numel() == src.numel():
                    src.copy_(x)
                    s.record()
                    graph.replay()
                    e.record()
                    outs = out
                else:
                    s.record()
                    outs, _, counts = dynamic_bitrate_allreduce_single_pass([x], u, strategy=strategy, seed=3,
                                                                            work=None if graphed else work)
                    e.record()
                e.synchronize()
                times.append((s.elapsed_time(e), x.numel()))
                num += float(((outs[0].double() - b.double()) ** 2).sum())
                den += float((b.double() ** 2).sum())
                c = counts.tolist()
                bits += 8 * c[0] + 4 * c[1] + 2 * c[2]
                elems += sum(c[:3])
                check ^= int(outs[0].view(torch.int16).to(torch.int64).sum()) & 0xFFFFFFFF
            timed = times[3:] if len(times) > 3 else times
            gpu_ms = sum(t for t, _ in timed)
            _emit(config=4, method=name, pipeline="single_pass+graph" if graphed else "single_pass", buckets=len(times),
                  elements=elems * 256, u=u, achieved_avg_code_bits=bits / elems, achieved_bits_with_scales=bits / elems + OV,
                  nmse=num / den, output_checksum=check, ms_per_25MB_bucket=round(gpu_ms / len(timed), 4),
                  pipeline_GBps_of_bf16_input=round(2.0 * sum(m for _, m in timed) / (gpu_ms * 1e-3) / 1e9, 1))
    config4_streams(dev, u)


def config4_streams(dev, u, nbuckets=48, rounds=8):
    """Back-to-back buckets with no host work between them.  The launches of `nbuckets` buckets are captured into one
    graph per stream (each stream takes every k-th bucket; every capture is an ordinary single-stream one) and the
    graphs are replayed side by side: with several streams the small launches of a bucket -- statistics, plan -- overlap
    the codec launches of its neighbours."""
    xs = [b.to(torch.bfloat16).clone() for b in _llama_buckets(dev, limit=nbuckets)]
    keep = []                                   # graphs and streams stay alive until the function returns
    target = 5.0 - bitrate.DYNAMIC_BITRATE_HEADROOM
    # (streams, closed loop): in the closed loop the plans read u from device memory, every bucket adds its norms to the
    # histogram and a round ends with the correction of u for the next one -- a whole training step without a read-back
    for nstreams, closed in ((1, False), (2, False), (3, False), (4, False), (1, True), (2, True)):
        streams, _ = pick_streams(dev, nstreams)          # streams that share no hardware queue with each other or with `main`
        graphs = []
        hist = bitrate.NormHistogram(dev) if closed else None
        if closed:
            hist.result[0] = u
        for k, st in enumerate(streams):
            work, out = {}, [torch.empty_like(xs[0])]

            def share():
                for x in xs[k::nstreams]:
                    dynamic_bitrate_allreduce_single_pass([x], hist.result[0:1] if closed else u, strategy=2, seed=3, out=out,
                                                          work=work, norm_histogram=hist)

            with torch.cuda.stream(st):
                share()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(st):
                with torch.cuda.graph(g, stream=st):
                    share()
            graphs.append(g)
            keep.append((g, st, work, out))
        main = torch.cuda.current_stream()

        def replay_all():
            fence = torch.cuda.Event()
            fence.record(main)                   # one event before the first replay, not one between replays
            for st in streams:
                st.wait_event(fence)
            for g, st in zip(graphs, streams):
                with torch.cuda.stream(st):
                    g.replay()
            for st in streams:
                main.wait_stream(st)
            if closed:
                hist.launch_search(1, hist.result[0:1], target)

        replay_all()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(rounds):
            replay_all()
        e.record()
        e.synchronize()
        per = s.elapsed_time(e) / (rounds * len(xs))
        name = "single_pass, %d buckets replayed as graphs" % len(xs)
        extra = {}
        if closed:
            name += " + norm histogram + search for the next u (u read from device memory)"
            extra = dict(u_after_rounds=float(hist.result[0]), probes_last_search=int(hist.result[3]))
        _emit(config=4, method="aee", pipeline=name, streams=nstreams, rounds=rounds, ms_per_25MB_bucket=round(per, 4),
              pipeline_GBps_of_bf16_input=round(2.0 * xs[0].numel() / (per * 1e-3) / 1e9, 1), **extra)
    torch.cuda.synchronize()


def config5(dev, n=1 << 30):
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(n, generator=g, device=dev) * 1e-3
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    out = torch.empty_like(x)
    for nbits in (2, 4, 5, 8):
        packed = torch.zeros(capi.required_bytes(n, nbits, 16, 2), dtype=torch.uint8, device=dev)
        send = torch.zeros_like(packed)
        capi.scaling_compress(x, packed, rand, n, nbits, 16, 2)
        tc = _time_us(lambda: capi.scaling_compress(x, packed, rand, n, nbits, 16, 2), 3, 10)
        td = _time_us(lambda: capi.scaling_decompress(packed, out, n, nbits, 16, 2), 3, 10)
        tf = _time_us(lambda: capi.scaling_dec_comp(packed, x, send, rand, n, nbits, 16, 2), 3, 10)
        pb = (nbits + OV) / 8
        _emit(config=5, op="quantise", nbits=nbits, nmse=_nmse(x, out), compress_us=round(tc, 1), decompress_us=round(td, 1),
              fused_us=round(tf, 1), compress_GBps_fp32_in=round(4.0 * n / tc / 1e3, 1),
              compress_frac_hbm=round((4 + 2 + pb) * n / tc / 1e3 / HBM_PEAK, 4),
              decompress_frac_hbm=round((4 + pb) * n / td / 1e3 / HBM_PEAK, 4),
              fused_frac_hbm=round((4 + 2 + 2 * pb) * n / tf / 1e3 / HBM_PEAK, 4))
        del packed, send
    del out, rand
    sign = torch.empty(n, device=dev)
    capi.rand_diag(sign, 0)
    for kb in (10, 11, 12, 13, 14, 15):
        B = 1 << kb
        t = _time_us(lambda: capi.rht_blocked(x, sign, B, 1.0, False), 2, 5)
        _emit(config=5, op="rht_blocked", block=B, us=round(t, 1), GBps=round(12.0 * n / t / 1e3, 1),
              frac_hbm=round(12.0 * n / t / 1e3 / HBM_PEAK, 4))
    # the transform fused with the quantiser: the rotated vector never reaches memory (the in-place transforms
    # above have changed x: draw it again)
    x = torch.randn(n, generator=g, device=dev) * 1e-3
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    out = torch.empty_like(x)
    sign_bits = capi.pack_signs(sign)
    for kb, nbits in ((10, 4), (13, 2), (13, 4), (13, 5), (13, 8), (15, 4)):
        B = 1 << kb
        sc = 1.0 / math.sqrt(B)
        packed = torch.zeros(capi.required_bytes(n, nbits, 16, 2), dtype=torch.uint8, device=dev)
        tp = _time_us(lambda: capi.rht_scaling_compress(x, sign, packed, B, sc, nbits, 2, rand_pool=rand), 2, 5)
        tx = _time_us(lambda: capi.rht_scaling_compress(x, sign, packed, B, sc, nbits, 2, seed=1, step=0), 2, 5)
        td = _time_us(lambda: capi.scaling_decompress_irht(packed, sign, out, B, sc, nbits, 2), 2, 5)
        tb = _time_us(lambda: capi.rht_scaling_compress(x, sign_bits, packed, B, sc, nbits, 2, seed=1, step=0), 2, 5)
        tdb = _time_us(lambda: capi.scaling_decompress_irht(packed, sign_bits, out, B, sc, nbits, 2), 2, 5)
        pb = (nbits + OV) / 8
        _emit(config=5, op="rht+quantise fused", block=B, nbits=nbits, nmse=_nmse(x, out),
              compress_pool_us=round(tp, 1), compress_philox_us=round(tx, 1), decompress_us=round(td, 1),
              compress_pool_frac_hbm=round((4 + 4 + 2 + pb) * n / tp / 1e3 / HBM_PEAK, 4),
              compress_philox_frac_hbm=round((4 + 4 + pb) * n / tx / 1e3 / HBM_PEAK, 4),
              decompress_frac_hbm=round((4 + 4 + pb) * n / td / 1e3 / HBM_PEAK, 4),
              packed_signs_compress_philox_us=round(tb, 1), packed_signs_decompress_us=round(tdb, 1),
              packed_signs_compress_frac_hbm=round((4 + 0.125 + pb) * n / tb / 1e3 / HBM_PEAK, 4),
              packed_signs_decompress_frac_hbm=round((4 + 0.125 + pb) * n / tdb / 1e3 / HBM_PEAK, 4),
              roundtrip_GBps_fp32_in=round(4.0 * n / (tb + tdb) / 1e3, 1))
        del packed
    t = _time_us(lambda: capi.hadamard(x), 1, 3)
    _emit(config=5, op="hadamard_whole_vector", n=n, us=round(t, 1))


def kernels(dev, n=6553600):
    """every entry point of the library on one 25 MB bucket (n elements): device time per call and the fraction of
    the 8 TB/s HBM peak its algorithmic bytes amount to"""
    g = torch.Generator(device=dev).manual_seed(0)
    x32 = torch.randn(n, generator=g, device=dev) * 1e-3
    nsc = n // 256

    def line(name, fn, nbytes, **kw):
        t = _time_us(fn)
        _emit(kernel=name, us=round(t, 2), algorithmic_MB=round(nbytes / 1e6, 2), GBps=round(nbytes / t / 1e3, 1),
              frac_hbm=round(nbytes / t / 1e3 / HBM_PEAK, 4), **kw)

    # scaling quantisation: every element type and strategy at chunk 16, 4 and 8 bits
    for tdt, name, sb in ((torch.float32, "fp32", 4), (torch.bfloat16, "bf16", 2), (torch.float16, "fp16", 2)):
        src = x32.to(tdt)
        rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16 if tdt != torch.float16 else tdt)
        out = torch.empty_like(src)
        for strategy in (2, 3, 0, 1):
            for nbits in (4, 8):
                nb = capi.required_bytes(n, nbits, 16, strategy)
                packed = torch.zeros(nb, dtype=torch.uint8, device=dev)
                send = torch.zeros_like(packed)
                rnd = rand              # a bf16 pool beside fp32 elements as well
                capi.scaling_compress(src, packed, rnd, n, nbits, 16, strategy)
                tag = dict(elements=name, strategy=strategy, nbits=nbits)
                line("scaling_compress", lambda: capi.scaling_compress(src, packed, rnd, n, nbits, 16, strategy),
                     (sb + 2) * n + nb, **tag)
                line("scaling_decompress", lambda: capi.scaling_decompress(packed, out, n, nbits, 16, strategy),
                     sb * n + nb, **tag)
                line("scaling_decompress_add", lambda: capi.scaling_decompress(packed, out, n, nbits, 16, strategy, add=True),
                     2 * sb * n + nb, **tag)
                if strategy >= 2 and tdt != torch.float16:
                    line("scaling_dec_comp (fused)", lambda: capi.scaling_dec_comp(packed, src, send, rnd, n, nbits, 16, strategy),
                         (sb + 2) * n + 2 * nb, **tag)
        if tdt != torch.float16:
            # the launch of the chunk-16 codec's shape with the arithmetic taken away, over the same buffers: what the 4-bit
            # lines above can be held against (the bytes named are those of the codec call of that shape)
            nb4 = capi.required_bytes(n, 4, 16, 2)
            packed4 = torch.zeros(nb4, dtype=torch.uint8, device=dev)
            run = nb4 * 1024 // n
            line("tile_io_floor (encoder shape: elements + pool read, records written)",
                 lambda: capi.tile_io_floor(0, src, rand, packed4, run, n // 1024), (sb + 2) * n + nb4, elements=name, nbits=4)
            line("tile_io_floor (encoder shape without a pool)",
                 lambda: capi.tile_io_floor(0, src, None, packed4, run, n // 1024), sb * n + nb4, elements=name, nbits=4)
            line("tile_io_floor (decoder shape: records read, elements written)",
                 lambda: capi.tile_io_floor(1, out, None, packed4, run, n // 1024), sb * n + nb4, elements=name, nbits=4)
        del src, rand, out
    # chunk sizes other than 16: the thread-per-chunk kernels
    src = x32.to(torch.bfloat16)
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    out = torch.empty_like(src)
    for C in (8, 32):
        nb = capi.required_bytes(n, 4, C, 2)
        packed = torch.zeros(nb, dtype=torch.uint8, device=dev)
        line("scaling_compress", lambda: capi.scaling_compress(src, packed, rand, n, 4, C, 2), 4 * n + nb,
             elements="bf16", strategy=2, nbits=4, chunk_size=C)
        line("scaling_decompress", lambda: capi.scaling_decompress(packed, out, n, 4, C, 2), 2 * n + nb,
             elements="bf16", strategy=2, nbits=4, chunk_size=C)
    # superchunk statistics, groups
    res = torch.empty_like(src)
    stats = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
    line("superchunk_mean_center", lambda: capi.superchunk_mean_center(src, res, stats, n, 8), 4 * n + 4 * nsc, elements="bf16")
    line("superchunk_add_mean_copy", lambda: capi.superchunk_add_mean_copy(res, out, stats, n), 4 * n + 2 * nsc, elements="bf16")
    order = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
    work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=dev)
    qbits = torch.empty(nsc, dtype=torch.int64, device=dev)
    u, _, _ = bitrate.dynamic_bitrate_binary_search_u([stats[:, 1]], 4.375)
    line("group_plan_stats", lambda: capi.group_plan_stats(stats, u, qbits, order, work), 4 * nsc + 12 * nsc, superchunks=nsc)
    line("group_plan", lambda: capi.group_plan(qbits, order, work), 8 * nsc + 4 * nsc, superchunks=nsc)
    # the fixed-proportion allocation: stable descending sort of the norms, top 35 % / bottom 20 % (x_5bit)
    line("group_plan_sorted", lambda: capi.group_plan_sorted(stats, int(nsc * 0.35), int(nsc * 0.2), order, work), 4 * nsc + 4 * nsc,
         superchunks=nsc)
    # the search for u: the norm patterns of the bucket into the histogram; the whole bisection on an empty histogram
    # (never meets the tolerance: all 33 probes)
    hist = torch.zeros(capi.bitrate_hist_ints(), dtype=torch.int32, device=dev)
    found = torch.zeros(4, dtype=torch.float64, device=dev)
    line("norm_histogram", lambda: capi.norm_histogram(stats, hist), 4 * nsc, superchunks=nsc)
    hist.zero_()
    line("bitrate_search", lambda: capi.bitrate_search(hist, 0, 0.0, 4.375, found), 8 * hist.numel(), probes=33)
    # statistics without the residual, then the three widths of the plan in one launch (centring folded into the load,
    # rounding stream drawn in the kernel) and back (mean added on the store)
    mean32 = torch.empty(nsc, dtype=torch.float32, device=dev)
    line("superchunk_stats", lambda: capi.superchunk_stats(src, stats, mean32, n, 8), 2 * n + 8 * nsc, elements="bf16")
    capi.group_plan_stats(stats, u, None, order, work)
    counts = work[:3]
    n8, n4, n2 = (int(c) for c in counts.tolist())
    stream_bytes = 274 * n8 + 146 * n4 + 82 * n2
    mixed = torch.zeros(capi.mixed_required_bytes(nsc), dtype=torch.uint8, device=dev)
    line("mixed_compress (centred load)",
         lambda: capi.mixed_compress(src, order, counts, mixed, nsc, 2, seed=1, step=0, center_mean=mean32, center_world=8, n=n),
         2 * n + 4 * nsc + 4 * nsc + stream_bytes, elements="bf16", groups=[n8, n4, n2])
    mixed2 = torch.zeros_like(mixed)
    line("mixed_compress (fused ring step: decode recv, add, centre, encode)",
         lambda: capi.mixed_compress(src, order, counts, mixed2, nsc, 2, seed=1, step=1, recv=mixed, center_mean=mean32,
                                     center_world=8, n=n),
         2 * n + 4 * nsc + 4 * nsc + 2 * stream_bytes, elements="bf16", groups=[n8, n4, n2])
    line("mixed_decompress (+mean)", lambda: capi.mixed_decompress(mixed, out, order, counts, nsc, 2, stats=stats),
         2 * n + 4 * nsc + 4 * nsc + stream_bytes, elements="bf16", groups=[n8, n4, n2])
    rows = torch.arange(0, nsc, 2, dtype=torch.int32, device=dev)
    nr = rows.numel()
    nb = capi.required_bytes(nr * 256, 4, 16, 2)
    packed = torch.zeros(nb, dtype=torch.uint8, device=dev)
    line("scaling_compress_rows", lambda: capi.scaling_compress_rows(res, rows, packed, rand, nr, 4, 2), 4 * nr * 256 + nb + 4 * nr,
         elements="bf16", rows="every second superchunk")
    line("scaling_decompress_rows (+mean)", lambda: capi.scaling_decompress_rows(packed, out, rows, stats, n, nr, 4, 2),
         2 * nr * 256 + nb + 8 * nr, elements="bf16", rows="every second superchunk")
    del src, rand, out, res
    # transforms: whole-vector Hadamard on the padded bucket (THC: d = 2^23), blocked RHT
    d = 1 << 23
    y = torch.randn(d, generator=g, device=dev)
    sign = torch.empty(d, device=dev)
    line("rand_diag", lambda: capi.rand_diag(sign, 0), 4 * d, n=d)
    dbits = torch.empty(d // 32, dtype=torch.int32, device=dev)
    line("rand_diag_bits", lambda: capi.rand_diag_bits(dbits, d, 0), d // 8, n=d)
    line("Hadamard (whole vector)", lambda: capi.hadamard(y), 16 * d, n=d, passes=2)
    y.normal_(generator=g)
    line("rht_blocked (whole vector, sign + scale)", lambda: capi.rht_blocked(y, sign, d, 1.0, False), 20 * d, n=d, passes=2)
    for kb in (10, 15):
        y.normal_(generator=g)
        line("rht_blocked", lambda: capi.rht_blocked(y, sign, 1 << kb, 1.0, False), 12 * d, n=d, block=1 << kb)
    # consumers of the rotated vector
    from dynamiq_sigcomm_artifact_amd.eden import normal_centroids_and_boundaries
    y.normal_(generator=g)
    for nbits in (4, 8):
        cen, bnd = (t.to(dev) for t in normal_centroids_and_boundaries(nbits))
        packed = torch.empty(d // 32 * nbits, dtype=torch.int32, device=dev)
        result = torch.empty(4, device=dev)
        work64 = torch.empty(capi.eden_work_doubles(d), dtype=torch.float64, device=dev)
        out = torch.empty(d, device=dev)
        line("eden_quantize", lambda: capi.eden_quantize(y, bnd, cen, nbits, packed, result, work64), 8 * d + d // 8 * nbits, n=d, nbits=nbits)
        line("eden_dequantize", lambda: capi.eden_dequantize(packed, d, cen, nbits, out), 4 * d + d // 8 * nbits, n=d, nbits=nbits)
    # EDEN end to end on the padded bucket (srrcomp.py:293-354): fresh diagonal, rotation, quantiser -- with the float
    # diagonal and with the diagonal as bits
    cen, bnd = (t.to(dev) for t in normal_centroids_and_boundaries(4))
    packed = torch.empty(d // 32 * 4, dtype=torch.int32, device=dev)
    inv_d = 1.0 / math.sqrt(d)
    line("eden compress: rand_diag + rht_blocked + eden_quantize", lambda: (
        capi.rand_diag(sign, 1), capi.rht_blocked(y, sign, d, inv_d, False),
        capi.eden_quantize(y, bnd, cen, 4, packed, result, work64)), 4 * d + 20 * d + 8.5 * d, n=d, nbits=4, launches=7)
    line("eden compress: rand_diag_bits + rht_blocked + eden_quantize", lambda: (
        capi.rand_diag_bits(dbits, d, 1), capi.rht_blocked(y, dbits, d, inv_d, False),
        capi.eden_quantize(y, bnd, cen, 4, packed, result, work64)), 0.125 * d + 16.125 * d + 8.5 * d, n=d, nbits=4, launches=7)
    line("eden decompress: eden_dequantize + rand_diag_bits + inverse rht_blocked", lambda: (
        capi.eden_dequantize(packed, d, cen, 4, out), capi.rand_diag_bits(dbits, d, 1),
        capi.rht_blocked(out, dbits, d, inv_d, True)), 4.5 * d + 0.125 * d + 16.125 * d, n=d, nbits=4, launches=4)
    line("eden decompress: rand_diag_bits + eden_dequantize_irht (folded, scale included)", lambda: (
        capi.rand_diag_bits(dbits, d, 1),
        capi.eden_dequantize_irht(packed, d, cen, 4, dbits, out, d, inv_d, post_scale=result[2:3])),
        0.125 * d + 0.5 * d + 0.125 * d + 12 * d, n=d, nbits=4, launches=3)
    uni = torch.rand(d, generator=g, device=dev)
    lev = torch.empty(d, dtype=torch.bfloat16, device=dev)
    lo, delta = torch.tensor([-4.0], device=dev), torch.tensor([8.0 / 63], device=dev)
    line("thc_quantize", lambda: capi.thc_quantize(y, uni, lev, lo, delta, 64), 10 * d, n=d)
    line("thc_dequantize", lambda: capi.thc_dequantize(lev, y, delta, lo), 6 * d, n=d)
    # THC end to end on the padded bucket: rotation and quantiser as separate calls and folded into the transform's passes
    inv = 1.0 / math.sqrt(d)
    line("thc: rht_blocked + thc_quantize", lambda: (capi.rht_blocked(y, sign, d, inv, False),
                                                      capi.thc_quantize(y, uni, lev, lo, delta, 64)), 30 * d, n=d, launches=3)
    line("thc_rht_quantize (folded)", lambda: capi.thc_rht_quantize(y, sign, uni, lev, d, inv, lo, delta, 64), 22 * d, n=d,
         launches=2)
    line("thc: thc_dequantize + inverse rht_blocked", lambda: (capi.thc_dequantize(lev, y, delta, lo),
                                                                capi.rht_blocked(y, sign, d, inv, True)), 26 * d, n=d, launches=3)
    line("thc_dequantize_irht (folded)", lambda: capi.thc_dequantize_irht(lev, sign, y, d, inv, delta, lo), 18 * d, n=d,
         launches=2)
    # the same with the diagonal as packed bits
    sbits = capi.pack_signs(sign)
    for kb in (10, 15):
        y.normal_(generator=g)
        line("rht_blocked (packed signs)", lambda: capi.rht_blocked(y, sbits, 1 << kb, 1.0, False), 8.125 * d, n=d, block=1 << kb)
    line("thc_rht_quantize (folded, packed signs)", lambda: capi.thc_rht_quantize(y, sbits, uni, lev, d, inv, lo, delta, 64),
         18.125 * d, n=d, launches=2)
    line("thc_dequantize_irht (folded, packed signs)", lambda: capi.thc_dequantize_irht(lev, sbits, y, d, inv, delta, lo),
         14.125 * d, n=d, launches=2)
    # the transform folded into the hierarchical codec (blocks of 2^13, 4-bit)
    x32 = torch.randn(d, generator=g, device=dev) * 1e-3
    sign_bits = capi.pack_signs(sign)
    pk = torch.zeros(capi.required_bytes(d, 4, 16, 2), dtype=torch.uint8, device=dev)
    pb = (4 + OV) / 8
    line("rht_scaling_compress (packed signs, in-kernel rounding stream)",
         lambda: capi.rht_scaling_compress(x32, sign_bits, pk, 8192, 1.0 / math.sqrt(8192), 4, 2, seed=1, step=0),
         (4 + 0.125 + pb) * d, n=d, block=8192, nbits=4)
    line("scaling_decompress_irht (packed signs)",
         lambda: capi.scaling_decompress_irht(pk, sign_bits, x32, 8192, 1.0 / math.sqrt(8192), 4, 2),
         (4 + 0.125 + pb) * d, n=d, block=8192, nbits=4)
    bins = torch.randint(0, 32, (d,), generator=g, device=dev, dtype=torch.int32)
    arr = torch.empty(d // 32 * 5, dtype=torch.int32, device=dev)
    line("EdenBinsToBits", lambda: capi.bins_to_bits(bins, arr, 5), 4 * d + d // 32 * 5 * 4, n=d, nbits=5)
    line("EdenBitsToBins", lambda: capi.bits_to_bins(bins, arr, 5), 4 * d + d // 32 * 5 * 4, n=d, nbits=5)
    line("quantization_compression", lambda: capi.quantization(y, 0.5, 15.0, 1), 8 * d, n=d)


def quantiser_sizes(dev, nbits=4):
    """the production quantiser (bf16, chunk 16, hierarchical) at the three sizes that matter: one 25 MB bucket, one ring
    chunk of the 8 x 124,439,808 configuration, and 2^28 elements (beyond every cache): compress, decompress and the
    fused ring step for AEE and MEE, graph-replayed"""
    for n in (6553600, 15555072, 1 << 28):
        g = torch.Generator(device=dev).manual_seed(n & 0xffff)
        src = (torch.randn(n, generator=g, device=dev) * 1e-3).to(torch.bfloat16)
        inp = (torch.randn(n, generator=g, device=dev) * 1e-3).to(torch.bfloat16)
        rnd = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
        out = torch.empty_like(src)
        pk = (nbits + OV) / 8.0
        iters = 10 if n > (1 << 27) else 50
        for strategy, name in ((2, "aee"), (3, "mee")):
            enc = torch.zeros(capi.required_bytes(n, nbits, 16, strategy), dtype=torch.uint8, device=dev)
            send = torch.zeros_like(enc)
            capi.scaling_compress(src, enc, rnd, n, nbits, 16, strategy)
            for op, fn, bpe in (("compress", lambda: capi.scaling_compress(src, enc, rnd, n, nbits, 16, strategy), 4 + pk),
                                ("decompress", lambda: capi.scaling_decompress(enc, out, n, nbits, 16, strategy), 2 + pk),
                                ("dec_comp", lambda: capi.scaling_dec_comp(enc, inp, send, rnd, n, nbits, 16, strategy), 4 + 2 * pk)):
                t = _time_us(fn, 5, iters)
                _emit(sizes=True, op=op, method=name, n=n, nbits=nbits, us=round(t, 2), GBps_algorithmic=round(bpe * n / t / 1e3, 1),
                      frac_hbm=round(bpe * n / t / 1e3 / HBM_PEAK, 4))
            del enc, send
        del src, inp, rnd, out


def long_bucket(dev, sizes=(1 << 26, 1 << 28)):
    """the kernels of the dynamic-bitrate pipeline on buckets of the size the reference trains with
    (bucket_cap_mb=4000, testbed_evaluation/train_llm_causal.py:416: up to 2 * 10^9 bf16 elements in one bucket):
    statistics, plan, the three-width codec with centring on load and the mean added on store, and the single-width
    codec beside them; bf16, target 4.375 bits, in-kernel rounding stream, graph-replayed"""
    for n in sizes:
        nsc = n // 256
        g = torch.Generator(device=dev).manual_seed(3)
        scale = torch.exp(torch.randn(nsc, 1, generator=g, device=dev) * 1.5 - 7)
        src = (torch.randn(nsc, 256, generator=g, device=dev) * scale).reshape(-1).to(torch.bfloat16)
        stats = torch.empty((nsc, 2), dtype=torch.bfloat16, device=dev)
        mean32 = torch.empty(nsc, dtype=torch.float32, device=dev)
        iters = 10 if n > (1 << 27) else 30
        rows = []
        rows.append(("superchunk_stats", _time_us(lambda: capi.superchunk_stats(src, stats, mean32, n, 8), 3, iters), 2.0 * n))
        u, _, _ = bitrate.dynamic_bitrate_binary_search_u([stats[:, 1]], 4.375)
        order = torch.empty(3 * nsc, dtype=torch.int32, device=dev)
        work = torch.zeros(capi.group_plan_work_ints(nsc), dtype=torch.int32, device=dev)
        rows.append(("group_plan_stats", _time_us(lambda: capi.group_plan_stats(stats, u, None, order, work), 3, iters), 4.0 * nsc + 4.0 * nsc))
        counts = work[:3].clone()
        n8, n4, n2 = (int(c) for c in counts.tolist())
        sb = 274 * n8 + 146 * n4 + 82 * n2
        mixed = torch.zeros(capi.mixed_required_bytes(nsc), dtype=torch.uint8, device=dev)
        mixed2 = torch.zeros_like(mixed)
        out = torch.empty_like(src)
        rows.append(("mixed_compress (centred load)", _time_us(
            lambda: capi.mixed_compress(src, order, counts, mixed, nsc, 2, seed=1, step=0, center_mean=mean32, center_world=8, n=n),
            3, iters), 2.0 * n + sb))
        rows.append(("mixed_compress (fused ring step)", _time_us(
            lambda: capi.mixed_compress(src, order, counts, mixed2, nsc, 2, seed=1, step=1, recv=mixed, center_mean=mean32,
                                        center_world=8, n=n), 3, iters), 2.0 * n + 2.0 * sb))
        rows.append(("mixed_decompress (+mean)", _time_us(
            lambda: capi.mixed_decompress(mixed, out, order, counts, nsc, 2, stats=stats, n_limit=n), 3, iters), 2.0 * n + sb))
        packed = torch.zeros(capi.required_bytes(n, 4, 16, 2), dtype=torch.uint8, device=dev)
        rows.append(("scaling_compress_philox (4-bit)", _time_us(
            lambda: capi.scaling_compress_philox(src, packed, n, 4, 16, 2, 1, 0), 3, iters), 2.0 * n + packed.numel()))
        rows.append(("scaling_decompress (4-bit)", _time_us(
            lambda: capi.scaling_decompress(packed, out, n, 4, 16, 2), 3, iters), 2.0 * n + packed.numel()))
        for name, t, nbytes in rows:
            _emit(long_bucket=True, kernel=name, elements=n, groups=[n8, n4, n2], us=round(t, 1),
                  GBps_algorithmic=round(nbytes / t / 1e3, 1), frac_hbm=round(nbytes / t / 1e3 / HBM_PEAK, 4))
        del src, stats, mean32, order, work, mixed, mixed2, out, packed


def mfma_experiment(dev, n=1 << 28, block=8192):
    """the transform fused with the quantiser (4-bit AEE, packed signs, in-kernel rounding stream), its first four stages
    as add / subtract butterflies (the library's kernel) and as a product with the +-1 matrix on the matrix cores"""
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(n, generator=g, device=dev) * 1e-3
    sign = torch.empty(n // 32, dtype=torch.int32, device=dev)
    capi.rand_diag_bits(sign, n, 1)
    scale = 1.0 / math.sqrt(block)
    nbytes = capi.required_bytes(n, 4, 16, 2)
    a, b = (torch.zeros(nbytes, dtype=torch.uint8, device=dev) for _ in range(2))
    bytes_per = (4 + 0.125 + (4 + OV) / 8) * n
    variants = (("butterflies (VALU)", lambda: capi.rht_scaling_compress(x, sign, a, block, scale, 4, 2, seed=3, step=1)),
                ("H16 on the matrix cores (v_mfma_f32_16x16x4_f32)",
                 lambda: capi.rht_scaling_compress_mfma16(x, sign, b, block, scale, seed=3, step=1)))
    times = {name: [] for name, _ in variants}
    for _ in range(5):                      # alternating, so that clock and box drift hit both alike
        for name, fn in variants:
            times[name].append(_time_us(fn, 3, 10))
    for name, _ in variants:
        ts = sorted(times[name])
        _emit(mfma_experiment=True, first_four_stages=name, n=n, block=block, us_median=round(ts[2], 1), us_min=round(ts[0], 1),
              us_max=round(ts[-1], 1), frac_hbm_median=round(bytes_per / ts[2] / 1e3 / HBM_PEAK, 4))
    out_a, out_b = torch.empty_like(x), torch.empty_like(x)
    capi.scaling_decompress_irht(a, sign, out_a, block, scale, 4, 2)
    capi.scaling_decompress_irht(b, sign, out_b, block, scale, 4, 2)
    _emit(mfma_experiment=True, bytes_differing=float((a != b).float().mean()), nmse_butterflies=_nmse(x, out_a), nmse_matrix_cores=_nmse(x, out_b))


def fused_transform(dev, n=1 << 28, blocks=(1 << 10, 1 << 13, 1 << 15)):
    """the blocked randomized Hadamard transform alone and fused with the 4-bit AEE codec (packed signs, in-kernel rounding
    stream) for three block sizes: the launches whose LDS bank conflicts and vector-ALU load the counter runs look at"""
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(n, generator=g, device=dev) * 1e-3
    y = x.clone()
    out = torch.empty_like(x)
    sign = torch.empty(n // 32, dtype=torch.int32, device=dev)
    capi.rand_diag_bits(sign, n, 1)
    packed = torch.zeros(capi.required_bytes(n, 4, 16, 2), dtype=torch.uint8, device=dev)
    pb = (4 + OV) / 8

    # Three rounds over the block sizes, the median per size: the first measurements of a process run on a GPU that is
    # still raising its clock (whichever block size comes first reads 350-380 us instead of 295), and a median over
    # rounds drops them where a warm-up of a fixed length did not.
    times = {block: ([], [], []) for block in blocks}
    for _ in range(3):
        for block in blocks:
            scale = 1.0 / math.sqrt(block)
            tc, td, tb = times[block]
            tc.append(_time_us(lambda: capi.rht_scaling_compress(x, sign, packed, block, scale, 4, 2, seed=3, step=1), 3, 8))
            td.append(_time_us(lambda: capi.scaling_decompress_irht(packed, sign, out, block, scale, 4, 2), 3, 8))
            tb.append(_time_us(lambda: capi.rht_blocked(y, sign, block, scale, False), 3, 8))
    for block in blocks:
        tc, td, tb = (sorted(t)[1] for t in times[block])
        _emit(fused_transform=True, n=n, block=block, compress_us=round(tc, 1), decompress_us=round(td, 1), rht_blocked_us=round(tb, 1),
              compress_frac_hbm=round((4 + 0.125 + pb) * n / tc / 1e3 / HBM_PEAK, 4),
              decompress_frac_hbm=round((4 + 0.125 + pb) * n / td / 1e3 / HBM_PEAK, 4),
              rht_blocked_frac_hbm=round((8 + 0.125) * n / tb / 1e3 / HBM_PEAK, 4))


def reference_benchmark(dev, n=16 * 16 * 65536 * 16):
    """cuda_kernels/tests/benchmark_scaling_quantization.py:60-112 on this GPU, through the drop-in module: the same
    inputs (:31-39), the same eager timing loops (:41-57; 10 warm-up + 50 launches, 5 + 25 for the two ring-step
    variants), the same CSV columns, plus the fraction of the 8 TB/s HBM peak each time amounts to for the
    algorithmic bytes of the call (2 + 2 + (q + 0.5625) / 8 per element for compress, ...)."""
    import dynamiq_sigcomm_artifact_amd as pkg
    eden_utils = pkg.load_eden_utils()
    torch.manual_seed(2026)
    stream = torch.cuda.current_stream().cuda_stream

    def time_ms(fn, warmup=10, iters=50):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / iters

    print("device=%s" % torch.cuda.get_device_name(0), flush=True)
    print("dtype,chunk_size,nbits,strategy,compress_ms,decompress_ms,split_dec_comp_ms,fused_dec_comp_ms,"
          "frac_hbm_compress,frac_hbm_decompress,frac_hbm_split,frac_hbm_fused", flush=True)
    chunk_size, dtype = 16, torch.bfloat16
    idx = torch.arange(n, dtype=torch.float32, device=dev)
    values = torch.sin(idx * 0.017) * 1.7 + torch.cos(idx * 0.0071) * 0.3
    values += (idx.remainder(7) - 3.0) * 0.013
    src = values.to(dtype).contiguous()
    del idx, values
    inp_template = (src.float() * -0.25).to(dtype).contiguous()
    rand_pool = torch.rand(n, dtype=torch.float32, device=dev).to(dtype).contiguous()
    for nbits in (2, 4, 8):
        for strategy in (2, 3):
            encoded = torch.zeros(capi.required_bytes(n, nbits, chunk_size, strategy), dtype=torch.uint8, device=dev)
            send = torch.zeros_like(encoded)
            send_split = torch.zeros_like(encoded)
            decoded = torch.empty_like(src)
            inp = inp_template.clone()
            inp_split = inp_template.clone()
            eden_utils.scaling_compress(src, encoded, rand_pool, n, nbits, chunk_size, stream, strategy)
            torch.cuda.synchronize()
            c_ms = time_ms(lambda: eden_utils.scaling_compress(src, encoded, rand_pool, n, nbits, chunk_size, stream, strategy))
            d_ms = time_ms(lambda: eden_utils.scaling_decompress(encoded, decoded, n, nbits, chunk_size, stream, strategy))
            s_ms = time_ms(lambda: (eden_utils.scaling_decompress_add(encoded, inp_split, n, nbits, chunk_size, stream, strategy),
                                    eden_utils.scaling_compress(inp_split, send_split, rand_pool, n, nbits, chunk_size, stream, strategy)),
                           warmup=5, iters=25)
            f_ms = time_ms(lambda: eden_utils.scaling_dec_comp(encoded, inp, send, rand_pool, n, nbits, chunk_size, stream, strategy),
                           warmup=5, iters=25)
            pk = (nbits + OV) / 8.0
            frac = lambda bytes_per_elem, ms: bytes_per_elem * n / (ms * 1e-3) / 1e9 / HBM_PEAK
            print("%s,%d,%d,%d,%.4f,%.4f,%.4f,%.4f,%.3f,%.3f,%.3f,%.3f"
                  % (dtype, chunk_size, nbits, strategy, c_ms, d_ms, s_ms, f_ms, frac(4 + pk, c_ms), frac(2 + pk, d_ms),
                     frac((pk + 4) + (4 + pk), s_ms), frac(4 + 2 * pk, f_ms)), flush=True)
            del encoded, send, send_split, decoded, inp, inp_split


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--kernels", action="store_true", help="time every entry point of the library on a 25 MB bucket")
    ap.add_argument("--quantiser-sizes", action="store_true",
                    help="compress / decompress / fused step of the production quantiser (bf16, 4-bit, AEE and MEE) at 25 MB, at "
                         "the ring-chunk size of the 8-rank configuration and at 2^28 elements")
    ap.add_argument("--long-bucket", action="store_true",
                    help="the kernels of the dynamic-bitrate pipeline at 2^26 and 2^28 bf16 elements in one bucket")
    ap.add_argument("--mfma-experiment", action="store_true",
                    help="the transform fused with the quantiser (blocks of 8192) with its first four stages as butterflies and on the matrix cores")
    ap.add_argument("--fused-transform", action="store_true",
                    help="the blocked transform alone and fused with the 4-bit codec at 2^28 elements for blocks of 2^10, 2^13, 2^15")
    ap.add_argument("--reference-benchmark", action="store_true",
                    help="the table of cuda_kernels/tests/benchmark_scaling_quantization.py with the fraction of the HBM peak")
    ap.add_argument("--limit", type=int, default=None, help="config 4: number of 25 MB buckets to process")
    ap.add_argument("--n", type=int, default=None, help="configs 3 and 5: element count override")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("evaluate needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.kernels:
        kernels(dev, **({"n": args.n} if args.n else {}))
        return
    if args.quantiser_sizes:
        quantiser_sizes(dev)
        return
    if args.long_bucket:
        long_bucket(dev)
        return
    if args.mfma_experiment:
        mfma_experiment(dev, **({"n": args.n} if args.n else {}))
        return
    if args.fused_transform:
        fused_transform(dev, **({"n": args.n} if args.n else {}))
        return
    if args.reference_benchmark:
        reference_benchmark(dev, **({"n": args.n} if args.n else {}))
        return
    if args.config is None:
        raise SystemExit("give --config N, --kernels, --quantiser-sizes or --reference-benchmark")
    if args.config == 1:
        config1(dev)
    elif args.config == 2:
        config2(dev)
    elif args.config == 3:
        config3(dev, **({"n": args.n} if args.n else {}))
    elif args.config == 4:
        config4(dev, args.limit)
    else:
        config5(dev, **({"n": args.n} if args.n else {}))


if __name__ == "__main__":
    main()
