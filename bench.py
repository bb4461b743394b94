#!/usr/bin/env python3
"""Benchmark of the eden_utils compression hot path on one MI355X.

A step = scaling_compress followed by scaling_decompress of one 25 MB DDP
bucket (6,553,600 fp32 gradient elements, Student-t(3) * 1e-3 with 0.1 % of the
entries multiplied by 100), hierarchical AEE (strategy 2), chunk 16, 4-bit
codes, bf16 random pool -- the 25 MB bucket configuration the headline metric
is quoted on.  Inputs are resident in HBM before the timed region; the calls go
through the C ABI of libdynamiq_eden.so on torch's current stream.

Prints ONE JSON line (see the fields below).  `value` is fp32 gradient bytes
(4 * N) per second of compress+decompress with ONE bucket's buffers replayed
(69 MB: after the warm-up they sit partly in the 256 MB Infinity Cache);
`value_cold` is the same step walking a ring of distinct bucket sets whose
footprint exceeds 512 MB, so that every launch streams from and to HBM.
`roofline` prices the dominant kernel (compress) at its algorithmic bytes
(4 + 2 + (q + 0.5625) / 8 per element) against the 8 TB/s HBM peak, with the
kernel's average launch duration measured here with HIP events on the launch
stream (the timed launches are replayed from a HIP graph so that the host's
per-call cost is not part of the figure; `eager_ms_per_step` has it): `frac` for the replayed bucket, `frac_cold` for the ring of buckets.
`cpu_baseline` times the reference's CPU-runnable path for this workload -- the
hierarchical chunk quantiser as a torch op sequence (cpu_baselines.py) -- on all
host cores; `cpu_scalar_port` is the scalar C oracle on one core and
`cpu_rht_path` EDEN's torch round trip (srrcomp.py:293-353) on 2^20 elements.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
OVERHEAD_BITS = 0.5625  # hierarchical scale bytes per element, in bits

# HBM bytes per launch of the compress kernel from two `rocprofv3 --pmc` runs of this script
# (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for
# the --pmc-calibration copy kernel: FETCH_SIZE x 1.999, WRITE_SIZE x 1.000.
# key: (source dtype, nbits, strategy, elements)
MEASURED_TRAFFIC_BYTES = {
    ("fp32", 4, 2, 6553600): int((25600.0 / 12806.9 * 19253.6 + 1.0 * 3800.0) * 1024),
}


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


def event_ms(fn, iters):
    """average device time of one fn() in ms: `iters` calls recorded into one HIP graph on a side stream and replayed
    between two events on that stream, so that the host's per-call cost (a few microseconds through ctypes, about
    the duration of these kernels) cannot sit between the launches"""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(iters):
                fn()
        graph.replay()
        side.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record(side)
        graph.replay()
        end.record(side)
        end.synchronize()
    torch.cuda.current_stream().wait_stream(side)
    return start.elapsed_time(end) / iters


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--n", type=int, default=6553600, help="gradient elements in the bucket")
    ap.add_argument("--nbits", type=int, default=4)
    ap.add_argument("--strategy", type=int, default=2, help="2 = hierarchical AEE, 3 = hierarchical MEE")
    ap.add_argument("--src", choices=["fp32", "bf16"], default="fp32")
    ap.add_argument("--rand", choices=["pool", "philox"], default="pool",
                    help="pool: the reference's rand_pool tensor (default); philox: uniform values drawn in the kernel")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of each cpu_baseline leg (0 = skip)")
    ap.add_argument("--cold-sets", type=int, default=-1,
                    help="distinct bucket sets (source, random pool, packed, output) the cold leg walks; default: as many "
                         "as make up 640 MB, at least 10; 0 or 1 = skip the cold leg")
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

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    n = args.n // 256 * 256
    nbits, strategy, C = args.nbits, args.strategy, 16
    x32 = make_bucket(n, 0, dev)
    src = x32 if args.src == "fp32" else x32.to(torch.bfloat16)
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    rand = torch.rand(n, generator=g, device=dev).to(torch.bfloat16)
    packed = torch.zeros(capi.required_bytes(n, nbits, C, strategy), dtype=torch.uint8, device=dev)
    out = torch.empty_like(src)

    def compress():
        if args.rand == "philox":
            capi.scaling_compress_philox(src, packed, n, nbits, C, strategy, 2026, 0)
        else:
            capi.scaling_compress(src, packed, rand, n, nbits, C, strategy)

    def decompress():
        capi.scaling_decompress(packed, out, n, nbits, C, strategy)

    def step():
        compress()
        decompress()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # ---- timed region: exactly `steps` steps between two synchronisations ----
    ms_per_step = event_ms(step, args.steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eager_ms_per_step = eager_ms(step, args.steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    value = 4.0 * n / (ms_per_step * 1e-3) / 1e9

    # ---- per-kernel launch durations (same stream, HIP events) ----
    comp_ms = event_ms(compress, args.steps)
    dec_ms = event_ms(decompress, args.steps)
    sbytes = 4 if args.src == "fp32" else 2
    comp_bytes = (sbytes + (2 if args.rand == "pool" else 0) + (nbits + OVERHEAD_BITS) / 8.0) * n
    dec_bytes = (sbytes + (nbits + OVERHEAD_BITS) / 8.0) * n
    comp_gbs = comp_bytes / (comp_ms * 1e-3) / 1e9
    dec_gbs = dec_bytes / (dec_ms * 1e-3) / 1e9

    # ---- the same step over a ring of distinct buckets (> 512 MB): no launch finds its operands in a cache ----
    cold = None
    set_bytes = src.numel() * src.element_size() + rand.numel() * 2 + packed.numel() + out.numel() * out.element_size()
    if args.cold_sets < 0:
        args.cold_sets = max(10, -(-640000000 // set_bytes))
    if args.cold_sets > 1:
        sets = [(src, rand, packed, out)]
        for k in range(1, args.cold_sets):
            xk = make_bucket(n, k, dev)
            gk = torch.Generator(device=dev)
            gk.manual_seed(1000 + k)
            sets.append((xk if args.src == "fp32" else xk.to(torch.bfloat16),
                         torch.rand(n, generator=gk, device=dev).to(torch.bfloat16), torch.zeros_like(packed),
                         torch.empty_like(out)))
        pos = [0]

        def nxt():
            pos[0] = (pos[0] + 1) % len(sets)
            return sets[pos[0]]

        def compress_cold():
            s_, r_, p_, _ = nxt()
            if args.rand == "philox":
                capi.scaling_compress_philox(s_, p_, n, nbits, C, strategy, 2026, 0)
            else:
                capi.scaling_compress(s_, p_, r_, n, nbits, C, strategy)

        def decompress_cold():
            _, _, p_, o_ = nxt()
            capi.scaling_decompress(p_, o_, n, nbits, C, strategy)

        def step_cold():
            s_, r_, p_, o_ = nxt()
            if args.rand == "philox":
                capi.scaling_compress_philox(s_, p_, n, nbits, C, strategy, 2026, 0)
            else:
                capi.scaling_compress(s_, p_, r_, n, nbits, C, strategy)
            capi.scaling_decompress(p_, o_, n, nbits, C, strategy)

        for _ in range(len(sets)):
            step_cold()
        torch.cuda.synchronize()
        step_cold_ms = event_ms(step_cold, args.steps)
        comp_cold_ms = event_ms(compress_cold, args.steps)
        dec_cold_ms = event_ms(decompress_cold, args.steps)
        cold = {
            "sets": len(sets),
            "footprint_MB": round(set_bytes * len(sets) / 1e6, 1),
            "ms_per_step": round(step_cold_ms, 5),
            "value": round(4.0 * n / (step_cold_ms * 1e-3) / 1e9, 2),
            "compress_ms": round(comp_cold_ms, 5),
            "decompress_ms": round(dec_cold_ms, 5),
            "compress_GBps": round(comp_bytes / (comp_cold_ms * 1e-3) / 1e9, 1),
            "decompress_GBps": round(dec_bytes / (dec_cold_ms * 1e-3) / 1e9, 1),
        }
        del sets[1:]

    if args.pmc_calibration:
        cal_src = torch.empty(n, dtype=torch.float32, device=dev).normal_()
        cal_dst = torch.empty_like(cal_src)
        for _ in range(5):
            torch.neg(cal_src, out=cal_dst)
        torch.cuda.synchronize()

    # ---- quality: NMSE of the round trip ----
    xf = x32.double()
    nmse = float(((out.double() - xf) ** 2).sum() / (xf ** 2).sum())

    # ---- parity of a sample against the oracle (the checker, not the product) ----
    bit_exact = None
    cpu_scalar = None
    if not args.no_check or args.cpu_seconds > 0:
        import oracle as O
        odt = O.F32 if args.src == "fp32" else O.BF16
        m = min(n, 1 << 20)

        def host_bits(t):
            t = t[:m].cpu().contiguous()
            if t.dtype == torch.float32:
                return t.numpy().copy()
            return t.view(torch.int16).numpy().view(np.uint16).copy()

        src_h = host_bits(src)
        if args.rand == "philox":
            uni = O.philox_uniform(m, 2026, 0)
            rand_h = uni if args.src == "fp32" else (uni.view(np.uint32) >> 16).astype(np.uint16)   # k/256 is exact in bf16
        else:
            rand_h = host_bits(rand.float() if args.src == "fp32" else rand)
        if not args.no_check:
            enc_o = O.scaling_compress(src_h, rand_h, m, nbits, C, strategy, odt)
            dec_o = np.zeros(m, src_h.dtype)
            O.scaling_decompress(enc_o, dec_o, m, nbits, C, strategy, odt)
            nb = O.required_bytes(m, nbits, C, strategy)
            bit_exact = bool((packed[:nb].cpu().numpy() == enc_o).all() and (host_bits(out) == dec_o).all())
        if args.cpu_seconds > 0:
            reps, spent = 0, 0.0
            dec_o = np.zeros(m, src_h.dtype)
            while spent < args.cpu_seconds / 2 and reps < 64:
                t1 = time.perf_counter()
                enc_o = O.scaling_compress(src_h, rand_h, m, nbits, C, strategy, odt)
                O.scaling_decompress(enc_o, dec_o, m, nbits, C, strategy, odt)
                spent += time.perf_counter() - t1
                reps += 1
            cpu_scalar = {
                "value": round(4.0 * m * reps / spent / 1e9, 4),
                "unit": "GB/s",
                "cores": 1,
                "kind": "port",
                "sample": "first %d elements of the same bucket, %d compress+decompress round trips of the scalar C oracle"
                          % (m, reps),
            }

    # ---- the reference's CPU-runnable path for this workload on all host cores: the hierarchical chunk quantiser as a
    #      torch op sequence of the shape of the reference's own torch implementation (csrc/logic.py:225-296) ----
    cpu = None
    cpu_rht = None
    if args.cpu_seconds > 0:
        import cpu_baselines as CB
        xc, rc = x32.cpu(), torch.rand(n)
        if strategy == 2:
            sec, reps = CB.median_seconds(lambda: CB.hier_roundtrip(xc, rc, nbits), args.cpu_seconds)
            cpu = {
                "value": round(4.0 * n / sec / 1e9, 3),
                "unit": "GB/s",
                "cores": torch.get_num_threads(),
                "kind": "port",
                "sample": "the whole bucket (%d fp32 elements), median of %d compress+decompress round trips of the "
                          "hierarchical chunk-16 quantiser as torch CPU ops (output equal to the oracle's, tests/test_cpu_baselines.py)"
                          % (n, reps),
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
        sec, reps = CB.median_seconds(lambda: CB.rht_roundtrip(x1.clone(), 4, 0, cen, bnd), args.cpu_seconds / 2, max_reps=5)
        cpu_rht = {
            "value": round(4.0 * d1 / sec / 1e9, 4),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": "2^20 fp32 N(0, 1e-3^2), median of %d EDEN compress+decompress round trips at 4 bits as torch CPU ops "
                      "(randDiag, Hadamard / sqrt(n), bucketize, EdenBinsToBits and back)" % reps,
        }

    result = {
        "metric": "compress+decompress GB/s (fp32 grad in) on 1 MI355X, % of HBM peak; NMSE",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "one 25 MB DDP bucket: %d %s gradient elements, Student-t(3)*1e-3 with 0.1%% outliers x100; "
                        "%d-bit hierarchical %s compress + decompress, chunk 16, %s"
                        % (n, args.src, nbits, "AEE" if strategy == 2 else "MEE",
                           "bf16 rand_pool" if args.rand == "pool" else "in-kernel Philox rounding"),
            "elements": n,
            "nbits": nbits,
            "strategy": strategy,
            "chunk_size": C,
            "source_dtype": args.src,
            "packed_bytes": int(packed.numel()),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "hier16_compress_kernel",
            "achieved": round(comp_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(comp_gbs / HBM_PEAK_GBS, 4),
            "frac_is": "one bucket's buffers replayed (69 MB working set: cache-assisted, part of the traffic is served by "
                       "the 256 MB Infinity Cache); frac_cold is the HBM-only figure",
            "frac_cold": round(cold["compress_GBps"] / HBM_PEAK_GBS, 4) if cold else None,
            "achieved_cold": cold["compress_GBps"] if cold else None,
            "traffic": MEASURED_TRAFFIC_BYTES.get((args.src, nbits, strategy, n)) if args.rand == "pool" else None,
            "algorithmic_bytes_per_launch": int(comp_bytes),
            "avg_launch_ms": round(comp_ms, 5),
            "avg_launch_ms_cold": cold["compress_ms"] if cold else None,
        },
        "kernels": {
            "compress": {"ms": round(comp_ms, 5), "algorithmic_GBps": round(comp_gbs, 1), "frac_hbm": round(comp_gbs / HBM_PEAK_GBS, 4)},
            "decompress": {"ms": round(dec_ms, 5), "algorithmic_GBps": round(dec_gbs, 1), "frac_hbm": round(dec_gbs / HBM_PEAK_GBS, 4)},
        },
        "frac_hbm_roundtrip": round((comp_bytes + dec_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "nmse": nmse,
        "bit_exact_vs_oracle": bit_exact,
        "eager_ms_per_step": round(eager_ms_per_step, 5),
        "host_wall_ms_per_step": round(wall_ms, 5),
        "value_cold": cold["value"] if cold else None,
        "cold": cold,
        "cpu_baseline": cpu,
        "cpu_scalar_port": cpu_scalar,
        "cpu_rht_path": cpu_rht,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
