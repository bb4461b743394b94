"""Host-side mirrors of the reference's Python callers: bit-width allocation (CPU),
compressor objects and the simulated ring (GPU)."""
import types

import numpy as np
import pytest
import torch

from helpers import BF16, bits_to_f32, to_bits

DEV = "cuda:0"


# ---- bit-width allocation (torch ops, runs anywhere) ------------------------------------------

def test_bitrate_search_hits_target():
    from dynamiq_sigcomm_artifact_amd import bitrate as B
    g = torch.Generator().manual_seed(0)
    norms = [torch.exp(torch.randn(5000, generator=g) * 5 - 6).to(torch.bfloat16) for _ in range(3)]
    assert B.dynamic_bitrate_target_bitrate("dynamiQ_mee_5bit_dynamic_bitrate") == 5.0
    assert B.dynamic_bitrate_target_bitrate("dynamiq_aee_dynamic_bitrate") == 5.0
    assert B.dynamic_bitrate_target_bitrate("x_3bit") == 3.0
    target = 5.0 - B.DYNAMIC_BITRATE_HEADROOM
    u, avg, delta = B.dynamic_bitrate_binary_search_u(norms, target)
    assert B.DYNAMIC_BITRATE_U_MIN <= u <= B.DYNAMIC_BITRATE_U_MAX
    assert abs(avg - target) <= B.DYNAMIC_BITRATE_TOL and abs(delta - (target - avg)) < 1e-12
    # extremes of u (comm_hooks.py:1087: the first compressed round starts at u = 60 -> all 8-bit)
    assert B.dynamic_bitrate_average_bits(norms, 60.0) == 8.0
    assert B.dynamic_bitrate_average_bits(norms, -10.0) == 2.0
    # the incremental rule keeps a converged u and walks back from a bad one
    u2, avg2, d2 = B.dynamic_bitrate_adjust_u(norms, u, target)
    assert u2 == u and abs(d2) <= B.DYNAMIC_BITRATE_TOL
    u3, avg3, d3 = B.dynamic_bitrate_adjust_u(norms, u + 6.0, target)
    assert abs(d3) < abs(B.dynamic_bitrate_avg_delta(norms, u + 6.0, target)[1])
    # qbits values and monotonicity in the norm
    q = B.dynamic_bitrate_qbits(torch.sort(norms[0].float())[0], u)
    assert set(q.unique().tolist()) <= {2, 4, 8} and bool((q[1:] >= q[:-1]).all())
    assert B.dynamic_bitrate_average_bits([], 0.0) == 0.0


# ---- compressor objects -------------------------------------------------------------------------

def _params(d, world, method="dynamiQ_aee_5bit"):
    return {"d": {(0, 0): d}, "world_size": world, "rank": 0,
            "args": types.SimpleNamespace(aggregation_method=method)}


@pytest.mark.gpu
def test_compressor_object_matches_reference_bookkeeping(eden_utils, oracle):
    from dynamiq_sigcomm_artifact_amd.compressors import Aee_Dynamic_Range_GPU_kern, Mee_Dynamic_Range_GPU_kern
    d, W = 256 * 40, 4
    for cls, strategy in ((Aee_Dynamic_Range_GPU_kern, 2), (Mee_Dynamic_Range_GPU_kern, 3)):
        c = cls(4, 16, _params(d, W))
        assert c.strategy == strategy and c.supergroup == 16 and c.range == 7
        # utils_aggregation.py:380-389: pool rows = 3 * ((d + C) // C) // W
        assert tuple(c.randomized_vec_pool.shape) == (3 * ((d + 16) // 16) // W, 16)
        assert c.randomized_vec_pool.dtype == torch.bfloat16
        assert c.compressed_numel(1000) == 4 * 146 and c.padded_n(1000) == 1024
        assert c.create_tensor(torch.zeros(1000), torch.uint8).numel() == 4 * 146
        # LCG of the row offsets (:391,395-397,409-420)
        seed = (4 * 998244353) & 0xFFFFFFFF
        n = 256 * 8
        x = (torch.randn(n, device=DEV) * 1e-3).to(torch.bfloat16)
        send = c.create_tensor(x, torch.uint8)
        rows = c.randomized_vec_pool.shape[0]
        for _ in range(3):
            seed = (seed * 671431 + 1000000007) & 0xFFFFFFFF
            randl = seed % (rows - n // 16 - 1)
            c.compression(x, send)
            rnd = c.randomized_vec_pool[randl:randl + n // 16, :].reshape(-1)
            want = oracle.scaling_compress(to_bits(x), to_bits(rnd), n, 4, 16, strategy, BF16)
            assert (send.cpu().numpy() == want).all()
        out = torch.zeros_like(x)
        c.decompression(send, out)
        dec = np.zeros(n, np.uint16)
        oracle.scaling_decompress(want, dec, n, 4, 16, strategy, BF16)
        assert (to_bits(out) == dec).all()
        c.decompression_add(send, out)
        oracle.scaling_decompress(want, dec, n, 4, 16, strategy, BF16, add=True)
        assert (to_bits(out) == dec).all()


@pytest.mark.gpu
def test_loaded_random_pool_keeps_the_dtype_the_reference_keeps(eden_utils, oracle):
    """the "correlated" mode loads its pool from a file: the AEE class keeps the file's dtype (utils_aggregation.py:389),
    the MEE class casts it to float16 (:488), so a bfloat16 call of the MEE class rounds every value twice"""
    from dynamiq_sigcomm_artifact_amd.compressors import Aee_Dynamic_Range_GPU_kern, Mee_Dynamic_Range_GPU_kern
    d, W, n = 256 * 40, 2, 256 * 6
    g = torch.Generator().manual_seed(8)
    loaded = torch.rand(3 * ((d + 16) // 16) // W * 16 + 100, generator=g)
    x = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
    twice = loaded.to(torch.float16).to(torch.bfloat16)
    once = loaded.to(torch.bfloat16)
    assert not torch.equal(twice, once)
    for cls, strategy, seen, kept in ((Aee_Dynamic_Range_GPU_kern, 2, once, torch.float32),
                                      (Mee_Dynamic_Range_GPU_kern, 3, twice, torch.float16)):
        c = cls(4, 16, dict(_params(d, W), rand_pool_tensor=loaded))
        assert c.randomized_vec_pool.dtype == kept
        rows = c.randomized_vec_pool.shape[0]
        assert rows == 3 * ((d + 16) // 16) // W
        send = c.create_tensor(x, torch.uint8)
        c.compression(x.to(DEV), send)
        seed = ((4 * 998244353) & 0xFFFFFFFF) * 671431 + 1000000007 & 0xFFFFFFFF
        randl = seed % (rows - n // 16 - 1)
        rnd = seen[randl * 16:randl * 16 + n]
        want = oracle.scaling_compress(to_bits(x), to_bits(rnd), n, 4, 16, strategy, BF16)
        assert (send.cpu().numpy() == want).all()


def _oracle_ring(oracle, vecs_bits, pools, nbits, strategy, W):
    """the same schedule on the CPU with oracle calls (ring_rdma.py:590-631)"""
    n = vecs_bits[0].size
    csize = ((n + W - 1) // W + 255) // 256 * 256
    bounds = [(csize * i, min(csize * (i + 1), n)) for i in range(W)]
    seeds = [(nbits * 998244353) & 0xFFFFFFFF for _ in range(W)]
    send = [None] * W
    recv = [None] * W

    def rand_for(r, cnt):
        seeds[r] = (seeds[r] * 671431 + 1000000007) & 0xFFFFFFFF
        rows = pools[r].size // 16
        randl = seeds[r] % (rows - cnt // 16 - 1)
        return np.ascontiguousarray(pools[r][randl * 16: randl * 16 + cnt])

    def chunk(r, i):
        lo, hi = bounds[i]
        return vecs_bits[r][lo:hi]

    def exch(src):
        return [src[(r - 1) % W] for r in range(W)]

    for step in range(W - 1):
        for r in range(W):
            if step == 0:
                c = np.ascontiguousarray(chunk(r, r))
                send[r] = oracle.scaling_compress(c, rand_for(r, c.size), c.size, nbits, 16, strategy, BF16)
            else:
                c = np.ascontiguousarray(chunk(r, (r - step) % W))
                send[r] = oracle.scaling_dec_comp(recv[r], c, rand_for(r, c.size), c.size, nbits, 16, strategy, BF16)
        recv = exch(send)
    for r in range(W):
        lo, hi = bounds[(r + 1) % W]
        c = np.ascontiguousarray(vecs_bits[r][lo:hi])
        send[r] = oracle.scaling_dec_comp(recv[r], c, rand_for(r, c.size), c.size, nbits, 16, strategy, BF16)
        oracle.scaling_decompress(send[r], c, c.size, nbits, 16, strategy, BF16)
        vecs_bits[r][lo:hi] = c
    bufs = [send, recv]
    for step in range(W - 1):
        bufs[(step ^ 1) & 1] = exch(bufs[step & 1])
        for r in range(W):
            lo, hi = bounds[(r - step) % W]
            c = np.zeros(hi - lo, np.uint16)
            oracle.scaling_decompress(bufs[(step ^ 1) & 1][r], c, c.size, nbits, 16, strategy, BF16)
            vecs_bits[r][lo:hi] = c
    return vecs_bits


@pytest.mark.gpu
@pytest.mark.parametrize("W,nbits,strategy", [(4, 4, 2), (8, 8, 2), (3, 4, 3), (8, 2, 2)])
def test_simulated_ring_matches_oracle_schedule(eden_utils, oracle, W, nbits, strategy):
    from dynamiq_sigcomm_artifact_amd import compressors as CP
    from dynamiq_sigcomm_artifact_amd.ring_sim import ring_allreduce
    n = 256 * 37   # ragged: the last ring chunk is shorter than the others
    g = torch.Generator().manual_seed(W * 10 + nbits)
    sig = torch.exp(torch.rand(W, generator=g) * 4.6 - 9.2)          # log-uniform in [1e-4, 1e-2]
    grads = [(torch.randn(n, generator=g) * sig[r]).to(torch.bfloat16) for r in range(W)]
    exact = torch.stack([x.double() for x in grads]).sum(0)
    cls = CP.Aee_Dynamic_Range_GPU_kern if strategy == 2 else CP.Mee_Dynamic_Range_GPU_kern
    gen = torch.Generator(device=DEV).manual_seed(99)
    comps = [cls(nbits, 16, dict(_params(n, W), rank=r), generator=gen) for r in range(W)]
    vecs = [x.to(DEV) for x in grads]
    ring_allreduce(vecs, comps)
    torch.cuda.synchronize()
    # every rank holds the same bytes
    for r in range(1, W):
        assert torch.equal(vecs[r], vecs[0])
    # and they are the bytes the oracle produces for the same schedule and random offsets
    pools = [to_bits(c.randomized_vec_pool.reshape(-1)) for c in comps]
    want = _oracle_ring(oracle, [to_bits(x) for x in grads], pools, nbits, strategy, W)
    assert (to_bits(vecs[0]) == want[0]).all()
    nmse = float(((vecs[0].double().cpu() - exact) ** 2).sum() / (exact ** 2).sum())
    assert nmse < {2: 4.0, 4: 0.12, 8: 6e-4}[nbits], nmse


def test_bench_refuses_more_than_one_gpu():
    """no multi-GPU figure is produced: bench.py --gpus 2 exits with a message before touching a device"""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "--gpus must be 1" in r.stderr and r.stdout.strip() == ""


def test_division_by_the_world_size_as_a_multiplication():
    """The mixed kernels split a group of n superchunks over the ring as ceil(n / world) per rank and compute the
    quotient as (x * ceil(2^40 / world)) >> 40 for x < 2^24 and world <= 2^16 (dq_scaling_mixed.hip: divide_by_world).
    Brute force over every world size and the operands where such a reciprocal goes wrong first: multiples of the
    divisor minus one, the largest operands, and a random sample."""
    import numpy as np
    rng = np.random.default_rng(5)
    top = (1 << 24) - 1
    for d in range(2, 65537):
        m = ((1 << 40) + d - 1) // d
        k = np.concatenate([np.arange(1, 6, dtype=np.uint64), np.uint64(top // d) - np.arange(0, 4, dtype=np.uint64)])
        x = np.concatenate([k * np.uint64(d) - np.uint64(1), k * np.uint64(d), np.array([top, top - 1, 0, 1], np.uint64),
                            rng.integers(0, top + 1, 24, dtype=np.uint64)])
        x = x[x <= top]
        assert ((x * np.uint64(m)) >> np.uint64(40) == x // np.uint64(d)).all(), d
