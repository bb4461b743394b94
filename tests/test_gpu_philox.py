"""The in-kernel random stream: Philox4x32-10 keyed by the seed, counter = (chunk index, step), one block = the 16
uniform values of one chunk.  The kernels must (a) write exactly the oracle's stream, (b) give, with the stream drawn
inside, the bytes the rand_pool entry points give when fed that stream as a tensor, for every kernel family."""
import numpy as np
import pytest
import torch

from helpers import BF16, F16, F32, TORCH_DT, to_bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dt", [F16, BF16, F32])
def test_uniform_tensor_matches_oracle(capi, oracle, dt):
    for n, seed, step in ((16, 0, 0), (1000, 7, 3), (256 * 300 + 5, 0xDEADBEEFCAFEF00D, 1 << 40)):
        out = torch.full((n + 4,), 9.0, dtype=TORCH_DT[dt], device=DEV)
        capi.philox_uniform(out[:n], seed, step)
        want = oracle.philox_uniform(n, seed, step)
        assert (out[:n].float().cpu().numpy() == want).all()          # every value k/256 is exact in all three types
        assert bool((out[n:] == 9.0).all())
    u = oracle.philox_uniform(1 << 18, 1, 2)
    assert u.min() == 1 / 256 and u.max() == 255 / 256 and abs(u.mean() - 0.5) < 2e-3
    assert ((u * 256).astype(np.int64) % 2 == 1).all()
    assert not (oracle.philox_uniform(4096, 1, 2) == oracle.philox_uniform(4096, 1, 3)).all()
    assert not (oracle.philox_uniform(4096, 1, 2) == oracle.philox_uniform(4096, 2, 2)).all()


@pytest.mark.parametrize("dt,strategies", [(BF16, (0, 1, 2, 3)), (F32, (0, 2, 3)), (F16, (1, 2, 3))])
@pytest.mark.parametrize("nbits", [2, 4, 5, 8])
def test_philox_mode_equals_pool_mode(capi, oracle, dt, strategies, nbits):
    tdt = TORCH_DT[dt]
    seed, step = 0x1234567890ABCDEF, 41
    for strategy in strategies:
        n = 256 * 37 if strategy >= 2 else 16 * 333
        g = torch.Generator().manual_seed(nbits + strategy)
        src = (torch.randn(n, generator=g) * 1e-2).to(tdt).to(DEV)
        inp = (torch.randn(n, generator=g) * 1e-2).to(tdt).to(DEV)
        uni = torch.empty(n, dtype=tdt, device=DEV)
        capi.philox_uniform(uni, seed, step)
        nbytes = capi.required_bytes(n, nbits, 16, strategy)
        a = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        b = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
        capi.scaling_compress(src, a, uni, n, nbits, 16, strategy)
        capi.scaling_compress_philox(src, b, n, nbits, 16, strategy, seed, step)
        assert torch.equal(a, b), (dt, strategy)
        want = oracle.scaling_compress(to_bits(src), to_bits(uni), n, nbits, 16, strategy, dt)
        assert (b.cpu().numpy() == want).all()
        # ring step
        capi.philox_uniform(uni, seed, step + 1)
        sa, sb = torch.zeros_like(a), torch.zeros_like(a)
        ia, ib = inp.clone(), inp.clone()
        capi.scaling_dec_comp(a, ia, sa, uni, n, nbits, 16, strategy)
        capi.scaling_dec_comp_philox(a, ib, sb, n, nbits, 16, strategy, seed, step + 1)
        assert torch.equal(sa, sb) and torch.equal(to_bits_t(ia), to_bits_t(ib))
        # another step is another stream
        capi.scaling_compress_philox(src, sb, n, nbits, 16, strategy, seed, step + 2)
        assert not torch.equal(sb, b)


def to_bits_t(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def test_philox_binding_and_quality(eden_utils):
    n = 256 * 4096
    g = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn(n, generator=g, device=DEV) * 1e-3).to(torch.bfloat16)
    enc = torch.zeros(n // 256 * 146, dtype=torch.uint8, device=DEV)
    acc = torch.zeros(n, device=DEV)
    reps = 64
    for step in range(reps):
        eden_utils.scaling_compress_philox(x, enc, n, 4, 16, 99, step, 0, 2)
        out = torch.empty_like(x)
        eden_utils.scaling_decompress(enc, out, n, 4, 16, 0, 2)
        acc += out.float()
    # unbiased: the mean over independent steps approaches x (error falls as 1/sqrt(reps))
    one = float(((out.float() - x.float()) ** 2).sum() / (x.float() ** 2).sum())
    avg = float(((acc / reps - x.float()) ** 2).sum() / (x.float() ** 2).sum())
    assert 1.2e-2 < one < 1.8e-2 and avg < 1.5 * one / reps + 2e-5
    u = torch.empty(4096, dtype=torch.float32, device=DEV)
    eden_utils.philox_uniform(u, 5, 6)
    assert float(u.min()) > 0 and float(u.max()) < 1
    with pytest.raises(RuntimeError, match="chunk_size 16"):
        eden_utils.scaling_compress_philox(x, enc, n, 4, 32, 1, 1, 0, 2)


def test_ring_with_in_kernel_randomness(eden_utils):
    """the simulated ring with compressor objects that draw their randomness in the kernels: ranks agree, error as with pools"""
    import types
    from dynamiq_sigcomm_artifact_amd.compressors import Aee_Dynamic_Range_GPU_kern
    from dynamiq_sigcomm_artifact_amd.ring_sim import ring_allreduce
    W, n = 4, 256 * 1001
    g = torch.Generator(device=DEV).manual_seed(3)
    vecs = [(torch.randn(n, generator=g, device=DEV) * 1e-3).to(torch.bfloat16) for _ in range(W)]
    exact = torch.stack([v.double() for v in vecs]).sum(0)

    def run(extra):
        comps = []
        for r in range(W):
            params = dict({"d": {(0, 0): n}, "world_size": W, "rank": r,
                           "args": types.SimpleNamespace(aggregation_method="dynamiQ")}, **extra)
            comps.append(Aee_Dynamic_Range_GPU_kern(8, 16, params, generator=torch.Generator(device=DEV).manual_seed(r)))
        out = ring_allreduce([v.clone() for v in vecs], comps)
        assert all(torch.equal(out[0], o) for o in out[1:])
        return float(((out[0].double() - exact) ** 2).sum() / (exact ** 2).sum()), comps
    pool_nmse, _ = run({})
    phil_nmse, comps = run({"philox_seed": 11})
    assert comps[0].randomized_vec_pool is None
    assert abs(phil_nmse - pool_nmse) < 0.1 * pool_nmse
