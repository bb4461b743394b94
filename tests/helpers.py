"""Shared helpers of the test-suite: torch <-> numpy bit views and the
deterministic inputs of the reference's functional test
(cuda_kernels/tests/test_scaling_quantization_functional.py:274-284)."""
import numpy as np
import torch

F16, BF16, F32 = 0, 1, 2
TORCH_DT = {F16: torch.float16, BF16: torch.bfloat16, F32: torch.float32}


def to_bits(t):
    """CPU numpy view of a tensor in the oracle's storage convention."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    if t.dtype == torch.float32:
        return t.numpy().copy()
    if t.dtype == torch.uint8:
        return t.numpy().copy()
    raise TypeError(t.dtype)


def from_bits(a, dt, device="cpu"):
    if dt == F32:
        return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(device)
    t = torch.from_numpy(np.ascontiguousarray(a, np.uint16).view(np.int16)).view(TORCH_DT[dt])
    return t.to(device)


def bits_to_f32(a, dt):
    if dt == F32:
        return np.asarray(a, np.float32)
    if dt == BF16:
        return (np.asarray(a, np.uint16).astype(np.uint32) << 16).view(np.float32)
    return np.asarray(a, np.uint16).view(np.float16).astype(np.float32)


def make_input(n, dtype, device="cpu"):
    idx = torch.arange(n, dtype=torch.float32, device=device)
    values = torch.sin(idx * 0.17) * 1.7 + torch.cos(idx * 0.071) * 0.3
    values += (idx.remainder(7) - 3.0) * 0.013
    return values.to(dtype)


def make_rand(n, seed, dtype, device="cpu"):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return torch.rand(n, generator=g, dtype=torch.float32).to(dtype).to(device)


def unpack_stream(enc, n, nbits, C, strategy):
    """Parse a packed stream by the documented layout
    (cuda_kernels/documentation/scaling_quantization_algorithm.md:183-196,347-388).
    Returns codes[n], and for hierarchical streams (q[nchunks] uint8, unit[nsc] uint16),
    for flat streams (scale[nchunks] uint16, None)."""
    enc = np.asarray(enc, np.uint8)
    PB = C * nbits // 8
    nch = n // C
    if strategy >= 2:
        CB = PB + 1
        REC = 16 * CB + 2
        nsc = nch // 16
        rec = enc[:nsc * REC].reshape(nsc, REC)
        chunks = rec[:, :16 * CB].reshape(nsc, 16, CB)
        code_bytes = np.ascontiguousarray(chunks[:, :, :PB]).reshape(-1)
        q = np.ascontiguousarray(chunks[:, :, PB]).reshape(-1)
        unit = np.ascontiguousarray(rec[:, 16 * CB:]).view(np.uint16).reshape(-1)
        aux = (q, unit)
    else:
        rec = enc[:nch * (PB + 2)].reshape(nch, PB + 2)
        code_bytes = np.ascontiguousarray(rec[:, :PB]).reshape(-1)
        aux = (np.ascontiguousarray(rec[:, PB:]).view(np.uint16).reshape(-1), None)
    bits = np.unpackbits(code_bytes, bitorder="little").reshape(-1, nbits)
    codes = (bits.astype(np.int64) << np.arange(nbits)).sum(axis=1)
    return codes, aux
