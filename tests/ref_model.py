"""Vectorised numpy model of the scaling quantiser, written independently of the
C oracle (different language, different formulation, numpy's own float16 and
torch's own bfloat16 conversions).  It plays the part of the pure-numpy oracle
inside the reference's functional test
(cuda_kernels/tests/test_scaling_quantization_functional.py:25-259), but it
evaluates the bf16 path in float32 and the fp16 path in float16 op by op -- the
arithmetic the kernels use -- so AEE results can be compared bit for bit and MEE
results up to the implementation of log2.

All functions return (codes[n] int, decoded[n] float32).
"""
import numpy as np
import torch

f32 = np.float32
f16 = np.float16

EPS = {2: 0.23, 3: 0.18, 4: 0.18, 5: 0.18, 6: 0.1, 7: 0.1, 8: 0.1}


def bf16_round(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    return torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()


def mee_table(nbits):
    """table[2^nbits] and (c, cmm, l2b) as float16, built from the closed form
    ((1+2e^2)^j - 1) / (2e^2) * (1+e^2) in float32 with repeated multiplication."""
    eps = f32(EPS[nbits])
    two_e2 = f32(2.0) * eps * eps
    base = f32(1.0) + two_e2
    one_e2 = f32(1.0) + eps * eps
    anchor = (1 << (nbits - 1)) - 1
    table = np.zeros(1 << nbits, f16)
    pw = f32(1.0)
    for j in range(1, anchor + 1):
        pw = f32(pw * base)
        rep = f32(f32(f32(pw - f32(1.0)) / two_e2) * one_e2)
        table[anchor + j] = f16(rep)
        table[anchor - j] = f16(-rep)
    c = f16(one_e2 / two_e2)
    l2b = f16(np.log2(base, dtype=np.float32))
    return table, c, table[2 * anchor], l2b


def _sat16(x):
    x = np.nan_to_num(np.asarray(x, np.float64), nan=0.0, posinf=32767.0, neginf=-32768.0)
    return np.clip(np.trunc(x), -32768, 32767).astype(np.int64)


def _wrap16(x):
    return ((x + 32768) % 65536) - 32768


def model_bf16(src, rand, nbits, C, strategy, guarded=None):
    """src, rand: float32 arrays holding the (already widened) element values."""
    src = np.asarray(src, f32)
    rand = np.asarray(rand, f32)
    n = src.size
    R = (1 << (nbits - 1)) - 1
    hier = strategy >= 2
    mee = strategy in (1, 3)
    v = src.reshape(-1, C)
    table, c, cmm, l2b = mee_table(nbits) if mee else (None, None, None, None)
    with np.errstate(all="ignore"):
        absmax = np.abs(v).max(axis=1).astype(f32)
        div = f32(cmm) if mee else f32(R)
        s = (absmax / div + f32(1e-7)).astype(f32)
        if hier:
            s = np.maximum(s, f32(1e-30))
            g = s.reshape(-1, 16).max(axis=1)
            unit = np.maximum(bf16_round(np.maximum((g / f32(255.0)).astype(f32), f32(1e-30))), f32(1e-30))
            ratio = (s.reshape(-1, 16) / g[:, None] * f32(255.0)).astype(f32)
            q = np.clip(np.ceil(ratio), 1, 255).astype(f32)
            d = np.maximum((q * unit[:, None]).astype(f32), f32(1e-30)).reshape(-1)
        else:
            d = bf16_round(s)
        x = (v / d[:, None]).astype(f32)
        if mee:
            a = np.abs(x)
            lat = (np.log2((a / f32(c) + f32(1.0)).astype(f32), dtype=np.float32) / f32(l2b)).astype(f32)
            x = np.where(a > 0, np.sign(x) * lat, f32(0.0)).astype(f32)
        fl = np.floor(x)
        frac = (x - fl).astype(f32)
        inc = np.ceil((frac - rand.reshape(-1, C)).astype(f32))
        sv = _wrap16(_sat16(fl) + _sat16(inc))
        codes = np.clip(sv, -R, R) + R
        lev = table[codes].astype(f32) if mee else (codes - R).astype(f32)
        dec = (lev * d[:, None]).astype(f32)
    return codes.reshape(-1), dec.reshape(-1)


def model_f16(src, rand, nbits, C, strategy):
    """src, rand: float16 arrays; every operation rounds to float16."""
    v = np.asarray(src, f16).reshape(-1, C)
    r = np.asarray(rand, f16).reshape(-1, C)
    R = (1 << (nbits - 1)) - 1
    hier = strategy >= 2
    mee = strategy in (1, 3)
    table, c, cmm, l2b = mee_table(nbits) if mee else (None, None, None, None)
    with np.errstate(all="ignore"):
        absmax = np.abs(v).max(axis=1)
        div = cmm if mee else f16(R)
        s = (absmax / div).astype(f16) + f16(1e-7)
        s = s.astype(f16)
        if hier:
            g = s.reshape(-1, 16).max(axis=1)
            unit = (g / f16(255.0)).astype(f16)
            ratio = ((s.reshape(-1, 16) / g[:, None]).astype(f16) * f16(255.0)).astype(f16)
            q = np.minimum(np.ceil(ratio.astype(f32)), 255).astype(f16)
            d = (q * unit[:, None]).astype(f16).reshape(-1)
        else:
            d = s
        x = (v / d[:, None]).astype(f16)
        if mee:
            a = np.abs(x)
            arg = ((a / c).astype(f16) + f16(1.0)).astype(f16)
            lat = (np.log2(arg.astype(f32)).astype(f16) / l2b).astype(f16)
            x = np.where(a > 0, np.sign(x) * lat, f16(0.0)).astype(f16)
        fl = np.floor(x)
        frac = (x - fl).astype(f16)
        inc = np.ceil((frac - r).astype(f16).astype(f32))
        sv = _wrap16(_sat16(fl.astype(f32)) + _sat16(inc))
        codes = np.clip(sv, -R, R) + R
        lev = table[codes] if mee else (codes - R).astype(f16)
        dec = (lev * d[:, None]).astype(f16)
    return codes.reshape(-1), dec.reshape(-1).astype(f32)
