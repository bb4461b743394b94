"""The reference's CPU-runnable torch paths, restated as torch op sequences on CPU tensors, for the ``cpu_baseline``
figures of ``bench.py`` and ``evaluate.py``.  Measurement tooling, not part of the library: nothing in the package
imports this file, and it runs on the host cores only (torch's intra-op thread pool).

  * ``hier_roundtrip``  the hierarchical chunk-16 scaling quantiser (the arithmetic of
    csrc/cuda_hierarchical_mee.cu:203-343 / 345-505) written as the kind of torch op chain the reference uses for its
    own torch implementation of chunk scaling (csrc/logic.py:225-296): abs, row max, div, ceil, floor, stochastic carry
    from the random tensor, nibble pack; unpack, mul.
  * ``flat_roundtrip``  the flat variant exactly as csrc/logic.py:225-296 shapes it (one scale per chunk).
  * ``rht_roundtrip``   EDEN's compress / decompress of one power-of-two slice, cuda_kernels/src/srrcomp/srrcomp.py:293-353:
    randDiag (:61-106) * x -> Hadamard (:108-122) / sqrt(n) -> bucketize + scale (:356-361) -> EdenBinsToBits (:124-145)
    -> EdenBitsToBins (:147-167) -> take centroids -> Hadamard / sqrt(n) -> * randDiag -> * scale.
"""
import math
import time

import torch

_M32 = (1 << 32) - 1


# ---- chunk scaling quantiser ----------------------------------------------------------------------------------

def flat_roundtrip(x, rand, nbits, chunk=16):
    """csrc/logic.py:225-296: one float scale per chunk; returns the dequantised vector"""
    rng = (1 << (nbits - 1)) - 1
    v = x.view(-1, chunk).clone()
    scale = v.abs().max(dim=1, keepdim=True)[0].div_(rng).add_(1e-7)
    v.div_(scale)
    fl = torch.floor(v)
    codes = fl.add_(rand.view(-1, chunk) < v.sub_(fl)).clamp_(-rng, rng).add_(rng).to(torch.uint8)
    if nbits == 4:
        packed = codes[:, 0::2] | (codes[:, 1::2] << 4)
        codes = torch.stack((packed & 15, packed >> 4), dim=2).reshape(-1, chunk)
    return codes.float().sub_(rng).mul_(scale).reshape(-1)


def hier_roundtrip(x, rand, nbits, chunk=16, group=16):
    """the hierarchical (strategy 2) quantiser: per chunk s = absmax / R + 1e-7; per group of 16 chunks g = max s,
    unit = bf16(g / 255), q = clamp(ceil(s / g * 255), 1, 255); step = q * unit; code = clamp(floor(v / step) +
    carry, +-R) + R with carry = ceil(frac - rand); 4-bit codes packed two per byte; then the way back"""
    rng = (1 << (nbits - 1)) - 1
    v = x.view(-1, chunk).clone()
    s = v.abs().max(dim=1, keepdim=True)[0].div_(rng).add_(1e-7)                 # [chunks, 1]
    gmax = s.view(-1, group).max(dim=1, keepdim=True)[0]                          # [groups, 1]
    unit = gmax.div(255.0).clamp_(min=1e-30).to(torch.bfloat16).float()
    q = s.view(-1, group).div(gmax).mul_(255.0).ceil_().clamp_(1.0, 255.0)
    q8 = q.to(torch.uint8)                                                        # the stored scale byte
    step = q8.float().mul_(unit).clamp_(min=1e-30).view(-1, 1)
    v.div_(step)
    fl = torch.floor(v)
    carry = v.sub_(fl).sub_(rand.view(-1, chunk)).ceil_()
    codes = fl.add_(carry).clamp_(-rng, rng).add_(rng).to(torch.uint8)
    if nbits == 4:
        packed = codes[:, 0::2] | (codes[:, 1::2] << 4)
        codes = torch.stack((packed & 15, packed >> 4), dim=2).reshape(-1, chunk)
    return codes.float().sub_(rng).mul_(step).reshape(-1)


# ---- EDEN: randomized Hadamard transform, Lloyd-Max bins, bit planes ---------------------------------------------

def rand_diag(size, seed):
    """srrcomp.py:61-106 (the hash-based diagonal): +-1 float vector"""
    per_word, shift = 8, 4
    words = (size + per_word - 1) // per_word
    seed = (seed * 1664525 + 1013904223) & _M32
    seed = (seed * 8121 + 28411) & _M32
    r = torch.arange(words, dtype=torch.int64) + seed
    r = (1103515245 * r + 12345 + seed) & _M32
    r = (1140671485 * r + 12820163 + seed) & _M32
    r = r + 0x9e3779b9
    r = ((r ^ (r >> 16)) * 0x85ebca6b) & _M32
    r = ((r ^ (r >> 13)) * 0xc2b2ae35) & _M32
    r = (r ^ (r >> 16)) & _M32
    res = torch.zeros(words * per_word)
    at = 0
    for _ in range(per_word):
        res[at:at + words] = r & 15
        at += words
        r = r >> shift
    return (2 * (res >= 8) - 1)[:size]


def hadamard(vec):
    """srrcomp.py:108-122: in-place butterflies on views, strides ascending; the second half is formed as (a + b) - 2 b"""
    d = vec.numel()
    h = 2
    while h <= d:
        half = h // 2
        m = vec.view(d // h, h)
        m[:, :half] = m[:, :half] + m[:, half:]
        m[:, half:] = m[:, :half] - 2 * m[:, half:]
        h *= 2
    return vec.view(-1)


def bins_to_bits(bins, nbits):
    """srrcomp.py:124-145: one int32 word per 32 bins and bit plane, built by 32 multiply-adds per plane"""
    words = bins.numel() // 32
    bits = torch.zeros(words * nbits, dtype=torch.int32)
    for p in range(nbits):
        odd = (bins % 2 != 0).int().view(words, 32)
        word = torch.zeros(words, dtype=torch.int32)
        for i in range(32):
            word += odd[:, i] * (2 ** i)
        bits[words * p:words * (p + 1)] = word
        bins = torch.div(bins, 2, rounding_mode="floor")
    return bits


def bits_to_bins(bits, nbits):
    """srrcomp.py:147-167"""
    planes = bits.view(nbits, bits.numel() // nbits).to(torch.int64)
    words = planes.shape[1]
    bins = torch.zeros(words * 32)
    for p in range(nbits):
        v = torch.zeros((32, words))
        for i in range(32):
            v[i] = (torch.div(planes[p].clone(), 2 ** i, rounding_mode="floor").int() % 2 != 0).int()
        bins += 2 ** p * v.T.reshape(-1)
    return bins


def rht_roundtrip(x, nbits, seed, centroids, boundaries):
    """srrcomp.py:293-353 for one power-of-two slice with one rotation; returns the reconstruction"""
    n = x.numel()
    vec = x * rand_diag(n, seed)
    vec = hadamard(vec.to(torch.float32)) / math.sqrt(n)
    bins = torch.bucketize(vec * (n ** 0.5) / torch.norm(vec, 2), boundaries)
    scale = torch.norm(vec, 2) ** 2 / torch.dot(torch.take(centroids, bins), vec)
    packed = bins_to_bits(bins.to(torch.int32), nbits)
    back = bits_to_bins(packed.to(torch.int32), nbits)
    vec = torch.take(centroids, back.long())
    vec = hadamard(vec) / math.sqrt(n)
    vec = vec * rand_diag(n, seed)
    return scale * vec


# ---- timing ---------------------------------------------------------------------------------------------------

def median_seconds(fn, budget_s, max_reps=9):
    """one untimed call, then up to max_reps timed calls within the budget: (median seconds, calls timed)"""
    fn()
    ts = []
    while len(ts) < max_reps and (not ts or sum(ts) < budget_s):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], len(ts)
