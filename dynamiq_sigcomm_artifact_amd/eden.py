"""EDEN on the library's kernels -- the host-side mirror of ``srrcomp.Eden`` and of the ``SRRCompUtils`` it inherits
(cuda_kernels/src/srrcomp/srrcomp.py:13-447): the same slicing rule, the same
``compress`` / ``decompress`` signatures and the same per-slice dictionaries, with

  * randDiag + Hadamard + 1/sqrt(n) in one launch per rotation (``rht_blocked``),
  * ``_quantize`` + ``EdenBinsToBits`` in one call (``eden_quantize``: norm, bucketize,
    bit planes, dot product and scale on the device, no host synchronisation),
  * ``EdenBitsToBins`` + the centroid lookup in one call (``eden_dequantize``).

Tables.  The reference carries its Lloyd-Max tables as literals.  Here the centroids
are computed: the stationary point of the Lloyd-Max conditions for N(0, 1) with
2^nbits levels (scipy's normal pdf / cdf, a Newton-type root solve).  The reference's
literals deviate from that optimum by up to 1.7e-3 (8 bits); pass the reference's own
tensors as ``centroids=`` / ``boundaries=`` to reproduce its bins exactly.
"""
import math

import numpy as np
import torch

from . import capi

_TABLES = {}


def _conditional_means(c):
    from scipy.stats import norm
    b = np.concatenate(([-np.inf], (c[:-1] + c[1:]) / 2, [np.inf]))
    num = norm.pdf(b[:-1]) - norm.pdf(b[1:])
    den = np.where(b[:-1] > 0, norm.sf(b[:-1]) - norm.sf(b[1:]), norm.cdf(b[1:]) - norm.cdf(b[:-1]))
    return num / den


def lloyd_max_normal(nbits):
    """float64 centroids (2^nbits, ascending, symmetric) of the Lloyd-Max quantiser of N(0, 1)"""
    if nbits not in _TABLES:
        from scipy.optimize import root
        from scipy.stats import norm
        levels = 1 << nbits
        c = norm.ppf((np.arange(levels) + 0.5) / levels)
        for _ in range(500):
            c = _conditional_means(c)
        c = root(lambda x: x - _conditional_means(x), c, method="hybr", tol=1e-15).x
        _TABLES[nbits] = (c - c[::-1]) / 2
    return _TABLES[nbits]


def normal_centroids_and_boundaries(nbits):
    """float32 tensors shaped like srrcomp.py:364-447: centroids [2^nbits], boundaries = float32 midpoints"""
    c = torch.from_numpy(lloyd_max_normal(nbits).astype(np.float32))
    return c, (c[:-1] + c[1:]) / 2


class SRRCompUtils(object):
    """The helpers ``srrcomp.Eden`` inherits (srrcomp.py:13-167) on the library's kernels: ``randDiag``, ``Hadamard``,
    ``EdenBinsToBits`` / ``EdenBitsToBins`` and the ``utils`` table the reference looks its implementations up in.
    Only device tensors are served (the build has no CPU path): the 'cpu' entries of ``utils`` raise."""

    def __init__(self, gpuacctype="cuda"):
        if gpuacctype not in ("cuda", "torch"):
            raise Exception("Illegal gpuacctype {}, use 'cuda' or 'torch'.".format(gpuacctype))
        self.gpuacctype = gpuacctype                  # both values select the kernels here
        from . import load_eden_utils
        eu = load_eden_utils()
        gpu = {"Hadamard": eu.Hadamard, "BinsToBits": eu.EdenBinsToBits, "BitsToBins": eu.EdenBitsToBins}
        self.utils = {"gpu": gpu, "cpu": {name: self._device_only for name in gpu}}

    @staticmethod
    def _device_only(*args, **kwargs):
        raise RuntimeError("this build serves device tensors only: move the vector to the GPU")

    def randDiag(self, size, device, seed, torchRNG=False):
        """+-1 floats (srrcomp.py:61-106); with torchRNG torch's own Bernoulli stream, as there"""
        if torchRNG:
            prng = torch.Generator(device=device)
            prng.manual_seed(seed)
            half = torch.full((size,), 0.5, device=device)
            return 2 * torch.bernoulli(half, generator=prng) - 1
        out = torch.empty(size, dtype=torch.float32, device=device)
        if size:
            capi.rand_diag(out, seed)
        return out

    def Hadamard(self, vec):
        """unnormalised transform of a power-of-two vector, in place like srrcomp.py:108-122; returns the flat view"""
        d = vec.numel()
        if d & (d - 1) != 0:
            raise Exception("input numel must be a power of 2")
        flat = vec.view(-1)
        capi.hadamard(flat)
        return flat

    def EdenBinsToBits(self, bins, nbits):
        """bit plane p of 32 consecutive bins -> bits[p * n/32 + w] (srrcomp.py:124-145); int32 like eden_utils"""
        return self.utils["gpu"]["BinsToBits"](bins.to(torch.int32).contiguous(), nbits)

    def EdenBitsToBins(self, bits, nbits):
        """the inverse (srrcomp.py:147-167); int32 bins like eden_utils (the torch version there returns floats)"""
        return self.utils["gpu"]["BitsToBins"](bits.to(torch.int32).contiguous(), nbits)


class Eden(SRRCompUtils):
    def __init__(self, gpuacctype="cuda", max_padding_overhead=0.1, centroids=None, boundaries=None, device="cuda"):
        super().__init__(gpuacctype)
        self.max_padding_overhead = max_padding_overhead
        self.device = torch.device(device)
        self.centroids = dict(centroids) if centroids is not None else {}
        self.boundaries = dict(boundaries) if boundaries is not None else {}
        self._dev_tables = {}
        capi.lib()

    def _tables(self, nbits):
        if nbits not in self._dev_tables:
            if nbits not in self.centroids:
                self.centroids[nbits], self.boundaries[nbits] = normal_centroids_and_boundaries(nbits)
            self._dev_tables[nbits] = (self.centroids[nbits].to(self.device, torch.float32).contiguous(),
                                       self.boundaries[nbits].to(self.device, torch.float32).contiguous())
        return self._dev_tables[nbits]

    # ---- srrcomp.py:251-291 ----
    def compress(self, vec, nbits, seed):
        vec_type = vec.dtype
        vec = vec.to(self.device, torch.float32).clone()        # the kernels only take buffers of self.device

        def low_po2(n):
            return 2 ** int(np.log2(n)) if n else 0

        def high_po2(n):
            return 2 ** (int(np.ceil(np.log2(n)))) if n else 0

        res = []
        dim = remaining = vec.numel()
        curr_index = 0
        while (high_po2(remaining) - remaining) / dim > self.max_padding_overhead:
            low = low_po2(remaining)
            num_hadamard = 1 + (low < 2 ** 10)
            res.append(self._compress_slice(vec[curr_index: curr_index + low], vec_type, nbits, num_hadamard, seed))
            curr_index += low
            remaining -= low
        num_hadamard = 1 + (dim - curr_index < 2 ** 10)
        res.append(self._compress_slice(vec[curr_index:], vec_type, nbits, num_hadamard, seed))
        return res

    @staticmethod
    def _inv_sqrt(n):
        # the divisor of `Hadamard(vec) / np.sqrt(n)` as torch applies a host scalar on the device: a product
        # with the float32 reciprocal
        return float(np.float32(1.0) / np.float32(math.sqrt(n)))

    # the diagonal of randDiag (srrcomp.py:61-106): one bit per element where the size allows it (multiples of 256),
    # the float vector otherwise -- the transform takes either
    def _diag_buffer(self, n):
        if n % 256 == 0:
            return torch.empty(n // 32, dtype=torch.int32, device=self.device)
        return torch.empty(n, dtype=torch.float32, device=self.device)

    @staticmethod
    def _rand_diag(diag, n, seed):
        if diag.dtype == torch.int32:
            capi.rand_diag_bits(diag, n, seed)
        else:
            capi.rand_diag(diag, seed)

    # ---- srrcomp.py:293-326 ----
    def _compress_slice(self, vec, vec_type, nbits, num_hadamard, seed):
        orig_dim = n = vec.numel()
        if not n & (n - 1) == 0 or n < 32:
            padded_dim = max(int(2 ** (np.ceil(np.log2(n)))), 32)
            padded = torch.zeros(padded_dim, device=self.device)
            padded[:n] = vec
            n, vec = padded_dim, padded
        else:
            vec = vec.contiguous().clone()
        diag = self._diag_buffer(n)
        for i in range(num_hadamard):
            self._rand_diag(diag, n, seed + i)
            capi.rht_blocked(vec, diag, n, self._inv_sqrt(n), False)
        centroids, boundaries = self._tables(nbits)
        packed = torch.empty(n // 32 * nbits, dtype=torch.int32, device=self.device)
        result = torch.empty(4, dtype=torch.float32, device=self.device)
        work = torch.empty(capi.eden_work_doubles(n), dtype=torch.float64, device=self.device)
        capi.eden_quantize(vec, boundaries, centroids, nbits, packed, result, work)
        return {"packed_bins": packed, "vec_type": vec_type, "nbits": nbits, "scale": result[2], "orig_dim": orig_dim,
                "num_hadamard": num_hadamard, "seed": seed}

    # ---- srrcomp.py:356-361 ----
    def _quantize(self, vec, nbits):
        """(bins, scale) of a rotated vector: bins int64 like torch.bucketize's, scale a 0-d tensor.  One call of the
        quantiser kernels (the bit planes it also writes are unpacked again here); ``compress`` does not go this way."""
        n = vec.numel()
        if n == 0 or n % 32:
            raise RuntimeError("_quantize: the kernels take a positive multiple of 32 elements")
        vec = vec.to(self.device, torch.float32).contiguous()
        centroids, boundaries = self._tables(nbits)
        packed = torch.empty(n // 32 * nbits, dtype=torch.int32, device=self.device)
        result = torch.empty(4, dtype=torch.float32, device=self.device)
        work = torch.empty(capi.eden_work_doubles(n), dtype=torch.float64, device=self.device)
        capi.eden_quantize(vec, boundaries, centroids, nbits, packed, result, work)
        return self.EdenBitsToBins(packed, nbits).to(torch.int64), result[2]

    # ---- srrcomp.py:328-354 ----
    def decompress(self, data):
        return torch.cat([self._decompress_slice(d["packed_bins"], d["vec_type"], d["nbits"], d["scale"], d["orig_dim"],
                                                 d["num_hadamard"], d["seed"]) for d in data])

    def _decompress_slice(self, packed_bins, vec_type, nbits, scale, orig_dim, num_hadamard, seed):
        n = packed_bins.numel() // nbits * 32
        centroids, _ = self._tables(nbits)
        vec = torch.empty(n, dtype=torch.float32, device=self.device)
        if num_hadamard == 0:
            capi.eden_dequantize(packed_bins.to(self.device, torch.int32), n, centroids, nbits, vec)
            return (scale * vec)[:orig_dim].to(vec_type)
        # the dequantiser rides on the first pass of the first rotation, the product with the scale on the last pass of
        # the last one: same bits as eden_dequantize, the rotations and `scale * vec`
        scale32 = scale.reshape(1).to(device=self.device, dtype=torch.float32) if isinstance(scale, torch.Tensor) else \
            torch.tensor([scale], dtype=torch.float32, device=self.device)
        diag = self._diag_buffer(n)
        for i in range(num_hadamard):
            self._rand_diag(diag, n, seed + num_hadamard - 1 - i)
            last = scale32 if i == num_hadamard - 1 else None
            if i == 0:
                capi.eden_dequantize_irht(packed_bins.to(self.device, torch.int32), n, centroids, nbits, diag, vec, n, self._inv_sqrt(n),
                                          post_scale=last)
            elif last is None:
                capi.rht_blocked(vec, diag, n, self._inv_sqrt(n), True)
            else:
                capi.rht_blocked(vec, diag, n, self._inv_sqrt(n), True)
                vec = scale32 * vec
        return vec[:orig_dim].to(vec_type)
