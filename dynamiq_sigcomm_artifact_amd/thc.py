"""THC's rotated uniform quantiser on the library's kernels: drop-in classes for ``EdenHadamardRHT`` and
``OldINCACudaHadamardCompressor`` (testbed_evaluation/new_comm_hooks/thc_hooks.py:81-181).

The public surface is the reference's -- constructor parameters, ``rht`` / ``irht``, ``compress(tensor, name,
max_norm)`` / ``decompress(tensor, name, max_norm=None)``, the attributes hooks read (``ds``, ``original_size``,
``quantization_levels``, ``nclients``, ``data``, ``hadamards``, ``random_diagonal``, ``sender_prng``) -- but the
element-wise torch chains are gone:

  compress    one call of thc_rht_quantize: diagonal, Hadamard, 1/sqrt(d) and the quantiser (subtract, divide,
              clamp, floor, Bernoulli carry, bf16 cast) in the store of the transform's last pass
  decompress  one call of thc_dequantize_irht: cast, multiply, add in the load of the inverse transform's first pass

The Bernoulli draws come from ``uniform_`` on the sender generator (the reference calls ``bernoulli_`` on the same
generator; the two consume torch's stream differently, so individual roundings differ while their distribution
does not).  World size and rank come from ``params`` (``nclients``, ``rank``) or from torch.distributed.
"""
import ast
import math
import os

import numpy as np
import torch

from . import capi

_TABLE_FILE = "{table_size}_tablesize_{max_val}_maxval_16_qlevels_{overflow_frequency}_ofreq_data.txt"
_TABLE_DEFAULTS = {"table_size": 10001, "max_val": 42, "overflow_frequency": 1024}


def _clip_threshold(params):
    """The clipping threshold T of the rotated coordinates (thc_hooks.py:41-78 reads it from the table metadata
    file): params['T'] when given, else the 'T' entry of the metadata file in $THC_TABLE_DIR or params['table_dir']."""
    if "T" in params:
        return {"T": float(params["T"])}
    name = _TABLE_FILE.format(**{k: params.get(k, v) for k, v in _TABLE_DEFAULTS.items()})
    tried = []
    for folder in (os.environ.get("THC_TABLE_DIR"), params.get("table_dir")):
        if not folder:
            continue
        path = os.path.join(str(folder), name)
        tried.append(path)
        if os.path.exists(path):
            with open(path, "r", encoding="utf-8") as f:
                meta = ast.literal_eval(f.read())
            if "T" not in meta:
                raise KeyError("THC table metadata at %s does not contain key 'T'" % path)
            return meta
    raise FileNotFoundError("THC oldINCA table metadata not found (%s): pass params['T'], or set THC_TABLE_DIR / "
                            "params['table_dir'] to the directory that holds it. Searched: %s" % (name, ", ".join(tried)))


def _world(params):
    if "nclients" in params:
        return int(params["nclients"]), int(params.get("rank", 0))
    import torch.distributed as dist
    if dist.is_available() and dist.is_initialized():
        return dist.get_world_size(), dist.get_rank()
    return 1, 0


class EdenHadamardRHT:
    """thc_hooks.py:81-107: y = H (D x) / sqrt(d) and its inverse, D a fixed random +-1 diagonal per (seed, key)"""

    def __init__(self, dim, seed, device, key):
        if dim <= 0 or dim & (dim - 1):
            raise ValueError("eden_utils.Hadamard requires a power-of-two dimension")
        self.dim, self.device, self.key = dim, device, key
        # the diagonal is torch's Bernoulli stream for this seed: drawn by torch here as well
        self.generator = torch.Generator(device=device)
        self.generator.manual_seed((seed + 1000003 * int(key[0]) + 9176 * int(key[1])) & 0xFFFFFFFF)
        coin = torch.empty(dim, dtype=torch.float32, device=device).bernoulli_(0.5, generator=self.generator)
        self.random_diagonal = coin.mul_(2.0).sub_(1.0)
        # the kernels take the diagonal as one bit per element (1/32 of the traffic, the same rotation), and the
        # division by sqrt(d) as the product with its float32 reciprocal, which is what torch's div_ by a host
        # scalar does on the device
        self.diagonal_bits = capi.pack_signs(self.random_diagonal)
        self.inv_sqrt = float(np.float32(1.0) / np.float32(math.sqrt(dim)))

    def _rotate(self, vec, inverse):
        if vec.numel() != self.dim:
            raise ValueError(f"expected {self.dim} elements, got {vec.numel()}")
        capi.rht_blocked(vec, self.diagonal_bits, self.dim, self.inv_sqrt, inverse)
        return vec

    def rht(self, vec):
        return self._rotate(vec, False)

    def irht(self, vec):
        return self._rotate(vec, True)


class OldINCACudaHadamardCompressor:
    """thc_hooks.py:110-181: pad to the rotation's dimension, rotate, quantise to `quantization_levels` uniform
    levels over [-T |x| / sqrt(d), +T |x| / sqrt(d)] with stochastic rounding; the aggregate of `nclients` such
    vectors decodes with the step divided by nclients"""

    def __init__(self, params):
        capi.lib()
        self.device = params.get("device", "cuda")
        self.ds = params["d"]
        self.original_size = params["size"]
        self.seed = params.get("seed", 42)
        self.quantization_levels = params.get("quantization_levels", 64)
        self.nclients, rank = _world(params)
        self.data = _clip_threshold(params)
        self.max_norm_dict = {}
        self.sender_prng = torch.Generator(device=self.device)
        self.sender_prng.manual_seed((self.seed + rank * 104729) & 0xFFFFFFFF)
        self.hadamards = {key: EdenHadamardRHT(dim, self.seed, self.device, key) for key, dim in self.ds.items()}
        self._scratch = {}

    def _buffer(self, name, role):
        """a float32 scratch vector of the rotation's dimension, kept per (tensor name, role)"""
        dim = self.ds[name]
        buf = self._scratch.get((name, role))
        if buf is None or buf.numel() != dim:
            buf = self._scratch[(name, role)] = torch.empty(dim, dtype=torch.float32, device=self.device)
        return buf

    def _grid(self, max_norm, dim):
        """(lowest level, level spacing) as float32 device scalars of shape [1]; the arithmetic and its order are the
        reference's (thc_hooks.py:143-147), done on max_norm's own type"""
        top = self.data["T"] * max_norm / math.sqrt(dim)
        low = -top
        spacing = (top - low) / (self.quantization_levels - 1) + 1e-23
        return low, spacing

    @staticmethod
    def _scalar(v, device):
        if isinstance(v, torch.Tensor):
            return v.to(device=device, dtype=torch.float32).reshape(1)
        return torch.tensor([v], dtype=torch.float32, device=device)

    def compress(self, tensor, name, max_norm, uniform=None):
        dim, used = self.ds[name], self.original_size[name]
        self.max_norm_dict[name] = max_norm
        work = self._buffer(name, "work")
        work[:used].copy_(tensor.float())
        if dim > used:
            work[used:].zero_()
        low, spacing = self._grid(max_norm, dim)
        if uniform is None:
            uniform = self._buffer(name, "uniform").uniform_(0.0, 1.0, generator=self.sender_prng)
        levels = torch.empty(dim, dtype=torch.bfloat16, device=self.device)
        rot = self.hadamards[name]
        capi.thc_rht_quantize(work, rot.diagonal_bits, uniform, levels, dim, rot.inv_sqrt, self._scalar(low, self.device),
                              self._scalar(spacing, self.device), self.quantization_levels)
        return levels

    def decompress(self, tensor, name, max_norm=None):
        if max_norm is None:
            max_norm = self.max_norm_dict[name]
        dim, used = self.ds[name], self.original_size[name]
        low, spacing = self._grid(max_norm, dim)
        out = self._buffer(name, "work")
        rot = self.hadamards[name]
        capi.thc_dequantize_irht(tensor, rot.diagonal_bits, out, dim, rot.inv_sqrt,
                                 self._scalar(spacing / self.nclients, self.device), self._scalar(low, self.device))
        return out[:used]
