"""THC's rotated uniform quantiser on the library's kernels -- the host-side mirror of
``EdenHadamardRHT`` and ``OldINCACudaHadamardCompressor``
(testbed_evaluation/new_comm_hooks/thc_hooks.py:81-181).

Same constructor parameters, same ``compress(tensor, name, max_norm)`` /
``decompress(tensor, name, max_norm=None)``; the element-wise chains of the reference
become the passes of one transform each way:

  compress    thc_rht_quantize: diagonal and Hadamard, with 1/sqrt(d) and the quantiser (sub, div, clamp, floor,
              Bernoulli add, bf16 cast) in the store of the last pass -- one pass in all for d <= 2^15
  decompress  thc_dequantize_irht: the dequantiser (cast, mul, add) in the load of the first pass of the inverse
              transform

The Bernoulli draws come from ``torch.rand`` on the sender generator (the reference calls
``bernoulli_`` on the same generator; the two consume torch's stream differently, so the
individual roundings differ while their distribution does not).  World size and rank come from
``params`` (``nclients``, ``rank``) or from torch.distributed when it is initialised.
"""
import ast
import math
import os
from pathlib import Path

import numpy as np
import torch

from . import capi


def _load_table_data(params):
    """thc_hooks.py:41-78: {'T': ...} from params, or from <table_dir>/<stem>data.txt"""
    if "T" in params:
        return {"T": float(params["T"])}
    table_size = params.get("table_size", 10001)
    max_val = params.get("max_val", 42)
    overflow_frequency = params.get("overflow_frequency", 1024)
    stem = f"{table_size}_tablesize_{max_val}_maxval_16_qlevels_{overflow_frequency}_ofreq_"
    candidates = []
    if os.environ.get("THC_TABLE_DIR"):
        candidates.append(Path(os.environ["THC_TABLE_DIR"]))
    if params.get("table_dir"):
        candidates.append(Path(params["table_dir"]))
    for table_dir in candidates:
        path = table_dir / f"{stem}data.txt"
        if path.exists():
            with path.open("r", encoding="utf-8") as fin:
                data = ast.literal_eval(fin.read())
            if "T" not in data:
                raise KeyError(f"THC table metadata at {path} does not contain key 'T'")
            return data
    searched = ", ".join(str(p / f"{stem}data.txt") for p in candidates)
    raise FileNotFoundError(
        "THC oldINCA table metadata not found. Set THC_TABLE_DIR to a directory containing "
        f"{stem}data.txt, or pass params['T']. Searched: {searched}")


def _world(params):
    if "nclients" in params:
        return int(params["nclients"]), int(params.get("rank", 0))
    import torch.distributed as dist
    if dist.is_available() and dist.is_initialized():
        return dist.get_world_size(), dist.get_rank()
    return 1, 0


class EdenHadamardRHT:
    """thc_hooks.py:81-107"""

    def __init__(self, dim, seed, device, key):
        if dim & (dim - 1):
            raise ValueError("eden_utils.Hadamard requires a power-of-two dimension")
        self.dim = dim
        self.device = device
        self.key = key
        self.generator = torch.Generator(device=device)
        self.generator.manual_seed((seed + 1000003 * int(key[0]) + 9176 * int(key[1])) & 0xFFFFFFFF)
        self.random_diagonal = torch.empty(dim, dtype=torch.float32, device=device)
        self.random_diagonal.bernoulli_(0.5, generator=self.generator)
        self.random_diagonal.mul_(2.0).sub_(1.0)
        # the kernels read the diagonal as one bit per element (1/32 of the traffic, same rotation)
        self.diagonal_bits = capi.pack_signs(self.random_diagonal)
        # div_(math.sqrt(dim)) with a host scalar is a product with the float32 reciprocal on the device
        self.inv_sqrt = float(np.float32(1.0) / np.float32(math.sqrt(dim)))

    def rht(self, vec):
        if vec.numel() != self.dim:
            raise ValueError(f"expected {self.dim} elements, got {vec.numel()}")
        capi.rht_blocked(vec, self.diagonal_bits, self.dim, self.inv_sqrt, False)
        return vec

    def irht(self, vec):
        if vec.numel() != self.dim:
            raise ValueError(f"expected {self.dim} elements, got {vec.numel()}")
        capi.rht_blocked(vec, self.diagonal_bits, self.dim, self.inv_sqrt, True)
        return vec


class OldINCACudaHadamardCompressor:
    """thc_hooks.py:110-181"""

    def __init__(self, params):
        capi.lib()
        self.device = params.get("device", "cuda")
        self.ds = params["d"]
        self.original_size = params["size"]
        self.seed = params.get("seed", 42)
        self.quantization_levels = params.get("quantization_levels", 64)
        self.nclients, rank = _world(params)
        self.data = _load_table_data(params)
        self.max_norm_dict = {}
        self.sender_prng = torch.Generator(device=self.device)
        self.sender_prng.manual_seed((self.seed + rank * 104729) & 0xFFFFFFFF)
        self.hadamards = {key: EdenHadamardRHT(dim, self.seed, self.device, key) for key, dim in self.ds.items()}
        self.work_buffers = {}

    def _work_buffer(self, name, dtype=torch.float32, tag="work"):
        dim = self.ds[name]
        buf = self.work_buffers.get((name, dtype, tag))
        if buf is None or buf.numel() != dim or buf.dtype != dtype:
            buf = torch.empty(dim, dtype=dtype, device=self.device)
            self.work_buffers[(name, dtype, tag)] = buf
        return buf

    def _coordinate_range(self, max_norm, dim):
        max_coordinate = self.data["T"] * max_norm / math.sqrt(dim)
        min_coordinate = -max_coordinate
        delta = (max_coordinate - min_coordinate) / (self.quantization_levels - 1) + 1e-23
        return min_coordinate, delta

    def compress(self, tensor, name, max_norm, uniform=None):
        orig_size = self.original_size[name]
        dim = self.ds[name]
        self.max_norm_dict[name] = max_norm
        work = self._work_buffer(name)
        work[:orig_size].copy_(tensor.float())
        if dim > orig_size:
            work[orig_size:].zero_()
        min_coordinate, delta = self._coordinate_range(max_norm, dim)
        if uniform is None:
            uniform = self._work_buffer(name, tag="uniform")
            uniform.uniform_(0.0, 1.0, generator=self.sender_prng)
        out = torch.empty(dim, dtype=torch.bfloat16, device=self.device)
        # rotation and quantiser in the transform's own passes: the rotated vector is never stored
        h = self.hadamards[name]
        capi.thc_rht_quantize(work, h.diagonal_bits, uniform, out, dim, h.inv_sqrt, min_coordinate.float().reshape(1),
                              delta.float().reshape(1), self.quantization_levels)
        return out

    def decompress(self, tensor, name, max_norm=None):
        if max_norm is None:
            max_norm = self.max_norm_dict[name]
        dim = self.ds[name]
        orig_size = self.original_size[name]
        min_coordinate, delta = self._coordinate_range(max_norm, dim)
        work = self._work_buffer(name)
        h = self.hadamards[name]
        capi.thc_dequantize_irht(tensor, h.diagonal_bits, work, dim, h.inv_sqrt,
                                 (delta / self.nclients).float().reshape(1), min_coordinate.float().reshape(1))
        return work[:orig_size]
