"""Compressor objects over the ``eden_utils`` module: drop-ins for ``Aee_Dynamic_Range_GPU_kern`` and
``Mee_Dynamic_Range_GPU_kern`` (testbed_evaluation/new_comm_hooks/utils_aggregation.py:369-569), the objects the ring
schedules call as ``compression / decompression / dec_compression / decompression_add / create_tensor``.

What callers and wire partners depend on is kept: the attribute names, the packed size of a vector, and which rows of
the pre-generated random pool a call uses (an LCG keyed by the code width picks the first row, so two ranks built with
the same arguments walk the same offsets).  Two additions: ``params`` may carry ``world_size`` / ``rank`` so that
several simulated ranks can live in one process on one GPU, and ``params["philox_seed"]`` switches to rounding
randomness drawn inside the kernels (no pool).  The ``*_rows`` methods serve a list of superchunks of a larger buffer
without gathering it first.
"""
import torch

from . import load_eden_utils

_U32 = 0xFFFFFFFF
_SUPERGROUP = 16                      # chunks per superchunk


def _world(params):
    if "world_size" in params:
        return int(params["world_size"]), int(params.get("rank", 0))
    import torch.distributed as dist
    if dist.is_available() and dist.is_initialized():
        return dist.get_world_size(), dist.get_rank()
    return 1, 0


def record_geometry(nbits, chunk_size, supergroup=_SUPERGROUP):
    """(elements per superchunk, bytes per record): a record is `supergroup` x (packed codes + one scale byte) + the
    two-byte unit -- utils_aggregation.py:403-407, eden_utils.cpp:33-40"""
    return chunk_size * supergroup, supergroup * (chunk_size * nbits // 8 + 1) + 2


class _DynamicRangeGPUKern(object):
    strategy = 2
    given_pool_dtype = None           # dtype a pool passed in params["rand_pool_tensor"] is kept in (None: its own)

    def __init__(self, nbits, chunk_size, params, device="cuda", generator=None):
        eu = self.eden_utils = load_eden_utils()
        # the reference module takes 2/4/8-bit codes and fp16/bf16 buffers; other widths and fp32 buffers go through
        # the *_ex entry points, on request only
        suffix = "_ex" if params.get("extended", False) or nbits not in (2, 4, 8) else ""
        self._compress = getattr(eu, "scaling_compress" + suffix)
        self._decompress = getattr(eu, "scaling_decompress" + suffix)
        self._decompress_add = getattr(eu, "scaling_decompress_add" + suffix)
        self._dec_comp = getattr(eu, "scaling_dec_comp" + suffix)

        self.nbits, self.chunk_size, self.params, self.device = nbits, chunk_size, params, device
        self.supergroup = _SUPERGROUP
        self.range = (1 << (nbits - 1)) - 1
        self.nclients, self.client_rank = _world(params)
        self._super_elems, self._record_bytes = record_geometry(nbits, chunk_size, self.supergroup)

        # pool rows: three times the chunks of the longest vector, shared out over the ranks (:384-386)
        self.cur_max_size = max([(d + chunk_size) // chunk_size for d in params["d"].values()] + [0])
        self.three_times_cur_max_size = 3 * self.cur_max_size // self.nclients
        self.rand_seed = (nbits * 998244353) & _U32

        self.philox_seed = params.get("philox_seed")
        self.randomized_vec_pool, self.randomized_vec_pools = None, {}
        if self.philox_seed is not None:
            # one stream per rank, one step per call
            self.philox_seed = (int(self.philox_seed) + self.client_rank * 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
            self.philox_step = nbits << 32
            return
        rows = self.three_times_cur_max_size
        given = params.get("rand_pool_tensor")          # the reference's "correlated" mode loads its pool from disk
        if given is None:
            pool = torch.rand((rows, chunk_size), device=device, generator=generator).to(torch.bfloat16)   # values in [0, 1]
        else:
            pool = given.to(device=device)[:rows * chunk_size].view(rows, chunk_size)
            if self.given_pool_dtype is not None:
                # the MEE class keeps a loaded pool in binary16 (:488), the AEE class in the dtype of the file (:389): a
                # bf16 caller of the MEE class therefore sees values rounded twice, and so must this one
                pool = pool.to(dtype=self.given_pool_dtype)
        self.randomized_vec_pool = pool
        self.randomized_vec_pools[pool.dtype] = pool

    # ---- sizes --------------------------------------------------------------------------------------------
    def padded_n(self, n):
        return -(-n // self._super_elems) * self._super_elems

    def compressed_numel(self, n):
        return self.padded_n(n) // self._super_elems * self._record_bytes

    def create_tensor(self, tensor, dtype):
        n = tensor.numel()
        size = self.compressed_numel(n) if dtype == torch.uint8 else self.padded_n(n)
        return torch.zeros(size, dtype=dtype, device=self.device)

    # ---- rounding randomness ------------------------------------------------------------------------------
    def gen_next_rand(self):
        """the LCG of :391-393; its state is an attribute the reference's callers may read"""
        self.rand_seed = (self.rand_seed * 671431 + 1000000007) & _U32
        return self.rand_seed

    def rand_pool(self, n, dtype):
        """n / chunk_size consecutive pool rows in `dtype`, starting at a row the LCG picks (:409-420)"""
        pool = self.randomized_vec_pools.get(dtype)
        if pool is None:
            pool = self.randomized_vec_pools[dtype] = self.randomized_vec_pool.to(dtype=dtype)
        rows = n // self.chunk_size
        choices = pool.shape[0] - rows - 1
        if choices <= 0:
            raise RuntimeError("randomized_vec_pool is too small for scaling quantization")
        first = self.gen_next_rand() % choices
        return pool[first:first + rows, :]

    def _next_step(self):
        self.philox_step += 1
        return self.philox_step

    @staticmethod
    def _stream():
        return torch.cuda.current_stream().cuda_stream

    # ---- the calls of the ring schedules (:422-466) ------------------------------------------------------
    def compression(self, input_chunk, send_chunk, interm_chunk=None):
        n = input_chunk.numel()
        if n == 0:
            return
        tail = (n, self.nbits, self.chunk_size)
        if self.philox_seed is None:
            self._compress(input_chunk, send_chunk, self.rand_pool(n, input_chunk.dtype), *tail, self._stream(), self.strategy)
        else:
            self.eden_utils.scaling_compress_philox(input_chunk, send_chunk, *tail, self.philox_seed, self._next_step(),
                                                    self._stream(), self.strategy)

    def decompression(self, recv_chunk, input_chunk, interm_chunk=None):
        n = input_chunk.numel()
        if n:
            self._decompress(recv_chunk, input_chunk, n, self.nbits, self.chunk_size, self._stream(), self.strategy)

    def decompression_add(self, recv_chunk, input_chunk, interm_chunk=None):
        n = input_chunk.numel()
        if n:
            self._decompress_add(recv_chunk, input_chunk, n, self.nbits, self.chunk_size, self._stream(), self.strategy)

    def dec_compression(self, recv_chunk, input_chunk, send_chunk, interm_chunk=None, interm_chunk2=None):
        n = input_chunk.numel()
        if n == 0:
            return
        tail = (n, self.nbits, self.chunk_size)
        if self.philox_seed is None:
            self._dec_comp(recv_chunk, input_chunk, send_chunk, self.rand_pool(n, input_chunk.dtype), *tail, self._stream(),
                           self.strategy)
        else:
            self.eden_utils.scaling_dec_comp_philox(recv_chunk, input_chunk, send_chunk, *tail, self.philox_seed,
                                                    self._next_step(), self._stream(), self.strategy)

    # ---- the same steps over a list of superchunk indices: index_select + the call above + index_copy_
    #      (comm_hooks.py:1001-1011) without the gathered copy; no counterpart in the reference ----
    def _rows_supported(self):
        if self.chunk_size != 16:
            raise ValueError("the row-list kernels serve superchunks of 16 chunks of 16 elements; chunk_size is %d" % self.chunk_size)

    def compression_rows(self, full_tensor, rows, send_chunk):
        """send record k = compressed superchunk rows[k] of full_tensor"""
        self._rows_supported()
        count = rows.numel()
        if count:
            self.eden_utils.scaling_compress_rows(full_tensor, rows, send_chunk, self.rand_pool(count * self._super_elems, full_tensor.dtype),
                                                  count, self.nbits, self._stream(), self.strategy)

    def dec_compression_rows(self, recv_chunk, full_tensor, rows, send_chunk):
        self._rows_supported()
        count = rows.numel()
        if count:
            self.eden_utils.scaling_dec_comp_rows(recv_chunk, full_tensor, rows, send_chunk,
                                                  self.rand_pool(count * self._super_elems, full_tensor.dtype), count, self.nbits,
                                                  self._stream(), self.strategy)

    def decompression_rows(self, recv_chunk, full_output, rows, stats=None, n_limit=None):
        """superchunk rows[k] of full_output = decoded record k (+ its mean from stats)"""
        self._rows_supported()
        count = rows.numel()
        if count:
            self.eden_utils.scaling_decompress_rows(recv_chunk, full_output, rows, stats,
                                                    full_output.numel() if n_limit is None else n_limit, count, self.nbits,
                                                    self._stream(), self.strategy)


class Aee_Dynamic_Range_GPU_kern(_DynamicRangeGPUKern):
    """utils_aggregation.py:369-466 (hierarchical AEE, strategy 2)"""
    strategy = 2


class Mee_Dynamic_Range_GPU_kern(_DynamicRangeGPUKern):
    """utils_aggregation.py:470-569 (hierarchical MEE, strategy 3)"""
    strategy = 3
    given_pool_dtype = torch.float16

    def __init__(self, nbits, chunk_size, params, device="cuda", generator=None):
        super().__init__(nbits, chunk_size, params, device=device, generator=generator)
        self.eden_utils.init_lookup_table()


def superchunk_mean_center(input_tensor, residual, stats, n, world_size, superchunk_size):
    """utils_aggregation.py:340-352"""
    load_eden_utils().superchunk_mean_center(input_tensor, residual, stats, n, world_size, superchunk_size,
                                             torch.cuda.current_stream().cuda_stream)


def superchunk_add_mean_copy(residual, output_tensor, stats, n, superchunk_size):
    """utils_aggregation.py:355-366"""
    load_eden_utils().superchunk_add_mean_copy(residual, output_tensor, stats, n, superchunk_size,
                                               torch.cuda.current_stream().cuda_stream)
