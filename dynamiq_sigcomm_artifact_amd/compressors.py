"""Compressor objects that wrap the `eden_utils` module -- the host-side mirror of
``Aee_Dynamic_Range_GPU_kern`` / ``Mee_Dynamic_Range_GPU_kern``
(testbed_evaluation/new_comm_hooks/utils_aggregation.py:369-569).

Same attribute names, the same buffer-size formulas, the same LCG that picks the
row offset into the pre-generated random pool, and the same five methods the ring
schedules call (compression / decompression / dec_compression /
decompression_add / create_tensor).  The only difference is where the world size
comes from: the reference asks ``torch.distributed``; here ``params`` may carry
``world_size`` / ``rank`` so that several simulated ranks can live in one
process on one GPU (``torch.distributed`` is still used when it is initialised
and ``params`` does not say otherwise).
"""
import torch

from . import load_eden_utils


def _world(params):
    if "world_size" in params:
        return int(params["world_size"]), int(params.get("rank", 0))
    import torch.distributed as dist
    if dist.is_available() and dist.is_initialized():
        return dist.get_world_size(), dist.get_rank()
    return 1, 0


def _method(params):
    args = params.get("args")
    return getattr(args, "aggregation_method", "") if args is not None else ""


class _DynamicRangeGPUKern(object):
    strategy = 2

    def __init__(self, nbits, chunk_size, params, device="cuda", generator=None):
        self.eden_utils = load_eden_utils()
        # the reference module only takes nbits in {2, 4, 8} and fp16/bf16 buffers; the *_ex
        # entry points (3/5/6/7-bit codes, fp32 buffers) are used only when asked for
        ex = bool(params.get("extended", False)) or nbits not in (2, 4, 8)
        eu = self.eden_utils
        self._compress = eu.scaling_compress_ex if ex else eu.scaling_compress
        self._decompress = eu.scaling_decompress_ex if ex else eu.scaling_decompress
        self._decompress_add = eu.scaling_decompress_add_ex if ex else eu.scaling_decompress_add
        self._dec_comp = eu.scaling_dec_comp_ex if ex else eu.scaling_dec_comp
        self.nbits = nbits
        self.chunk_size = chunk_size
        self.supergroup = 16
        self.range = (1 << (self.nbits - 1)) - 1
        self.params = params
        self.cur_max_size = 0
        self.nclients, self.client_rank = _world(params)
        self.device = device

        for d_index in params["d"]:
            self.cur_max_size = max(self.cur_max_size, (params["d"][d_index] + chunk_size) // chunk_size)

        self.three_times_cur_max_size = (3 * self.cur_max_size) // self.nclients
        pool = params.get("rand_pool_tensor")
        # not in the reference: params["philox_seed"] draws the rounding randomness inside the kernels (one stream per
        # rank, one step per call) and allocates no pool
        self.philox_seed = params.get("philox_seed")
        if self.philox_seed is not None:
            self.philox_seed = (int(self.philox_seed) + self.client_rank * 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF
            self.philox_step = (self.nbits << 32)
            self.randomized_vec_pool = None
            self.randomized_vec_pools = {}
            self.rand_seed = (self.nbits * 998244353) & 0xFFFFFFFF
            return
        if pool is not None:
            # caller-provided pool (the reference's "correlated" mode loads one from disk)
            self.randomized_vec_pool = pool.to(device=device)[: self.three_times_cur_max_size * self.chunk_size].view(
                self.three_times_cur_max_size, self.chunk_size)
        else:
            # NOTE: range is [0, 1]
            self.randomized_vec_pool = torch.rand(size=(self.three_times_cur_max_size, chunk_size), device=device,
                                                  generator=generator).to(torch.bfloat16)
        self.randomized_vec_pools = {self.randomized_vec_pool.dtype: self.randomized_vec_pool}
        self.rand_seed = (self.nbits * 998244353) & 0xFFFFFFFF

    def gen_next_rand(self):
        self.rand_seed = (self.rand_seed * 671431 + 1000000007) & 0xFFFFFFFF
        return self.rand_seed

    def padded_n(self, n):
        superchunk_elems = self.chunk_size * self.supergroup
        return (n + superchunk_elems - 1) // superchunk_elems * superchunk_elems

    def compressed_numel(self, n):
        padded_n = self.padded_n(n)
        packed_bytes = (self.chunk_size * self.nbits) // 8
        superchunks = padded_n // (self.chunk_size * self.supergroup)
        return superchunks * (self.supergroup * (packed_bytes + 1) + 2)

    def rand_pool(self, n, dtype):
        pool = self.randomized_vec_pools.get(dtype)
        if pool is None:
            pool = self.randomized_vec_pool.to(dtype=dtype)
            self.randomized_vec_pools[dtype] = pool

        randl_mod = pool.numel() // self.chunk_size - n // self.chunk_size - 1
        if randl_mod <= 0:
            raise RuntimeError("randomized_vec_pool is too small for scaling quantization")

        randl = self.gen_next_rand() % randl_mod
        return pool[randl:randl + n // self.chunk_size, :]

    def create_tensor(self, tensor, dtype):
        n = tensor.numel()
        padded_n = self.padded_n(n)
        if dtype == torch.uint8:
            padded_vec_size = self.compressed_numel(n)
        else:
            padded_vec_size = padded_n
        return torch.zeros(padded_vec_size, dtype=dtype, device=self.device)

    def _stream(self):
        return torch.cuda.current_stream().cuda_stream

    def _next_step(self):
        self.philox_step += 1
        return self.philox_step

    def compression(self, input_chunk, send_chunk, interm_chunk=None):
        n = input_chunk.numel()
        if n == 0:
            return
        if self.philox_seed is not None:
            self.eden_utils.scaling_compress_philox(input_chunk, send_chunk, n, self.nbits, self.chunk_size, self.philox_seed,
                                                    self._next_step(), self._stream(), self.strategy)
            return
        rand_vec = self.rand_pool(n, input_chunk.dtype)
        self._compress(input_chunk, send_chunk, rand_vec, n, self.nbits, self.chunk_size,
                                         self._stream(), self.strategy)

    def decompression(self, recv_chunk, input_chunk, interm_chunk=None):
        n = input_chunk.numel()
        if n == 0:
            return
        self._decompress(recv_chunk, input_chunk, n, self.nbits, self.chunk_size, self._stream(),
                                           self.strategy)

    def dec_compression(self, recv_chunk, input_chunk, send_chunk, interm_chunk=None, interm_chunk2=None):
        n = input_chunk.numel()
        if n == 0:
            return
        if self.philox_seed is not None:
            self.eden_utils.scaling_dec_comp_philox(recv_chunk, input_chunk, send_chunk, n, self.nbits, self.chunk_size,
                                                    self.philox_seed, self._next_step(), self._stream(), self.strategy)
            return
        rand_vec = self.rand_pool(n, input_chunk.dtype)
        self._dec_comp(recv_chunk, input_chunk, send_chunk, rand_vec, n, self.nbits, self.chunk_size,
                                         self._stream(), self.strategy)

    def decompression_add(self, recv_chunk, input_chunk, interm_chunk=None):
        n = input_chunk.numel()
        if n == 0:
            return
        self._decompress_add(recv_chunk, input_chunk, n, self.nbits, self.chunk_size, self._stream(),
                                               self.strategy)


    # ---- the same three steps over a list of superchunk indices (no counterpart in the reference:
    # they stand for index_select + the call above + index_copy_, comm_hooks.py:1001-1011) ----

    def compression_rows(self, full_tensor, rows, send_chunk):
        """send record k = compressed superchunk rows[k] of full_tensor"""
        nrows = rows.numel()
        if nrows == 0:
            return
        rand_vec = self.rand_pool(nrows * 256, full_tensor.dtype)
        self.eden_utils.scaling_compress_rows(full_tensor, rows, send_chunk, rand_vec, nrows, self.nbits,
                                              self._stream(), self.strategy)

    def dec_compression_rows(self, recv_chunk, full_tensor, rows, send_chunk):
        nrows = rows.numel()
        if nrows == 0:
            return
        rand_vec = self.rand_pool(nrows * 256, full_tensor.dtype)
        self.eden_utils.scaling_dec_comp_rows(recv_chunk, full_tensor, rows, send_chunk, rand_vec, nrows, self.nbits,
                                              self._stream(), self.strategy)

    def decompression_rows(self, recv_chunk, full_output, rows, stats=None, n_limit=None):
        """superchunk rows[k] of full_output = decoded record k (+ its mean from stats)"""
        nrows = rows.numel()
        if nrows == 0:
            return
        if n_limit is None:
            n_limit = full_output.numel()
        self.eden_utils.scaling_decompress_rows(recv_chunk, full_output, rows, stats, n_limit, nrows, self.nbits,
                                                self._stream(), self.strategy)


class Aee_Dynamic_Range_GPU_kern(_DynamicRangeGPUKern):
    """utils_aggregation.py:369-466 (hierarchical AEE, strategy 2)"""
    strategy = 2


class Mee_Dynamic_Range_GPU_kern(_DynamicRangeGPUKern):
    """utils_aggregation.py:470-569 (hierarchical MEE, strategy 3)"""
    strategy = 3

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
