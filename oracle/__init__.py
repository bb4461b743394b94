"""ctypes front-end of the CPU oracle (``libdq_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and there only as the checker.

All element buffers are numpy arrays: fp16 / bf16 data travel as ``uint16``
bit patterns (``dtype`` says which), fp32 as ``float32``, packed records as
``uint8``.
"""
import ctypes
import os
import subprocess

import numpy as np

F16, BF16, F32 = 0, 1, 2
_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "libdq_oracle.so")

ERRORS = {
    1: "n must be positive",
    2: "nbits must be one of {2, 4, 8}",
    3: "strategy must be 0 (AEE), 1 (MEE), 2 (hierarchical AEE), or 3 (hierarchical MEE)",
    4: "chunk_size must be in [1, 32]",
    5: "chunk_size must be a power of two",
    6: "chunk_size * nbits must be divisible by 8",
    7: "n must be a multiple of chunk_size",
    8: "hierarchical mode requires n to contain a whole number of 16-chunk superchunks",
    9: "unsupported dtype",
}


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _DIR])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(L):
    c = ctypes
    vp, i64, i32 = c.c_void_p, c.c_int64, c.c_int
    L.dqo_scaling_required_bytes.restype = i64
    L.dqo_scaling_required_bytes.argtypes = [i64, i32, i32, i32]
    L.dqo_scaling_check.restype = i32
    L.dqo_scaling_check.argtypes = [i64, i32, i32, i32, i32]
    L.dqo_mee_lut.restype = None
    L.dqo_mee_lut.argtypes = [i32, vp, vp]
    L.dqo_log2f.restype = c.c_float
    L.dqo_log2f.argtypes = [c.c_float]
    L.dqo_bf16_to_f32.restype = c.c_float
    L.dqo_bf16_to_f32.argtypes = [c.c_uint16]
    L.dqo_f32_to_bf16.restype = c.c_uint16
    L.dqo_f32_to_bf16.argtypes = [c.c_float]
    L.dqo_f16_to_f32.restype = c.c_float
    L.dqo_f16_to_f32.argtypes = [c.c_uint16]
    L.dqo_f32_to_f16.restype = c.c_uint16
    L.dqo_f32_to_f16.argtypes = [c.c_float]
    L.dqo_scaling_compress.restype = i32
    L.dqo_scaling_compress.argtypes = [vp, vp, vp, i64, i32, i32, i32, i32]
    L.dqo_scaling_decompress.restype = i32
    L.dqo_scaling_decompress.argtypes = [vp, vp, i64, i32, i32, i32, i32, i32]
    L.dqo_scaling_dec_comp.restype = i32
    L.dqo_scaling_dec_comp.argtypes = [vp, vp, vp, vp, i64, i32, i32, i32, i32]
    L.dqo_superchunk_stats.restype = None
    L.dqo_superchunk_stats.argtypes = [vp, vp, vp, i64, i32, i32]
    L.dqo_superchunk_mean_center.restype = None
    L.dqo_superchunk_mean_center.argtypes = [vp, vp, vp, i64, i32, i32]
    L.dqo_superchunk_add_mean_copy.restype = None
    L.dqo_superchunk_add_mean_copy.argtypes = [vp, vp, vp, i64, i32]
    L.dqo_fwht.restype = None
    L.dqo_fwht.argtypes = [vp, i64]
    L.dqo_rht_blocked.restype = None
    L.dqo_rht_blocked.argtypes = [vp, vp, i64, i64, c.c_float, i32]
    L.dqo_rand_diag.restype = None
    L.dqo_rand_diag.argtypes = [vp, i64, i64]
    L.dqo_bins_to_bits.restype = None
    L.dqo_bins_to_bits.argtypes = [vp, i64, vp, i32]
    L.dqo_bits_to_bins.restype = None
    L.dqo_bits_to_bins.argtypes = [vp, i64, vp, i32]
    L.dqo_dynamic_bitrate_qbits.restype = None
    L.dqo_dynamic_bitrate_qbits.argtypes = [vp, i64, i64, c.c_double, vp]


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _elem_dtype(dtype):
    return np.float32 if dtype == F32 else np.uint16


def _chk(a, dt, name):
    if not isinstance(a, np.ndarray) or a.dtype != dt or not a.flags["C_CONTIGUOUS"]:
        raise TypeError("%s must be a C-contiguous numpy array of %s" % (name, np.dtype(dt)))


def _raise(rc):
    if rc:
        raise RuntimeError(ERRORS.get(rc, "oracle error %d" % rc))


def required_bytes(n, nbits, chunk_size, strategy):
    return int(lib().dqo_scaling_required_bytes(n, nbits, chunk_size, strategy))


def scaling_check(n, nbits, chunk_size, strategy, strict=True):
    return int(lib().dqo_scaling_check(n, nbits, chunk_size, strategy, 1 if strict else 0))


def mee_lut(nbits):
    """Returns (table[256] uint16 half bits, params[4] uint16 half bits)."""
    table = np.zeros(256, np.uint16)
    params = np.zeros(4, np.uint16)
    lib().dqo_mee_lut(nbits, _p(table), _p(params))
    return table, params


def log2f(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x)
    L = lib()
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    for i in range(flat_in.size):
        flat_out[i] = L.dqo_log2f(float(flat_in[i]))
    return out


def f32_to_bf16(x):
    L = lib()
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    return np.array([L.dqo_f32_to_bf16(float(v)) for v in x], np.uint16)


def f32_to_f16(x):
    L = lib()
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    return np.array([L.dqo_f32_to_f16(float(v)) for v in x], np.uint16)


def bf16_to_f32(h):
    return (np.ascontiguousarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f16_to_f32(h):
    return np.ascontiguousarray(h, np.uint16).view(np.float16).astype(np.float32)


def scaling_compress(src, rand_pool, n, nbits, chunk_size, strategy, dtype, dst=None):
    ed = _elem_dtype(dtype)
    _chk(src, ed, "src")
    _chk(rand_pool, ed, "rand_pool")
    _raise(scaling_check(n, nbits, chunk_size, strategy, strict=False))
    assert src.size >= n and rand_pool.size >= n
    nbytes = required_bytes(n, nbits, chunk_size, strategy)
    if dst is None:
        dst = np.zeros(nbytes, np.uint8)
    _chk(dst, np.uint8, "dst")
    assert dst.size >= nbytes
    _raise(lib().dqo_scaling_compress(_p(src), _p(dst), _p(rand_pool), n, nbits, chunk_size, strategy, dtype))
    return dst


def scaling_decompress(src, dst, n, nbits, chunk_size, strategy, dtype, add=False):
    _chk(src, np.uint8, "src")
    _chk(dst, _elem_dtype(dtype), "dst")
    _raise(scaling_check(n, nbits, chunk_size, strategy, strict=False))
    assert src.size >= required_bytes(n, nbits, chunk_size, strategy) and dst.size >= n
    _raise(lib().dqo_scaling_decompress(_p(src), _p(dst), n, nbits, chunk_size, strategy, dtype, 1 if add else 0))
    return dst


def scaling_dec_comp(recv, inp, rand_pool, n, nbits, chunk_size, strategy, dtype, send=None):
    ed = _elem_dtype(dtype)
    _chk(recv, np.uint8, "recv")
    _chk(inp, ed, "inp")
    _chk(rand_pool, ed, "rand_pool")
    _raise(scaling_check(n, nbits, chunk_size, strategy, strict=False))
    nbytes = required_bytes(n, nbits, chunk_size, strategy)
    if send is None:
        send = np.zeros(nbytes, np.uint8)
    _chk(send, np.uint8, "send")
    assert recv.size >= nbytes and send.size >= nbytes and inp.size >= n and rand_pool.size >= n
    _raise(lib().dqo_scaling_dec_comp(_p(recv), _p(inp), _p(send), _p(rand_pool), n, nbits, chunk_size, strategy, dtype))
    return send


def superchunk_mean_center(src, n, world_size, dtype):
    ed = _elem_dtype(dtype)
    _chk(src, ed, "src")
    nsc = (n + 255) // 256
    residual = np.zeros(nsc * 256, ed)
    stats = np.zeros(nsc * 2, np.uint16)
    lib().dqo_superchunk_mean_center(_p(src), _p(residual), _p(stats), n, world_size, dtype)
    return residual, stats


def superchunk_stats(src, n, world_size, dtype):
    """(stats uint16 [2 nsc], means float32 [nsc]) of superchunk_mean_center, no residual"""
    _chk(src, _elem_dtype(dtype), "src")
    nsc = (n + 255) // 256
    stats = np.zeros(nsc * 2, np.uint16)
    mean = np.zeros(nsc, np.float32)
    lib().dqo_superchunk_stats(_p(src), _p(stats), _p(mean), n, world_size, dtype)
    return stats, mean


def superchunk_add_mean_copy(residual, stats, n, dtype, dst=None):
    ed = _elem_dtype(dtype)
    _chk(residual, ed, "residual")
    _chk(stats, np.uint16, "stats")
    if dst is None:
        dst = np.zeros(n, ed)
    _chk(dst, ed, "dst")
    lib().dqo_superchunk_add_mean_copy(_p(residual), _p(dst), _p(stats), n, dtype)
    return dst


def fwht(x):
    x = np.array(x, np.float32, copy=True)
    n = x.size
    assert n > 0 and (n & (n - 1)) == 0
    lib().dqo_fwht(_p(x), n)
    return x


def rht_blocked(x, sign, block, scale, inverse=False):
    x = np.array(x, np.float32, copy=True)
    _chk(sign, np.float32, "sign")
    assert sign.size >= x.size and x.size % block == 0
    lib().dqo_rht_blocked(_p(x), _p(sign), x.size, block, float(scale), 1 if inverse else 0)
    return x


def rand_diag(size, seed):
    out = np.zeros(size, np.float32)
    lib().dqo_rand_diag(_p(out), size, seed)
    return out


def bins_to_bits(bins, nbits):
    _chk(bins, np.int32, "bins")
    assert bins.size % 32 == 0
    arr = np.zeros(bins.size // 32 * nbits, np.uint32)
    lib().dqo_bins_to_bits(_p(bins), bins.size, _p(arr), nbits)
    return arr


def bits_to_bins(arr, nbits):
    _chk(arr, np.uint32, "arr")
    bins = np.zeros(arr.size // nbits * 32, np.int32)
    lib().dqo_bits_to_bins(_p(arr), arr.size, _p(bins), nbits)
    return bins


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, np.uint32)
    k = np.asarray(key, np.uint32)
    out = np.zeros(4, np.uint32)
    f = lib().dqo_philox4x32_10
    f.restype = None
    f.argtypes = [ctypes.c_void_p] * 3
    f(_p(c), _p(k), _p(out))
    return out


def philox_uniform(n, seed, step):
    out = np.zeros(n, np.float32)
    f = lib().dqo_philox_uniform
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_uint64]
    f(_p(out), n, int(seed), int(step))
    return out


def philox_uniform_rows(rows, seed, step):
    """the values of philox_uniform for the superchunks (256 elements each) listed in rows, concatenated"""
    rows = np.ascontiguousarray(rows, np.int64)
    out = np.zeros(rows.size * 256, np.float32)
    f = lib().dqo_philox_uniform_rows
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_uint64]
    f(_p(out), _p(rows), rows.size, int(seed), int(step))
    return out


def eden_quantize(vec, boundaries, centroids, nbits):
    """-> (bins int32 [n], result float32 [4] = sumsq, dot, scale, norm)"""
    _chk(vec, np.float32, "vec")
    _chk(boundaries, np.float32, "boundaries")
    _chk(centroids, np.float32, "centroids")
    assert boundaries.size == (1 << nbits) - 1 and centroids.size == 1 << nbits
    bins = np.zeros(vec.size, np.int32)
    result = np.zeros(4, np.float32)
    f = lib().dqo_eden_quantize
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    f(_p(vec), vec.size, _p(boundaries), _p(centroids), nbits, _p(bins), _p(result))
    return bins, result


def eden_dequantize(bins, centroids):
    _chk(bins, np.int32, "bins")
    _chk(centroids, np.float32, "centroids")
    out = np.zeros(bins.size, np.float32)
    f = lib().dqo_eden_dequantize
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    f(_p(bins), bins.size, _p(centroids), _p(out))
    return out


def thc_quantize(rotated, uniform, lo, delta, levels):
    _chk(rotated, np.float32, "rotated")
    _chk(uniform, np.float32, "uniform")
    out = np.zeros(rotated.size, np.uint16)
    f = lib().dqo_thc_quantize
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_float, ctypes.c_int]
    f(_p(rotated), _p(uniform), _p(out), rotated.size, float(lo), float(delta), levels)
    return out


def thc_dequantize(levels_bf16, step, lo):
    _chk(levels_bf16, np.uint16, "levels")
    out = np.zeros(levels_bf16.size, np.float32)
    f = lib().dqo_thc_dequantize
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_float]
    f(_p(levels_bf16), _p(out), levels_bf16.size, float(step), float(lo))
    return out


def dynamic_bitrate_qbits(norms_bf16, u, stride=1):
    _chk(norms_bf16, np.uint16, "norms")
    count = (norms_bf16.size + stride - 1) // stride
    q = np.zeros(count, np.int64)
    lib().dqo_dynamic_bitrate_qbits(_p(norms_bf16), stride, count, float(u), _p(q))
    return q


def argsort_descending_stable(norms_bf16, stride=1):
    """comm_hooks.py:718 on bf16 bit patterns: int64 order"""
    _chk(norms_bf16, np.uint16, "norms")
    count = (norms_bf16.size + stride - 1) // stride
    order = np.zeros(count, np.int64)
    f = lib().dqo_argsort_descending_stable
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]
    f(_p(norms_bf16), stride, count, _p(order))
    return order


def fixed_proportion_groups(norms_bf16, top_count, bottom_count, stride=1):
    """comm_hooks.py:718-721: the 8-, 4- and 2-bit index lists, each in sorted order"""
    order = argsort_descending_stable(norms_bf16, stride)
    n = order.size
    return order[:top_count], order[top_count:n - bottom_count], order[n - bottom_count:]


def quantization(vec, div_factor, tensor_max, seed):
    """cuda_hadamard.cu:607-627 on a float32 array (returns a new array)"""
    out = np.ascontiguousarray(vec, np.float32).copy()
    f = lib().dqo_quantization
    f.restype = None
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_float, ctypes.c_uint64]
    f(_p(out), out.size, float(div_factor), float(tensor_max), int(seed))
    return out


# ---- the search for the offset u (comm_hooks.py:48-139) -----------------------------------------------
# Plain Python around dqo_dynamic_bitrate_qbits: at most 33 evaluations, each one pass of the C rule over the
# norms.  Pinned by the same search written with the reference's own torch ops on the CPU (the package's
# bitrate module) -- see tests/test_oracle_misc.py.

BITRATE_U_MIN, BITRATE_U_MAX, BITRATE_TOL, BITRATE_MAX_ITERS = -10.0, 60.0, 0.1, 32


def dynamic_bitrate_avg_delta(norms_list, u, target):
    """comm_hooks.py:73-91; norms_list: arrays of bf16 bit patterns"""
    bits = chunks = 0
    for norms in norms_list:
        if norms.size:
            bits += int(dynamic_bitrate_qbits(np.ascontiguousarray(norms), u).sum())
            chunks += norms.size
    avg = float(bits) / chunks if chunks else 0.0
    return avg, target - avg


def dynamic_bitrate_binary_search_u(norms_list, target):
    """comm_hooks.py:94-114"""
    low, high = BITRATE_U_MIN, BITRATE_U_MAX
    best = (high,) + dynamic_bitrate_avg_delta(norms_list, high, target)
    for _ in range(BITRATE_MAX_ITERS):
        mid = (low + high) * 0.5
        avg, delta = dynamic_bitrate_avg_delta(norms_list, mid, target)
        if abs(delta) < abs(best[2]):
            best = (mid, avg, delta)
        if abs(delta) <= BITRATE_TOL:
            return mid, avg, delta
        if delta > 0:
            low = mid
        else:
            high = mid
    return best


def dynamic_bitrate_adjust_u(norms_list, prev_u, target):
    """comm_hooks.py:117-139"""
    prev_u = max(BITRATE_U_MIN, min(BITRATE_U_MAX, float(prev_u)))
    old_avg, old_delta = dynamic_bitrate_avg_delta(norms_list, prev_u, target)
    if abs(old_delta) <= BITRATE_TOL:
        return prev_u, old_avg, old_delta
    step = old_delta
    best = (prev_u, old_avg, old_delta)
    for _ in range(BITRATE_MAX_ITERS):
        cand = max(BITRATE_U_MIN, min(BITRATE_U_MAX, prev_u + step))
        avg, delta = dynamic_bitrate_avg_delta(norms_list, cand, target)
        if abs(delta) < abs(best[2]):
            best = (cand, avg, delta)
        if abs(delta) <= BITRATE_TOL or old_delta * delta >= 0:
            return cand, avg, delta
        step *= 0.5
    return best
