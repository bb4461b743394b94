"""ctypes binding of the C ABI (``include/dynamiq_eden.h``) for torch tensors.

Thin and explicit on purpose: each wrapper passes ``data_ptr()``, sizes, the
device index and a stream handle straight to ``libdynamiq_eden.so`` and raises
``RuntimeError`` with the library's message when the status is non-zero.  The
library must be present; there is no fallback path.
"""
import ctypes
import threading
import os

import torch

F16, BF16, F32 = 0, 1, 2
RAND_BF16 = 0x10
_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libdynamiq_eden.so")

EXPORTS = [
    "dq_status_string", "dq_last_error", "dq_version",
    "dq_scaling_required_bytes", "dq_scaling_check_common",
    "dq_init_lookup_table", "dq_mee_lookup_table",
    "dq_scaling_compress", "dq_scaling_decompress", "dq_scaling_dec_comp",
    "dq_scaling_compress_philox", "dq_scaling_dec_comp_philox", "dq_philox_uniform",
    "dq_group_plan_work_ints", "dq_group_plan_sorted_work_ints", "dq_group_plan", "dq_group_plan_stats",
    "dq_group_plan_stats_dev_u", "dq_group_plan_sorted", "dq_bitrate_hist_ints", "dq_norm_histogram", "dq_bitrate_search",
    "dq_scaling_compress_rows", "dq_scaling_dec_comp_rows", "dq_scaling_decompress_rows",
    "dq_mixed_required_bytes", "dq_mixed_compress", "dq_mixed_decompress", "dq_superchunk_stats",
    "dq_dynamic_bitrate_bucket", "dq_streams_overlap", "dq_stream_order_after", "dq_tile_io_floor",
    "dq_superchunk_mean_center", "dq_superchunk_add_mean_copy",
    "dq_hadamard", "dq_rht_blocked", "dq_rand_diag", "dq_rand_diag_bits", "dq_rht_scaling_compress", "dq_rht_scaling_compress_mfma16", "dq_scaling_decompress_irht", "dq_pack_signs",
    "dq_bins_to_bits", "dq_bits_to_bins", "dq_quantization",
    "dq_eden_work_doubles", "dq_eden_quantize", "dq_eden_quantize_static_max_n", "dq_eden_quantize_static", "dq_eden_dequantize", "dq_eden_dequantize_irht", "dq_thc_quantize", "dq_thc_dequantize", "dq_thc_rht_quantize", "dq_thc_dequantize_irht",
]

STAGE_STATS, STAGE_PLAN, STAGE_COMPRESS, STAGE_DECOMPRESS = 1, 2, 4, 8
STAGE_ALL = 15


class Bucket(ctypes.Structure):
    """dq_bucket_t of include/dynamiq_eden.h"""
    _fields_ = [
        ("src", ctypes.c_void_p), ("n", ctypes.c_int64), ("dtype", ctypes.c_int32), ("strategy", ctypes.c_int32),
        ("center_world", ctypes.c_int32), ("ring_chunk", ctypes.c_int32), ("ring_world", ctypes.c_int32),
        ("reserved", ctypes.c_int32), ("u", ctypes.c_double), ("u_dev", ctypes.c_void_p), ("stats", ctypes.c_void_p),
        ("mean", ctypes.c_void_p), ("reduced_stats", ctypes.c_void_p), ("order", ctypes.c_void_p),
        ("work", ctypes.c_void_p), ("work_ints", ctypes.c_int64), ("recv", ctypes.c_void_p), ("packed", ctypes.c_void_p),
        ("packed_bytes", ctypes.c_int64), ("out", ctypes.c_void_p), ("hist", ctypes.c_void_p),
        ("hist_ints", ctypes.c_int64), ("seed", ctypes.c_uint64), ("step", ctypes.c_uint64), ("step_dev", ctypes.c_void_p),
    ]


_lib = None


def lib():
    """The loaded shared library (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m dynamiq_sigcomm_artifact_amd.build`" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        c = ctypes
        vp, i64, i32, f32, u64 = c.c_void_p, c.c_int64, c.c_int, c.c_float, c.c_uint64
        L.dq_status_string.restype = c.c_char_p
        L.dq_status_string.argtypes = [i32]
        L.dq_last_error.restype = c.c_char_p
        L.dq_last_error.argtypes = []
        L.dq_version.restype = c.c_char_p
        L.dq_version.argtypes = []
        L.dq_scaling_required_bytes.restype = i64
        L.dq_scaling_required_bytes.argtypes = [i64, i32, i32, i32]
        L.dq_scaling_check_common.restype = i32
        L.dq_scaling_check_common.argtypes = [i64, i32, i32, i32, i32]
        L.dq_init_lookup_table.restype = i32
        L.dq_init_lookup_table.argtypes = []
        L.dq_mee_lookup_table.restype = i32
        L.dq_mee_lookup_table.argtypes = [i32, vp, vp]
        L.dq_scaling_compress.restype = i32
        L.dq_scaling_compress.argtypes = [vp, vp, vp, i64, i32, i32, i32, i32, i32, vp]
        L.dq_scaling_decompress.restype = i32
        L.dq_scaling_decompress.argtypes = [vp, vp, i64, i32, i32, i32, i32, i32, vp, i32]
        L.dq_scaling_dec_comp.restype = i32
        L.dq_scaling_dec_comp.argtypes = [vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp]
        L.dq_scaling_compress_philox.restype = i32
        L.dq_scaling_compress_philox.argtypes = [vp, vp, i64, i32, i32, i32, i32, i32, u64, u64, vp]
        L.dq_scaling_dec_comp_philox.restype = i32
        L.dq_scaling_dec_comp_philox.argtypes = [vp, vp, vp, i64, i32, i32, i32, i32, i32, u64, u64, vp]
        L.dq_philox_uniform.restype = i32
        L.dq_philox_uniform.argtypes = [vp, i64, i32, i32, u64, u64, vp]
        L.dq_group_plan_work_ints.restype = i64
        L.dq_group_plan_work_ints.argtypes = [i64]
        L.dq_group_plan_sorted_work_ints.restype = i64
        L.dq_group_plan_sorted_work_ints.argtypes = [i64]
        L.dq_group_plan.restype = i32
        L.dq_group_plan.argtypes = [vp, i64, vp, vp, i64, i32, vp]
        L.dq_group_plan_stats.restype = i32
        L.dq_group_plan_stats.argtypes = [vp, c.c_double, i64, vp, vp, vp, i64, i32, vp]
        L.dq_group_plan_sorted.restype = i32
        L.dq_group_plan_sorted.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, i32, vp]
        L.dq_group_plan_stats_dev_u.restype = i32
        L.dq_group_plan_stats_dev_u.argtypes = [vp, vp, i64, vp, vp, vp, i64, vp, i64, i32, vp]
        L.dq_bitrate_hist_ints.restype = i64
        L.dq_bitrate_hist_ints.argtypes = []
        L.dq_norm_histogram.restype = i32
        L.dq_norm_histogram.argtypes = [vp, i64, vp, i64, i32, vp]
        L.dq_bitrate_search.restype = i32
        L.dq_bitrate_search.argtypes = [vp, i64, i32, c.c_double, vp, c.c_double, vp, i32, vp]
        L.dq_scaling_compress_rows.restype = i32
        L.dq_scaling_compress_rows.argtypes = [vp, vp, vp, vp, i64, i32, i32, i32, i32, vp]
        L.dq_scaling_dec_comp_rows.restype = i32
        L.dq_scaling_dec_comp_rows.argtypes = [vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, vp]
        L.dq_scaling_decompress_rows.restype = i32
        L.dq_scaling_decompress_rows.argtypes = [vp, vp, vp, vp, i64, i64, i32, i32, i32, i32, vp, i32]
        L.dq_mixed_required_bytes.restype = i64
        L.dq_mixed_required_bytes.argtypes = [i64, i32]
        L.dq_mixed_compress.restype = i32
        L.dq_mixed_compress.argtypes = [vp, vp, i32, i64, vp, vp, i32, i32, vp, vp, vp, u64, u64, i64, i32, i32, i32, vp]
        L.dq_mixed_decompress.restype = i32
        L.dq_mixed_decompress.argtypes = [vp, vp, vp, vp, i32, i32, vp, i64, i64, i32, i32, i32, vp]
        L.dq_superchunk_stats.restype = i32
        L.dq_superchunk_stats.argtypes = [vp, vp, vp, i64, i32, i32, i32, vp]
        L.dq_dynamic_bitrate_bucket.restype = i32
        L.dq_dynamic_bitrate_bucket.argtypes = [c.POINTER(Bucket), i32, i32, vp]
        L.dq_tile_io_floor.restype = i32
        L.dq_tile_io_floor.argtypes = [i32, vp, i32, vp, i32, vp, i32, i64, i32, vp]
        L.dq_stream_order_after.restype = i32
        L.dq_stream_order_after.argtypes = [vp, vp, i32]
        L.dq_streams_overlap.restype = i32
        L.dq_streams_overlap.argtypes = [vp, vp, i32, c.POINTER(c.c_int)]
        L.dq_superchunk_mean_center.restype = i32
        L.dq_superchunk_mean_center.argtypes = [vp, vp, vp, i64, i32, i32, i32, i32, vp]
        L.dq_superchunk_add_mean_copy.restype = i32
        L.dq_superchunk_add_mean_copy.argtypes = [vp, vp, vp, i64, i32, i32, i32, vp]
        L.dq_hadamard.restype = i32
        L.dq_hadamard.argtypes = [vp, i64, i32, vp, i32]
        L.dq_rht_blocked.restype = i32
        L.dq_rht_blocked.argtypes = [vp, vp, i32, i64, i64, f32, i32, i32, vp]
        L.dq_rht_scaling_compress.restype = i32
        L.dq_rht_scaling_compress.argtypes = [vp, vp, i32, vp, vp, i32, i64, i64, f32, i32, i32, i32, u64, u64, vp]
        L.dq_rht_scaling_compress_mfma16.restype = i32
        L.dq_rht_scaling_compress_mfma16.argtypes = [vp, vp, i32, vp, i64, i64, f32, i32, u64, u64, vp]
        L.dq_scaling_decompress_irht.restype = i32
        L.dq_scaling_decompress_irht.argtypes = [vp, vp, i32, vp, i64, i64, f32, i32, i32, i32, vp]
        L.dq_pack_signs.restype = i32
        L.dq_pack_signs.argtypes = [vp, vp, i64, i32, vp]
        L.dq_rand_diag.restype = i32
        L.dq_rand_diag.argtypes = [vp, i64, i64, i32, vp]
        L.dq_rand_diag_bits.restype = i32
        L.dq_rand_diag_bits.argtypes = [vp, i64, i64, i32, vp]
        L.dq_bins_to_bits.restype = i32
        L.dq_bins_to_bits.argtypes = [vp, i64, vp, i64, i32, i32, vp]
        L.dq_bits_to_bins.restype = i32
        L.dq_bits_to_bins.argtypes = [vp, i64, vp, i64, i32, i32, vp]
        L.dq_eden_work_doubles.restype = i64
        L.dq_eden_work_doubles.argtypes = [i64]
        L.dq_eden_quantize.restype = i32
        L.dq_eden_quantize.argtypes = [vp, i64, vp, vp, i32, vp, vp, vp, i64, i32, vp]
        L.dq_eden_quantize_static_max_n.restype = i64
        L.dq_eden_quantize_static_max_n.argtypes = []
        L.dq_eden_quantize_static.restype = i32
        L.dq_eden_quantize_static.argtypes = [vp, i64, vp, vp, i32, vp, vp, i32, vp]
        L.dq_eden_dequantize.restype = i32
        L.dq_eden_dequantize.argtypes = [vp, i64, vp, i32, vp, i32, vp]
        L.dq_thc_quantize.restype = i32
        L.dq_thc_quantize.argtypes = [vp, vp, vp, i64, vp, vp, i32, i32, vp]
        L.dq_thc_dequantize.restype = i32
        L.dq_thc_dequantize.argtypes = [vp, vp, i64, vp, vp, i32, vp]
        L.dq_eden_dequantize_irht.restype = i32
        L.dq_eden_dequantize_irht.argtypes = [vp, i64, vp, i32, vp, i32, vp, i64, f32, vp, i32, vp]
        L.dq_thc_rht_quantize.restype = i32
        L.dq_thc_rht_quantize.argtypes = [vp, vp, i32, vp, vp, i64, i64, f32, vp, vp, i32, i32, vp]
        L.dq_thc_dequantize_irht.restype = i32
        L.dq_thc_dequantize_irht.argtypes = [vp, vp, i32, vp, i64, i64, f32, vp, vp, i32, vp]
        L.dq_quantization.restype = i32
        L.dq_quantization.argtypes = [vp, i64, i32, f32, f32, u64, vp]
        _lib = L
    return _lib


def dtype_code(t):
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.bfloat16:
        return BF16
    if t.dtype == torch.float32:
        return F32
    raise RuntimeError("unsupported element dtype %s" % t.dtype)


def _pair_code(elem, rand_pool):
    """dtype argument for the compress-side calls: fp32 gradients may come with a bf16 rand_pool."""
    code = dtype_code(elem)
    if rand_pool.dtype != elem.dtype:
        if code == F32 and rand_pool.dtype == torch.bfloat16:
            return code | RAND_BF16
        raise RuntimeError("rand_pool dtype must match input dtype")
    return code


def _check(rc):
    if rc != 0:
        raise RuntimeError(lib().dq_last_error().decode())


# The kernels dereference whatever address they are given: a host pointer, a strided view or a buffer of another
# GPU is a memory fault on the device, not an error code.  Every tensor whose address goes into the library passes
# through _p / _ptr / _dev, which refuse anything but contiguous device tensors and note the device; _call refuses a
# mix of devices before the library is entered.
_seen = threading.local()


def _refuse(t):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError("a tensor argument is required, got %s" % type(t).__name__)
    if not t.is_cuda:
        raise RuntimeError("tensor arguments must live on the GPU (got a %s tensor)" % t.device.type)
    raise RuntimeError("tensor arguments must be contiguous")


def _p(t):
    try:
        ok = t.is_cuda and t.is_contiguous()
    except AttributeError:
        ok = False
    if not ok:
        _refuse(t)
    try:
        _seen.devices.append(t.device.index)
    except AttributeError:
        _seen.devices = [t.device.index]
    return t.data_ptr()


def _ptr(t):
    return 0 if t is None else _p(t)


def _dev(t):
    _p(t)
    return t.device.index


def _call(fn, *args):
    devices = getattr(_seen, "devices", None)
    if devices:
        first = devices[0]
        mixed = any(d != first for d in devices)
        del devices[:]
        if mixed:
            raise RuntimeError("tensor arguments live on different devices")
    _check(fn(*args))


def _stream(stream):
    """a raw stream handle (int), a torch.cuda.Stream, or None for torch's current stream"""
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    elif hasattr(stream, "cuda_stream"):
        stream = stream.cuda_stream
    return ctypes.c_void_p(int(stream))


def torch_stream(stream, device=None):
    """the torch.cuda.Stream object for what the wrappers accept as `stream` (None, a raw handle, a torch stream), so
    that torch ops, waits and read-backs can be put on the stream the kernels run on"""
    if stream is None:
        return torch.cuda.current_stream(device)
    if hasattr(stream, "cuda_stream"):
        return stream
    if int(stream) == 0:
        return torch.cuda.default_stream(device)
    return torch.cuda.ExternalStream(int(stream), device=device)


def required_bytes(n, nbits, chunk_size, strategy):
    return int(lib().dq_scaling_required_bytes(n, nbits, chunk_size, strategy))


def check_common(n, nbits, chunk_size, strategy, strict=True):
    _call(lib().dq_scaling_check_common, n, nbits, chunk_size, strategy, 1 if strict else 0)


def mee_lookup_table(nbits):
    import numpy as np
    table = np.zeros(256, np.uint16)
    params = np.zeros(4, np.uint16)
    _call(lib().dq_mee_lookup_table, nbits, table.ctypes.data_as(ctypes.c_void_p), params.ctypes.data_as(ctypes.c_void_p))
    return table, params


def scaling_compress(src, dst, rand_pool, n, nbits, chunk_size, strategy, stream=None):
    _call(lib().dq_scaling_compress, _p(src), _p(dst), _p(rand_pool), n, nbits, chunk_size,
                                     _pair_code(src, rand_pool), _dev(src), strategy, _stream(stream))


def scaling_decompress(src, dst, n, nbits, chunk_size, strategy, add=False, stream=None):
    _call(lib().dq_scaling_decompress, _p(src), _p(dst), n, nbits, chunk_size, dtype_code(dst), _dev(dst),
                                       strategy, _stream(stream), 1 if add else 0)


def scaling_dec_comp(recv, inp, send, rand_pool, n, nbits, chunk_size, strategy, stream=None):
    _call(lib().dq_scaling_dec_comp, _p(recv), _p(inp), _p(send), _p(rand_pool), n, nbits,
                                     chunk_size, _pair_code(inp, rand_pool), _dev(inp), strategy, _stream(stream))


def group_plan_work_ints(nsc):
    return int(lib().dq_group_plan_work_ints(nsc))


def group_plan(qbits, order, work, stream=None):
    """qbits int64 [nsc] -> order int32 [3 * nsc]: the 8-bit rows from entry 0, the 4-bit rows from nsc, the 2-bit rows
    from 2 * nsc (group_rows() slices them); work[0:3] = counts"""
    if qbits.dtype != torch.int64 or order.dtype != torch.int32 or work.dtype != torch.int32:
        raise RuntimeError("group_plan: qbits must be int64, order and work int32")
    if order.numel() < 3 * qbits.numel():
        raise RuntimeError("group_plan: order has fewer than 3 * nsc entries")
    _call(lib().dq_group_plan, _p(qbits), qbits.numel(), _p(order), _p(work), work.numel(),
                               _dev(qbits), _stream(stream))


def group_rows(order, nsc, width, count):
    """the row list of one width in a planned `order` (a view)"""
    base = {8: 0, 4: 1, 2: 2}[width] * nsc
    return order[base:base + count]


def group_plan_sorted_work_ints(nsc):
    """int32 entries of the work buffer of group_plan_sorted: 4 up to 65535 superchunks, the radix sort's buffers beyond"""
    return int(lib().dq_group_plan_sorted_work_ints(nsc))


def group_plan_sorted(stats, top_count, bottom_count, order, work, stream=None, qbits_out=None):
    """fixed-proportion groups (comm_hooks.py:710-721): order / work[0:3] as group_plan writes them, every list in
    the order of the stable descending sort of the norms stats[:, 1]; work: group_plan_sorted_work_ints(nsc) ints"""
    if stats.dtype != torch.bfloat16 or order.dtype != torch.int32 or work.dtype != torch.int32:
        raise RuntimeError("group_plan_sorted: stats must be bfloat16, order and work int32")
    nsc = stats.numel() // 2
    if order.numel() < 3 * nsc or (qbits_out is not None and (qbits_out.dtype != torch.int64 or qbits_out.numel() < nsc)):
        raise RuntimeError("group_plan_sorted: order / qbits_out too small or of the wrong dtype")
    _call(lib().dq_group_plan_sorted, _p(stats), nsc, int(top_count), int(bottom_count), _ptr(qbits_out),
                                      _p(order), _p(work), work.numel(), _dev(stats), _stream(stream))


def group_plan_stats(stats, u, qbits_out, order, work, stream=None, hist=None):
    """stats bf16 [nsc, 2] (mean, reduced sum of squares), offset u (a number, or a float64 device tensor read when the
    kernels run) -> qbits_out (int64 or None), order, work; hist (int32 [bitrate_hist_ints()] or None) also gets the bucket's
    norm patterns -- within the same launch when u is a device tensor"""
    if stats.dtype != torch.bfloat16 or order.dtype != torch.int32 or work.dtype != torch.int32:
        raise RuntimeError("group_plan_stats: stats must be bfloat16, order and work int32")
    nsc = stats.numel() // 2
    if order.numel() < 3 * nsc or (qbits_out is not None and (qbits_out.dtype != torch.int64 or qbits_out.numel() < nsc)):
        raise RuntimeError("group_plan_stats: order / qbits_out too small or of the wrong dtype")
    if isinstance(u, torch.Tensor):
        # the offset stays on the device (one float64, e.g. the first entry of bitrate_search's result)
        if u.dtype != torch.float64 or u.numel() < 1 or u.device != stats.device:
            raise RuntimeError("group_plan_stats: a tensor u must be float64 on the device of stats")
        if hist is not None and hist.dtype != torch.int32:
            raise RuntimeError("group_plan_stats: hist must be int32")
        _call(lib().dq_group_plan_stats_dev_u, _p(stats), _p(u), nsc, _ptr(qbits_out), _p(order),
                                               _p(work), work.numel(), _ptr(hist), 0 if hist is None else hist.numel(),
                                               _dev(stats), _stream(stream))
        return
    if hist is not None:
        norm_histogram(stats, hist, stream)
    _call(lib().dq_group_plan_stats, _p(stats), float(u), nsc, _ptr(qbits_out), _p(order), _p(work),
                                     work.numel(), _dev(stats), _stream(stream))


def bitrate_hist_ints():
    return int(lib().dq_bitrate_hist_ints())


def norm_histogram(stats, hist, stream=None):
    """adds the norm patterns of stats (bf16 [nsc, 2]: mean, reduced sum of squares) to hist (int32 [bitrate_hist_ints()])"""
    if stats.dtype != torch.bfloat16 or hist.dtype != torch.int32:
        raise RuntimeError("norm_histogram: stats must be bfloat16 and hist int32")
    _call(lib().dq_norm_histogram, _p(stats), stats.numel() // 2, _p(hist), hist.numel(), _dev(stats),
                                   _stream(stream))


def bitrate_search(hist, mode, prev_u, target_avg_bits, result, stream=None):
    """mode 0: bisection, 1: correction from prev_u (a number or a float64 device tensor); result float64 [4] = u, average
    width, target - average, probes; hist comes back zeroed"""
    if hist.dtype != torch.int32 or result.dtype != torch.float64 or result.numel() < 4:
        raise RuntimeError("bitrate_search: hist must be int32 and result float64 [4]")
    prev_dev = None
    if isinstance(prev_u, torch.Tensor):        # the starting point stays on the device (it may be result itself)
        if prev_u.dtype != torch.float64 or prev_u.numel() < 1 or prev_u.device != hist.device:
            raise RuntimeError("bitrate_search: a tensor prev_u must be float64 on the device of hist")
        prev_dev, prev_u = prev_u, 0.0
    _call(lib().dq_bitrate_search, _p(hist), hist.numel(), int(mode), float(prev_u), _ptr(prev_dev),
                                   float(target_avg_bits), _p(result), _dev(hist), _stream(stream))


def scaling_compress_rows(src, rows, dst, rand_pool, nrows, nbits, strategy, stream=None):
    _call(lib().dq_scaling_compress_rows, _p(src), _ptr(rows), _p(dst), _p(rand_pool), nrows, nbits,
                                          _pair_code(src, rand_pool), _dev(src), strategy, _stream(stream))


def scaling_dec_comp_rows(recv, inp, rows, send, rand_pool, nrows, nbits, strategy, stream=None):
    _call(lib().dq_scaling_dec_comp_rows, _p(recv), _p(inp), _ptr(rows), _p(send),
                                          _p(rand_pool), nrows, nbits, _pair_code(inp, rand_pool), _dev(inp),
                                          strategy, _stream(stream))


def scaling_decompress_rows(src, dst, rows, stats, n_limit, nrows, nbits, strategy, add=False, stream=None):
    _call(lib().dq_scaling_decompress_rows, _p(src), _p(dst), _ptr(rows), _ptr(stats), n_limit, nrows,
                                            nbits, dtype_code(dst), _dev(dst), strategy, _stream(stream),
                                            1 if add else 0)


def mixed_required_bytes(nsc, ring_world=1):
    return int(lib().dq_mixed_required_bytes(nsc, ring_world))


def mixed_compress(src, order, counts, dst, nsc, strategy, rand_pool=None, seed=0, step=0, recv=None, center_mean=None,
                   center_world=1, n=0, ring_chunk=0, ring_world=1, stream=None):
    """all three bit-width groups of the plan (order, counts = work[0:3] of group_plan*) in one launch; recv makes it
    the ring's fused step; center_mean (float32 per superchunk, from superchunk_stats) centres src on load"""
    code = dtype_code(src) if rand_pool is None else _pair_code(src, rand_pool)
    _call(lib().dq_mixed_compress, _p(src), _ptr(center_mean), center_world, n, _p(order), _p(counts),
                                   ring_chunk, ring_world, _ptr(recv), _p(dst), _ptr(rand_pool), int(seed), int(step),
                                   nsc, code, _dev(src), strategy, _stream(stream))


def mixed_decompress(src, dst, order, counts, nsc, strategy, stats=None, n_limit=None, ring_chunk=0, ring_world=1,
                     stream=None):
    _call(lib().dq_mixed_decompress, _p(src), _p(dst), _p(order), _p(counts), ring_chunk,
                                     ring_world, _ptr(stats), nsc * 256 if n_limit is None else n_limit, nsc,
                                     dtype_code(dst), _dev(dst), strategy, _stream(stream))


def bucket_descriptor(src, n, stats, mean, order, work, packed, strategy=2, out=None, u=0.0, reduced_stats=None,
                      center_world=1, ring_chunk=0, ring_world=1, recv=None, hist=None, seed=0, step=0, step_dev=None):
    """A dq_bucket_t for dynamic_bitrate_bucket, filled from tensors (each checked: contiguous, on one GPU, of the dtype
    and size the stages need).  u: a number, or a float64 device tensor read when the plan runs.  The descriptor keeps
    addresses, not tensors: whoever holds it keeps the tensors alive.  Returns (descriptor, device index)."""
    nsc = (n + 255) // 256
    code = dtype_code(src)
    need = [(stats, torch.bfloat16, 2 * nsc, "stats"), (mean, torch.float32, nsc, "mean"), (order, torch.int32, 3 * nsc, "order"),
            (work, torch.int32, group_plan_work_ints(nsc), "work"),
            (packed, torch.uint8, mixed_required_bytes(nsc, ring_world), "packed")]
    if out is not None:
        need.append((out, src.dtype, n, "out"))
    if reduced_stats is not None:
        need.append((reduced_stats, torch.bfloat16, 2 * nsc, "reduced_stats"))
    if recv is not None:
        need.append((recv, torch.uint8, 0, "recv"))
    if hist is not None:
        need.append((hist, torch.int32, bitrate_hist_ints(), "hist"))
    if step_dev is not None:
        need.append((step_dev, torch.int64, 1, "step_dev"))
    if src.numel() < n:
        raise RuntimeError("bucket_descriptor: src has fewer than n elements")
    for t, dt, count, name in need:
        if t.dtype != dt or t.numel() < count:
            raise RuntimeError("bucket_descriptor: %s must be %s with at least %d entries" % (name, dt, count))
    b = Bucket()
    b.src, b.n, b.dtype, b.strategy = _p(src), n, code, strategy
    b.center_world, b.ring_chunk, b.ring_world = center_world, ring_chunk, ring_world
    if isinstance(u, torch.Tensor):
        if u.dtype != torch.float64 or u.numel() < 1:
            raise RuntimeError("bucket_descriptor: a tensor u must be float64")
        b.u, b.u_dev = 0.0, _p(u)
    else:
        b.u, b.u_dev = float(u), None
    b.stats, b.mean, b.reduced_stats = _p(stats), _p(mean), _ptr(reduced_stats) or None
    b.order, b.work, b.work_ints = _p(order), _p(work), work.numel()
    b.recv, b.packed, b.packed_bytes = _ptr(recv) or None, _p(packed), packed.numel()
    b.out = _ptr(out) or None
    b.hist, b.hist_ints = _ptr(hist) or None, 0 if hist is None else hist.numel()
    b.seed, b.step, b.step_dev = int(seed) & 0xFFFFFFFFFFFFFFFF, int(step) & 0xFFFFFFFFFFFFFFFF, _ptr(step_dev) or None
    devices = _seen.devices
    dev = devices[0]
    if any(d != dev for d in devices):
        del devices[:]
        raise RuntimeError("tensor arguments live on different devices")
    del devices[:]
    return b, dev


def dynamic_bitrate_bucket(desc, device, stages=STAGE_ALL, stream=None):
    """one host call for any run of the stages statistics -> plan -> mixed compress -> mixed decompress of one bucket
    (desc, device: from bucket_descriptor)"""
    _check(lib().dq_dynamic_bitrate_bucket(ctypes.byref(desc), stages, device, _stream(stream)))


def tile_io_floor(direction, a, b, run, run_bytes_per_tile, tiles, stream=None):
    """a launch with the shape and the memory accesses of the chunk-16 codec on `tiles` tiles of 1,024 elements and no
    arithmetic: direction 0 reads the element tensor a and the pool b (may be None) and writes `run_bytes_per_tile` bytes per
    tile to `run`; direction 1 reads `run` (and b) and overwrites a.  A measurement aid: what it writes has no meaning."""
    a_bytes = 1024 * a.element_size()
    b_bytes = 1024 * b.element_size() if b is not None else 0
    if a.numel() < 1024 * tiles or (b is not None and b.numel() < 1024 * tiles) or run.numel() * run.element_size() < run_bytes_per_tile * tiles:
        raise ValueError("a tensor is shorter than tiles * bytes per tile")
    _call(lib().dq_tile_io_floor, int(direction), _ptr(a), a_bytes, _ptr(b), b_bytes, _ptr(run), int(run_bytes_per_tile),
          int(tiles), a.device.index, _stream(stream))


def stream_order_after(stream, after, device):
    """`stream` waits for everything enqueued on `after` so far (raw handles or torch streams); an event from the library's
    own ring, nothing allocated per call"""
    _check(lib().dq_stream_order_after(_stream(stream), _stream(after), int(device)))


def streams_overlap(a, b, device):
    """True when kernels enqueued on the HIP streams a and b (raw handles) run side by side on `device`, False when the
    runtime has put the two on one hardware queue (they then take turns).  Synchronises with both: a set-up call."""
    res = ctypes.c_int(0)
    _check(lib().dq_streams_overlap(_stream(a), _stream(b), int(device), ctypes.byref(res)))
    return bool(res.value)


def superchunk_stats(src, stats, mean, n, world_size, stream=None):
    """the statistics of superchunk_mean_center without the residual; mean (float32 [nsc] or None) gets the unrounded means"""
    _call(lib().dq_superchunk_stats, _p(src), _p(stats), _ptr(mean), n, world_size, dtype_code(src), _dev(src),
                                     _stream(stream))


def scaling_compress_philox(src, dst, n, nbits, chunk_size, strategy, seed, step, stream=None):
    """scaling_compress with the uniform values drawn in the kernel (Philox keyed by seed, counter = chunk, step)"""
    _call(lib().dq_scaling_compress_philox, _p(src), _p(dst), n, nbits, chunk_size, dtype_code(src), _dev(src),
                                            strategy, int(seed), int(step), _stream(stream))


def scaling_dec_comp_philox(recv, inp, send, n, nbits, chunk_size, strategy, seed, step, stream=None):
    _call(lib().dq_scaling_dec_comp_philox, _p(recv), _p(inp), _p(send), n, nbits, chunk_size,
                                            dtype_code(inp), _dev(inp), strategy, int(seed), int(step), _stream(stream))


def philox_uniform(out, seed, step, stream=None):
    """the uniform values of that stream as a tensor (any of the three element types)"""
    _call(lib().dq_philox_uniform, _p(out), out.numel(), dtype_code(out), _dev(out), int(seed), int(step),
                                   _stream(stream))


def superchunk_mean_center(src, residual, stats, n, world_size, superchunk_size=256, stream=None):
    _call(lib().dq_superchunk_mean_center, _p(src), _p(residual), _p(stats), n, world_size,
                                           superchunk_size, dtype_code(src), _dev(src), _stream(stream))


def superchunk_add_mean_copy(residual, dst, stats, n, superchunk_size=256, stream=None):
    _call(lib().dq_superchunk_add_mean_copy, _p(residual), _p(dst), _p(stats), n, superchunk_size,
                                             dtype_code(residual), _dev(residual), _stream(stream))


def hadamard(vec, stream=None):
    _call(lib().dq_hadamard, _p(vec), vec.numel(), _dev(vec), _stream(stream), 0)


def rht_blocked(vec, sign, block, scale, inverse=False, stream=None):
    """sign: None, float32 +-1 values, or the int32 bit vector of pack_signs"""
    _check_sign(sign, vec.numel(), "rht_blocked")
    _call(lib().dq_rht_blocked, _p(vec), _ptr(sign), _packed(sign), vec.numel(), block, float(scale),
                                1 if inverse else 0, _dev(vec), _stream(stream))


def _packed(sign):
    return 1 if sign is not None and sign.dtype == torch.int32 else 0


def _check_sign(sign, n, what):
    """None, n float32 values or ceil(n / 32) int32 words"""
    if sign is None:
        return
    if sign.dtype == torch.int32:
        if sign.numel() < (n + 31) // 32:
            raise RuntimeError(what + ": the packed sign vector is too short")
    elif sign.dtype != torch.float32 or sign.numel() < n:
        raise RuntimeError(what + ": sign must be float32 [n] or the int32 bit vector of pack_signs")


def pack_signs(sign, stream=None):
    """float32 +-1 vector -> int32 [ceil(n / 32)], bit e % 32 of word e / 32 set where sign[e] < 0"""
    bits = torch.empty((sign.numel() + 31) // 32, dtype=torch.int32, device=sign.device)
    _call(lib().dq_pack_signs, _p(sign), _p(bits), sign.numel(), _dev(sign), _stream(stream))
    return bits


def rht_scaling_compress(src, sign, dst, block, scale, nbits, strategy, rand_pool=None, seed=0, step=0, stream=None):
    """rht_blocked (forward) + scaling_compress of the rotated fp32 vector in one launch; src is not modified.
    sign: None, float32 +-1 values, or the int32 bit vector of pack_signs.
    rand_pool: float32 or bfloat16 [n], or None for the in-kernel rounding stream keyed by (seed, step, chunk)"""
    if src.dtype != torch.float32:
        raise RuntimeError("rht_scaling_compress: src must be float32")
    code = 0
    if rand_pool is not None:
        code = dtype_code(rand_pool)
    _call(lib().dq_rht_scaling_compress, _p(src), _ptr(sign), _packed(sign), _p(dst), _ptr(rand_pool), code, src.numel(),
                                         block, float(scale), nbits, _dev(src), strategy, int(seed), int(step),
                                         _stream(stream))


def rht_scaling_compress_mfma16(src, sign, dst, block, scale, seed=0, step=0, stream=None):
    """measurement variant of rht_scaling_compress (4-bit AEE, in-kernel rounding stream): the first four stages of the
    transform on the matrix cores; agrees with the default to rounding error only"""
    if src.dtype != torch.float32:
        raise RuntimeError("rht_scaling_compress_mfma16: src must be float32")
    _check_sign(sign, src.numel(), "rht_scaling_compress_mfma16")
    _call(lib().dq_rht_scaling_compress_mfma16, _p(src), _ptr(sign), _packed(sign), _p(dst), src.numel(), block, float(scale),
          _dev(src), int(seed), int(step), _stream(stream))


def scaling_decompress_irht(src, sign, dst, block, scale, nbits, strategy, stream=None):
    """scaling_decompress into float32 + rht_blocked (inverse) in one launch"""
    if dst.dtype != torch.float32:
        raise RuntimeError("scaling_decompress_irht: dst must be float32")
    _call(lib().dq_scaling_decompress_irht, _p(src), _ptr(sign), _packed(sign), _p(dst), dst.numel(), block, float(scale),
                                            nbits, _dev(dst), strategy, _stream(stream))


def rand_diag(out, seed, stream=None):
    _call(lib().dq_rand_diag, _p(out), out.numel(), seed, _dev(out), _stream(stream))


def rand_diag_bits(bits, size, seed, stream=None):
    """the diagonal of rand_diag(size, seed) as the int32 bit vector of pack_signs; size a multiple of 256"""
    if bits.dtype != torch.int32 or bits.numel() < size // 32:
        raise RuntimeError("rand_diag_bits: bits must be int32 [size / 32]")
    _call(lib().dq_rand_diag_bits, _p(bits), size, seed, _dev(bits), _stream(stream))


def bins_to_bits(bins, arr, nbits, stream=None):
    _call(lib().dq_bins_to_bits, _p(bins), bins.numel(), _p(arr), arr.numel(), nbits, _dev(bins), _stream(stream))


def bits_to_bins(bins, arr, nbits, stream=None):
    _call(lib().dq_bits_to_bins, _p(bins), bins.numel(), _p(arr), arr.numel(), nbits, _dev(bins), _stream(stream))


def quantization(vec, div_factor, tensor_max, seed, stream=None):
    _call(lib().dq_quantization, _p(vec), vec.numel(), _dev(vec), float(div_factor), float(tensor_max), int(seed),
                                 _stream(stream))


def eden_work_doubles(n):
    return int(lib().dq_eden_work_doubles(n))


def eden_quantize(vec, boundaries, centroids, nbits, packed, result, work, stream=None):
    """vec float32 [n] -> packed int32/uint32 [n / 32 * nbits], result float32 [4] = (sumsq, dot, scale, norm)"""
    for t, name in ((vec, "vec"), (boundaries, "boundaries"), (centroids, "centroids"), (result, "result")):
        if t.dtype != torch.float32:
            raise RuntimeError("eden_quantize: %s must be float32" % name)
    if packed.dtype != torch.int32 or work.dtype != torch.float64:
        raise RuntimeError("eden_quantize: packed must be int32 and work float64")
    n = vec.numel()
    if boundaries.numel() < (1 << nbits) - 1 or centroids.numel() < (1 << nbits) or result.numel() < 4 \
            or packed.numel() < n // 32 * nbits:
        raise RuntimeError("eden_quantize: a buffer is too small")
    _call(lib().dq_eden_quantize, _p(vec), n, _p(boundaries), _p(centroids), nbits, _p(packed),
                                  _p(result), _p(work), work.numel(), _dev(vec), _stream(stream))


def eden_quantize_static(vec, boundaries, centroids, nbits, packed, result, stream=None, n=None):
    """eden_quantize with the partial sums in the library's static device array: nothing is allocated.
    Calls that overlap on one GPU race on that array."""
    for t, name in ((vec, "vec"), (boundaries, "boundaries"), (centroids, "centroids"), (result, "result")):
        if t.dtype != torch.float32:
            raise RuntimeError("eden_quantize_static: %s must be float32" % name)
    if packed.dtype != torch.int32:
        raise RuntimeError("eden_quantize_static: packed must be int32")
    n = vec.numel() if n is None else int(n)
    if boundaries.numel() < (1 << nbits) - 1 or centroids.numel() < (1 << nbits) or result.numel() < 4 \
            or packed.numel() < n // 32 * nbits or vec.numel() < n:
        raise RuntimeError("eden_quantize_static: a buffer is too small")
    _call(lib().dq_eden_quantize_static, _p(vec), n, _p(boundaries), _p(centroids), nbits,
                                         _p(packed), _p(result), _dev(vec), _stream(stream))


def eden_dequantize(packed, n, centroids, nbits, out, stream=None):
    if packed.dtype != torch.int32 or centroids.dtype != torch.float32 or out.dtype != torch.float32:
        raise RuntimeError("eden_dequantize: packed must be int32, centroids and out float32")
    if packed.numel() < n // 32 * nbits or out.numel() < n or centroids.numel() < (1 << nbits):
        raise RuntimeError("eden_dequantize: a buffer is too small")
    _call(lib().dq_eden_dequantize, _p(packed), n, _p(centroids), nbits, _p(out), _dev(out),
                                    _stream(stream))


def thc_quantize(rotated, uniform, levels_out, lo, delta, levels, stream=None):
    if rotated.dtype != torch.float32 or uniform.dtype != torch.float32 or levels_out.dtype != torch.bfloat16 \
            or lo.dtype != torch.float32 or delta.dtype != torch.float32:
        raise RuntimeError("thc_quantize: rotated, uniform, lo, delta must be float32 and the output bfloat16")
    n = rotated.numel()
    if uniform.numel() < n or levels_out.numel() < n:
        raise RuntimeError("thc_quantize: a buffer is too small")
    _call(lib().dq_thc_quantize, _p(rotated), _p(uniform), _p(levels_out), n, _p(lo),
                                 _p(delta), levels, _dev(rotated), _stream(stream))


def thc_dequantize(levels_in, out, step, lo, stream=None):
    if levels_in.dtype != torch.bfloat16 or out.dtype != torch.float32 or step.dtype != torch.float32 \
            or lo.dtype != torch.float32:
        raise RuntimeError("thc_dequantize: levels must be bfloat16, out, step, lo float32")
    n = levels_in.numel()
    if out.numel() < n:
        raise RuntimeError("thc_dequantize: out is too small")
    _call(lib().dq_thc_dequantize, _p(levels_in), _p(out), n, _p(step), _p(lo), _dev(out),
                                   _stream(stream))


def eden_dequantize_irht(packed, n, centroids, nbits, sign, out, block, scale, post_scale=None, stream=None):
    """eden_dequantize + rht_blocked (inverse) in the transform's own passes; post_scale: a float32 device scalar that
    multiplies the result (EDEN's scale), or None"""
    if packed.dtype != torch.int32 or centroids.dtype != torch.float32 or out.dtype != torch.float32:
        raise RuntimeError("eden_dequantize_irht: packed must be int32, centroids and out float32")
    if packed.numel() < n // 32 * nbits or centroids.numel() < (1 << nbits) or out.numel() < n:
        raise RuntimeError("eden_dequantize_irht: a buffer is too small")
    if post_scale is not None and (post_scale.dtype != torch.float32 or post_scale.device != out.device):
        raise RuntimeError("eden_dequantize_irht: post_scale must be a float32 tensor on the device of out")
    _check_sign(sign, n, "eden_dequantize_irht")
    _call(lib().dq_eden_dequantize_irht, _p(packed), n, _p(centroids), nbits, _ptr(sign), _packed(sign),
                                         _p(out), block, float(scale), _ptr(post_scale), _dev(out), _stream(stream))


def thc_rht_quantize(work, sign, uniform, levels_out, block, scale, lo, delta, levels, stream=None):
    """rht_blocked (forward) + thc_quantize in the transform's own passes; `work` holds the vector on entry and
    intermediate values on return"""
    if work.dtype != torch.float32 or uniform.dtype != torch.float32 or levels_out.dtype != torch.bfloat16 \
            or lo.dtype != torch.float32 or delta.dtype != torch.float32:
        raise RuntimeError("thc_rht_quantize: work, uniform, lo, delta must be float32 and the output bfloat16")
    n = work.numel()
    if uniform.numel() < n or levels_out.numel() < n:
        raise RuntimeError("thc_rht_quantize: a buffer is too small")
    _check_sign(sign, n, "thc_rht_quantize")
    _call(lib().dq_thc_rht_quantize, _p(work), _ptr(sign), _packed(sign), _p(uniform), _p(levels_out), n, block,
                                     float(scale), _p(lo), _p(delta), levels, _dev(work), _stream(stream))


def thc_dequantize_irht(levels_in, sign, out, block, scale, step, lo, stream=None):
    """thc_dequantize + rht_blocked (inverse) in the transform's own passes"""
    if levels_in.dtype != torch.bfloat16 or out.dtype != torch.float32 or step.dtype != torch.float32 \
            or lo.dtype != torch.float32:
        raise RuntimeError("thc_dequantize_irht: levels must be bfloat16, out, step, lo float32")
    n = out.numel()
    if levels_in.numel() < n:
        raise RuntimeError("thc_dequantize_irht: a buffer is too small")
    _check_sign(sign, n, "thc_dequantize_irht")
    _call(lib().dq_thc_dequantize_irht, _p(levels_in), _ptr(sign), _packed(sign), _p(out), n, block, float(scale),
                                        _p(step), _p(lo), _dev(out), _stream(stream))
