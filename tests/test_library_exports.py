"""The C-ABI library loads and exports every symbol include/dynamiq_eden.h declares;
the host-only entry points (sizes, validation, lookup table) behave like the reference."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "dynamiq_eden.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    from dynamiq_sigcomm_artifact_amd import capi
    L = ctypes.CDLL(capi.LIB_PATH)
    names = _declared()
    assert len(names) >= 18
    for name in names:
        assert hasattr(L, name), name
    assert sorted(capi.EXPORTS) == names


def test_host_side_entry_points(oracle):
    from dynamiq_sigcomm_artifact_amd import capi
    L = capi.lib()
    assert L.dq_version().decode().startswith("dynamiq_eden")
    for n, b, c, s in ((6553600, 4, 16, 2), (304, 8, 16, 0), (1024, 2, 32, 3), (124439808, 5, 16, 2)):
        assert capi.required_bytes(n, b, c, s) == oracle.required_bytes(n, b, c, s)
    cases = [(0, 4, 16, 0), (256, 3, 16, 0), (256, 4, 16, 4), (256, 4, 64, 0), (256, 4, 12, 0),
             (256, 2, 2, 0), (250, 4, 16, 0), (272, 4, 16, 2), (256, 4, 16, 2)]
    for args in cases:
        want = oracle.scaling_check(*args, strict=True)
        got = L.dq_scaling_check_common(*args, 1)
        assert got == want, args
        if want:
            assert L.dq_last_error().decode() == oracle.ERRORS[want]
            with pytest.raises(RuntimeError, match=re.escape(oracle.ERRORS[want])):
                capi.check_common(*args)
    assert L.dq_scaling_check_common(256, 5, 16, 2, 0) == 0 and L.dq_scaling_check_common(256, 5, 16, 2, 1) == 2
    for nbits in range(1, 9):
        t, p = capi.mee_lookup_table(nbits)
        to, po = oracle.mee_lut(nbits)
        assert (t == to).all() and (p == po).all()


def test_module_imports_without_gpu():
    import dynamiq_sigcomm_artifact_amd as pkg
    eu = pkg.load_eden_utils()
    reference_names = [
        "Hadamard", "EdenBinsToBits", "EdenBitsToBins", "Hadamard_init", "Hadamard_init_ptr", "Hadamard_inplace",
        "Hadamard_inplace_ptr", "quantization_compression", "scaling_compress", "scaling_decompress",
        "scaling_decompress_add", "scaling_dec_comp", "superchunk_mean_center", "superchunk_add_mean_copy",
        "init_lookup_table"]                                       # eden_utils.cpp:417-433
    for name in reference_names:
        assert callable(getattr(eu, name)), name
    import torch
    x = torch.zeros(256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        eu.scaling_compress(x, torch.zeros(146, dtype=torch.uint8), x, 256, 4, 16, 0, 2)
    with pytest.raises(RuntimeError, match="src must be a CUDA tensor"):
        eu.superchunk_mean_center(x, x, x, 256, 1)
    eu.init_lookup_table()


def test_argument_errors_are_reported_before_any_device_work():
    """every entry point rejects bad arguments with a status code and a message for the calling thread; these calls
    return before the first HIP call, so they run without a GPU (the pointers are never dereferenced)"""
    from dynamiq_sigcomm_artifact_amd import capi
    L = capi.lib()
    P = ctypes.c_void_p(0x1000)          # non-null placeholder
    N = ctypes.c_void_p(0)
    S = ctypes.c_void_p(0)               # stream

    def err(rc, text):
        assert rc != 0
        assert text in L.dq_last_error().decode(), (L.dq_last_error().decode(), text)

    Z = ctypes.c_uint64(0)
    err(L.dq_scaling_compress(P, P, P, 0, 4, 16, 1, 0, 2, S), "n must be positive")
    err(L.dq_scaling_compress(P, P, P, 256, 9, 16, 1, 0, 2, S), "nbits")
    err(L.dq_scaling_compress(P, P, P, 256, 4, 16, 7, 0, 2, S), "unsupported element dtype")
    err(L.dq_scaling_compress(P, P, P, 256, 4, 16, 1 | 0x10, 0, 2, S), "unsupported element dtype")   # bf16 pool flag needs f32
    err(L.dq_scaling_compress(N, P, P, 256, 4, 16, 1, 0, 2, S), "null pointer")
    err(L.dq_scaling_decompress(P, N, 256, 4, 16, 1, 0, 2, S, 0), "null pointer")
    err(L.dq_scaling_decompress(P, P, 250, 4, 16, 1, 0, 0, S, 0), "multiple of chunk_size")
    err(L.dq_scaling_dec_comp(P, P, P, P, 272, 4, 16, 1, 0, 3, S), "whole number of 16-chunk superchunks")
    err(L.dq_scaling_compress_philox(P, P, 512, 4, 32, 1, 0, 2, 1, 1, S), "chunk_size 16")
    err(L.dq_scaling_dec_comp_philox(P, P, N, 256, 4, 16, 1, 0, 2, 1, 1, S), "null pointer")
    err(L.dq_philox_uniform(P, 0, 1, 0, 1, 1, S), "n must be positive")
    err(L.dq_superchunk_mean_center(P, P, P, 256, 0, 256, 1, 0, S), "world_size must be positive")
    err(L.dq_superchunk_mean_center(P, P, P, 256, 2, 128, 1, 0, S), "superchunk_size must be 256")
    err(L.dq_superchunk_add_mean_copy(P, P, N, 256, 256, 1, 0, S), "null pointer")
    err(L.dq_hadamard(P, 1000, 0, S, 0), "power of 2")
    err(L.dq_rht_blocked(P, P, 0, 1024, 48, ctypes.c_float(1.0), 0, 0, S), "block")
    err(L.dq_rht_blocked(P, P, 1, 1000, 64, ctypes.c_float(1.0), 0, 0, S), "multiple of block")
    err(L.dq_rand_diag(P, 0, 1, 0, S), "n must be positive")
    F1 = ctypes.c_float(1.0)
    err(L.dq_rht_scaling_compress(P, P, 0, P, P, 2, 1024, 48, F1, 4, 0, 2, Z, Z, S), "power of 2")
    err(L.dq_rht_scaling_compress(P, P, 0, P, P, 2, 1 << 17, 1 << 16, F1, 4, 0, 2, Z, Z, S), "32768")
    err(L.dq_rht_scaling_compress(P, P, 0, P, P, 2, 1000, 8, F1, 4, 0, 2, Z, Z, S), "superchunk")          # n % 256
    err(L.dq_rht_scaling_compress(P, P, 0, P, P, 2, 1024, 64, F1, 9, 0, 2, Z, Z, S), "nbits")
    err(L.dq_rht_scaling_compress(P, P, 0, P, P, 2, 1024, 64, F1, 4, 0, 1, Z, Z, S), "strategy")
    err(L.dq_rht_scaling_compress(P, P, 0, P, P, 0, 1024, 64, F1, 4, 0, 2, Z, Z, S), "unsupported element dtype")   # binary16 pool
    err(L.dq_rht_scaling_compress(N, P, 0, P, P, 2, 1024, 64, F1, 4, 0, 2, Z, Z, S), "null pointer")
    err(L.dq_scaling_decompress_irht(P, P, 1, N, 1024, 64, F1, 4, 0, 2, S), "null pointer")
    err(L.dq_scaling_decompress_irht(P, P, 1, P, 1024, 96, F1, 4, 0, 2, S), "power of 2")
    err(L.dq_pack_signs(P, N, 100, 0, S), "null pointer")
    err(L.dq_streams_overlap(S, S, 0, None), "null pointer")
    err(L.dq_stream_order_after(S, S, -1), "device")
    err(L.dq_tile_io_floor(2, P, 4096, P, 2048, P, 584, 10, 0, S), "direction")
    err(L.dq_tile_io_floor(0, P, 1000, P, 2048, P, 584, 10, 0, S), "a_bytes_per_tile")
    err(L.dq_tile_io_floor(0, P, 4096, P, 2048, P, 580, 10, 0, S), "multiple of 8")
    err(L.dq_tile_io_floor(0, P, 4096, P, 2048, P, 584, 0, 0, S), "n must be positive")
    err(L.dq_tile_io_floor(0, P, 4096, N, 2048, P, 584, 10, 0, S), "null pointer")
    err(L.dq_tile_io_floor(0, ctypes.c_void_p(0x1008), 4096, N, 0, P, 584, 10, 0, S), "aligned")
    err(L.dq_rand_diag_bits(P, 100, 1, 0, S), "multiple of 256")
    err(L.dq_rand_diag_bits(N, 256, 1, 0, S), "null pointer")
    err(L.dq_pack_signs(P, P, 0, 0, S), "n must be positive")
    err(L.dq_bins_to_bits(P, 48, P, 6, 4, 0, S), "multiple of 32")
    err(L.dq_bits_to_bins(P, 64, P, 9, 4, 0, S), "narr")
    err(L.dq_quantization(N, 16, 0, ctypes.c_float(1.0), ctypes.c_float(1.0), 1, S), "null pointer")
    err(L.dq_group_plan(P, 0, P, P, 100, 0, S), "nsc")
    err(L.dq_group_plan(P, 5000, P, P, 8, 0, S), "work buffer is too small")
    err(L.dq_group_plan_stats(N, ctypes.c_double(1.0), 100, N, P, P, 100, 0, S), "null pointer")
    err(L.dq_group_plan_stats_dev_u(P, N, 100, N, P, P, 100, N, 0, 0, S), "null pointer")
    err(L.dq_group_plan_stats_dev_u(P, P, 100, N, P, P, 3, N, 0, 0, S), "work buffer is too small")
    err(L.dq_group_plan_stats_dev_u(P, P, 100, N, P, P, 100, P, 5, 0, S), "hist buffer is too small")
    err(L.dq_norm_histogram(P, 100, P, 100, 0, S), "hist buffer is too small")
    err(L.dq_norm_histogram(N, 100, P, 32768, 0, S), "null pointer")
    err(L.dq_norm_histogram(P, 0, P, 32768, 0, S), "nsc must be in")
    err(L.dq_bitrate_search(P, 32768, 2, ctypes.c_double(0.0), N, ctypes.c_double(4.0), P, 0, S), "mode must be 0")
    err(L.dq_bitrate_search(P, 100, 0, ctypes.c_double(0.0), N, ctypes.c_double(4.0), P, 0, S), "hist buffer is too small")
    err(L.dq_bitrate_search(P, 32768, 1, ctypes.c_double(float("nan")), N, ctypes.c_double(4.0), P, 0, S), "must be numbers")
    err(L.dq_bitrate_search(P, 32768, 0, ctypes.c_double(0.0), N, ctypes.c_double(4.0), N, 0, S), "null pointer")
    err(L.dq_scaling_compress_rows(P, P, P, P, 10, 4, 0, 0, 2, S), "unsupported element dtype")        # binary16 has no row-list kernels
    err(L.dq_scaling_compress_rows(P, P, P, P, 10, 4, 1, 0, 1, S), "strategy")
    err(L.dq_scaling_dec_comp_rows(P, P, P, P, P, 0, 4, 1, 0, 2, S), "n must be positive")
    err(L.dq_scaling_decompress_rows(P, P, P, P, 2560, 10, 4, 1, 0, 2, S, 1), "stats cannot be combined")
    err(L.dq_mixed_compress(P, N, 1, 0, P, P, 0, 0, N, P, P, Z, Z, 100, 1, 0, 2, S), "world")           # ring_world 0
    err(L.dq_mixed_compress(P, N, 1, 0, P, P, 3, 3, N, P, P, Z, Z, 100, 1, 0, 2, S), "world")           # chunk outside the ring
    err(L.dq_mixed_compress(P, N, 1, 0, P, P, 0, 1, N, P, P, Z, Z, 100, 0, 0, 2, S), "unsupported element dtype")
    err(L.dq_mixed_compress(P, N, 1, 0, P, P, 0, 1, N, P, P, Z, Z, 100, 1, 0, 0, S), "strategy")
    err(L.dq_mixed_compress(P, N, 1, 0, P, N, 0, 1, N, P, P, Z, Z, 100, 1, 0, 2, S), "null pointer")
    err(L.dq_mixed_compress(P, P, 1, 25700, P, P, 0, 1, N, P, P, Z, Z, 100, 1, 0, 2, S), "256 * nsc")   # n beyond the plan
    err(L.dq_mixed_compress(P, P, 0, 100, P, P, 0, 1, N, P, P, Z, Z, 100, 1, 0, 2, S), "world")         # centring by 0 ranks
    err(L.dq_mixed_decompress(P, P, P, P, 0, 1, N, 0, 100, 1, 0, 2, S), "n_limit")
    err(L.dq_mixed_decompress(P, P, P, P, 0, 1, N, 100, 0, 1, 0, 2, S), "n must be positive")
    err(L.dq_superchunk_stats(P, P, N, 0, 1, 1, 0, S), "n must be positive")
    err(L.dq_superchunk_stats(P, N, N, 100, 1, 1, 0, S), "null pointer")
    err(L.dq_superchunk_stats(P, P, N, 100, 0, 1, 0, S), "world")
    assert L.dq_mixed_required_bytes(25600, 1) == (25600 + 3) * 274 and L.dq_mixed_required_bytes(25600, 8) == (3200 + 3) * 274
    assert L.dq_mixed_required_bytes(0, 1) == 0
    err(L.dq_eden_quantize(P, 100, P, P, 4, P, P, P, 10, 0, S), "multiple of 32")
    err(L.dq_eden_quantize(P, 8192, P, P, 4, P, P, P, 1, 0, S), "work buffer is too small")
    err(L.dq_eden_dequantize(P, 64, P, 9, P, 0, S), "nbits")
    err(L.dq_eden_dequantize(P, 64, P, 4, ctypes.c_void_p(0x1004), 0, S), "16-byte aligned")
    err(L.dq_thc_quantize(P, P, P, 64, P, P, 1, 0, S), "levels")
    err(L.dq_thc_rht_quantize(P, P, 0, P, P, 96, 48, F1, P, P, 31, 0, S), "power of 2")
    err(L.dq_thc_rht_quantize(P, P, 1, P, P, 100, 64, F1, P, P, 31, 0, S), "multiple of block")
    err(L.dq_thc_rht_quantize(P, P, 0, P, P, 64, 64, F1, P, P, 1, 0, S), "levels")
    err(L.dq_thc_rht_quantize(P, P, 0, N, P, 64, 64, F1, P, P, 31, 0, S), "null pointer")
    err(L.dq_thc_dequantize_irht(P, P, 0, N, 64, 64, F1, P, P, 0, S), "null pointer")
    err(L.dq_eden_dequantize_irht(P, 64, P, 9, P, 0, P, 64, F1, N, 0, S), "nbits must be in")
    err(L.dq_eden_dequantize_irht(P, 48, P, 4, P, 0, P, 16, F1, N, 0, S), "multiple of 32")
    err(L.dq_eden_dequantize_irht(P, 64, P, 4, P, 0, P, 8, F1, N, 0, S), "block")
    err(L.dq_eden_dequantize_irht(P, 64, P, 4, P, 0, N, 64, F1, N, 0, S), "null pointer")
    err(L.dq_thc_dequantize_irht(P, P, 1, P, 0, 64, F1, P, P, 0, S), "multiple of block")
    err(L.dq_thc_dequantize(P, P, 64, N, P, 0, S), "null pointer")
    assert capi.group_plan_work_ints(25600) == 8 + 4 * 25 + 4 * 4 and capi.group_plan_work_ints(1048577) == 8 + 4 * 1025 + 4 * 33 and capi.eden_work_doubles(8192) == 4 and capi.eden_work_doubles(4096 * 1025) == 1025 and capi.bitrate_hist_ints() == 32768
    # the sorted plan: four ints up to 65535 superchunks, the radix sort's buffers (about 12.2 bytes per superchunk) beyond
    assert capi.group_plan_sorted_work_ints(65535) == 4
    big = capi.group_plan_sorted_work_ints(8_000_000)
    assert 4 * big >= 12 * 8_000_000 and 4 * big < 13 * 8_000_000
    # a good call clears the message
    assert L.dq_scaling_check_common(256, 4, 16, 2, 1) == 0 and L.dq_last_error().decode() == ""
    assert L.dq_status_string(16).decode() == "kernel launch failed"
