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
