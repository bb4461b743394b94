"""include/dynamiq_eden_launchers.hpp: the C++ launchers with the reference's names and argument lists
(csrc/cuda_hadamard.h:13-28, csrc/cuda_packing.h:10-11) that a ROCm build of the transport extension would call
(ring_allreduce_backend.cu:1255-1301,1678-1721).  tests/cxx/launchers_probe.cpp is such a caller: it binds every
launcher to a function pointer of exactly the declared type and re-exports them as plain C for ctypes.

Without a GPU: the probe compiles (warnings are errors) in both error modes, exports its wrappers, and a launcher
called with bad arguments prints the library's message and keeps the status.  On the GPU: every launcher writes
the bytes that the C-ABI entry point writes."""
import ctypes
import os
import subprocess

import pytest
import torch

from dynamiq_sigcomm_artifact_amd import build, capi

PROBES = ["probe_last_status", "probe_hadamard", "probe_compress", "probe_decompress", "probe_dec_comp",
          "probe_mean_center", "probe_add_mean_copy", "probe_init_lookup_table", "probe_bins_to_bits",
          "probe_bits_to_bins", "probe_quantization"]

# every launcher name that the reference's two headers declare for this path, and how often (overloads)
REFERENCE_LAUNCHERS = {"HadamardWithCudaNoSharedMemory": 1, "HadamardWithCuda": 1, "scaling_compress_with_cuda": 2,
                       "scaling_decompress_with_cuda": 2, "scaling_dec_comp_with_cuda": 1,
                       "superchunk_mean_center_with_cuda": 2, "superchunk_add_mean_copy_with_cuda": 2,
                       "init_lookup_table": 1, "BinsToBits": 1, "BitsToBins": 1}


def _compile(tmp_path, throw):
    out = str(tmp_path / ("probe_throw.so" if throw else "probe.so"))
    proc = subprocess.run(build.launchers_probe_command(out, throw=throw), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
    return out


def test_header_defines_every_reference_launcher():
    import re
    text = open(os.path.join(os.path.dirname(build.PKG_DIR), "include", "dynamiq_eden_launchers.hpp")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, count in REFERENCE_LAUNCHERS.items():
        assert len(re.findall(r"\binline void %s\(" % name, text)) == count, name


@pytest.mark.parametrize("throw", [False, True])
def test_probe_compiles_and_exports(tmp_path, throw):
    capi.lib()  # the probe's dependency, loaded from its in-tree path first
    L = ctypes.CDLL(_compile(tmp_path, throw))
    for name in PROBES:
        assert hasattr(L, name), name


def test_launcher_reports_bad_arguments_like_the_library(tmp_path, capfd):
    """n = 250 is not a multiple of the chunk size: the C ABI returns before any HIP call, the launcher prints the
    library's message (the reference's launchers print and return, cuda_hadamard.cu:1496-1499) and keeps the status"""
    capi.lib()
    L = ctypes.CDLL(_compile(tmp_path, False))
    P = ctypes.c_void_p(0x1000)
    assert L.probe_last_status() == 0
    L.probe_compress(0, P, P, P, 250, 4, 16, 0, 0, None)
    err = capfd.readouterr().err
    assert "scaling_compress_with_cuda" in err and "multiple of chunk_size" in err
    status = L.probe_last_status()
    assert status == capi.lib().dq_scaling_check_common(250, 4, 16, 0, 1) != 0
    assert L.probe_last_status() == 0          # reading clears it
    L.probe_mean_center(1, P, P, P, 256, 2, 128, 0, None)
    assert "superchunk_size must be 256" in capfd.readouterr().err
    assert L.probe_last_status() != 0
    L.probe_hadamard(P, 1000, 0, None, 1)
    assert "HadamardWithCuda:" in capfd.readouterr().err
    L.probe_hadamard(P, 1000, 0, None, 0)
    assert "HadamardWithCudaNoSharedMemory:" in capfd.readouterr().err
    L.probe_bins_to_bits(P, 48, P, 6, 4, 0)
    assert "BinsToBits" in capfd.readouterr().err


# ---- on the GPU: the launchers against the C ABI ----------------------------------------------------------

def _probe():
    capi.lib()
    if not os.path.exists(build.PROBE_PATH):
        pytest.fail("tests/cxx/liblaunchers_probe.so is not built (python -m dynamiq_sigcomm_artifact_amd.build probe)")
    L = ctypes.CDLL(build.PROBE_PATH)
    L.probe_quantization.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float,
                                     ctypes.c_uint64, ctypes.c_void_p]
    return L


def _vp(t):
    return ctypes.c_void_p(t.data_ptr())


def _st():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nbits,strategy", [(4, 2), (8, 3), (2, 0), (4, 1)])
def test_scaling_launchers_write_the_bytes_of_the_c_abi(dtype, nbits, strategy):
    L = _probe()
    dev = torch.device("cuda:0")
    half = 1 if dtype == torch.float16 else 0
    n = 256 * 37
    g = torch.Generator(device=dev).manual_seed(nbits * 10 + strategy)
    x = (torch.randn(n, generator=g, device=dev) * 1e-2).to(dtype)
    r = torch.rand(n, generator=g, device=dev).to(dtype)
    nbytes = capi.required_bytes(n, nbits, 16, strategy)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # a stream of the caller's, not the null stream
        want = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        got = torch.zeros_like(want)
        capi.scaling_compress(x, want, r, n, nbits, 16, strategy)
        L.probe_compress(half, _vp(x), _vp(got), _vp(r), n, nbits, 16, 0, strategy, _st())
        assert L.probe_last_status() == 0
        assert torch.equal(got, want)
        for add in (0, 1):
            base = (torch.randn(n, generator=g, device=dev) * 1e-2).to(dtype)
            a, b = base.clone(), base.clone()
            capi.scaling_decompress(want, a, n, nbits, 16, strategy, add=bool(add))
            L.probe_decompress(half, _vp(want), _vp(b), n, nbits, 16, 0, strategy, _st(), add)
            assert L.probe_last_status() == 0
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))
        if not half:
            inp = (torch.randn(n, generator=g, device=dev) * 1e-2).to(dtype)
            ia, ib = inp.clone(), inp.clone()
            sa, sb = torch.zeros_like(want), torch.zeros_like(want)
            capi.scaling_dec_comp(want, ia, sa, r, n, nbits, 16, strategy)
            L.probe_dec_comp(_vp(want), _vp(ib), _vp(sb), _vp(r), n, nbits, 16, 0, strategy, _st())
            assert L.probe_last_status() == 0
            assert torch.equal(sa, sb) and torch.equal(ia.view(torch.int16), ib.view(torch.int16))
    side.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_superchunk_launchers(dtype):
    L = _probe()
    dev = torch.device("cuda:0")
    half = 1 if dtype == torch.float16 else 0
    n = 256 * 21 + 100   # a ragged last superchunk
    nsc = (n + 255) // 256
    g = torch.Generator(device=dev).manual_seed(5)
    x = (torch.randn(n, generator=g, device=dev) * 1e-2 + 3e-3).to(dtype)
    ra, rb = (torch.empty(nsc * 256, dtype=dtype, device=dev) for _ in range(2))
    sa, sb = (torch.empty(2 * nsc, dtype=torch.bfloat16, device=dev) for _ in range(2))
    capi.superchunk_mean_center(x, ra, sa, n, 8)
    L.probe_mean_center(half, _vp(x), _vp(rb), _vp(sb), n, 8, 256, 0, _st())
    assert L.probe_last_status() == 0
    assert torch.equal(ra.view(torch.int16), rb.view(torch.int16)) and torch.equal(sa.view(torch.int16), sb.view(torch.int16))
    da, db = (torch.zeros(n, dtype=dtype, device=dev) for _ in range(2))
    capi.superchunk_add_mean_copy(ra, da, sa, n)
    L.probe_add_mean_copy(half, _vp(ra), _vp(db), _vp(sa), n, 256, 0, _st())
    assert L.probe_last_status() == 0
    assert torch.equal(da.view(torch.int16), db.view(torch.int16))


@pytest.mark.gpu
def test_transform_packing_and_rounding_launchers():
    L = _probe()
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(9)
    L.probe_init_lookup_table()
    assert L.probe_last_status() == 0
    x = torch.randn(1 << 14, generator=g, device=dev)
    want = x.clone()
    capi.hadamard(want)
    for shared in (1, 0):
        got = x.clone()
        L.probe_hadamard(_vp(got), got.numel(), 0, _st(), shared)
        assert L.probe_last_status() == 0
        assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    # the packers run on the null stream, as the reference's do: order them against torch's stream by hand
    nbits = 5
    bins = torch.randint(0, 1 << nbits, (4096,), generator=g, device=dev, dtype=torch.int32)
    arr_w = torch.zeros(4096 // 32 * nbits, dtype=torch.int32, device=dev)
    arr_g = torch.zeros_like(arr_w)
    back = torch.zeros_like(bins)
    capi.bins_to_bits(bins, arr_w, nbits)
    torch.cuda.synchronize()
    L.probe_bins_to_bits(_vp(bins), bins.numel(), _vp(arr_g), arr_g.numel(), nbits, 0)
    L.probe_bits_to_bins(_vp(back), back.numel(), _vp(arr_g), arr_g.numel(), nbits, 0)
    torch.cuda.synchronize()
    assert L.probe_last_status() == 0
    assert torch.equal(arr_g, arr_w) and torch.equal(back, bins)
    v = torch.randn(10000, generator=g, device=dev) * 20
    a, b = v.clone(), v.clone()
    capi.quantization(a, 1.5, 15.0, 77)
    L.probe_quantization(_vp(b), b.numel(), 0, 1.5, 15.0, 77, _st())
    assert L.probe_last_status() == 0
    assert torch.equal(a, b)
