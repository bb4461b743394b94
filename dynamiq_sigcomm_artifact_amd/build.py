"""Build the native parts of the package in-tree.

  libdynamiq_eden.so   HIP kernels + C ABI (hipcc, gfx950)
  eden_utils*.so       pybind11 / libtorch binding with the reference module's
                       function names (g++), linked against libdynamiq_eden.so
  tests/cxx/liblaunchers_probe.so
                       test helper: a C++ caller of include/dynamiq_eden_launchers.hpp
                       (amdclang++, host code only), linked against libdynamiq_eden.so

Run as ``python -m dynamiq_sigcomm_artifact_amd.build`` or call ``build_all()``.
hipcc cross-compiles for gfx950 without a GPU present.
"""
import os
import subprocess
import sys
import sysconfig
import time
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "_obj")
LIB_NAME = "libdynamiq_eden.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

HIP_SOURCES = [
    "dq_api.hip",
    "dq_scaling_generic.hip",
    "dq_scaling_hier16.hip",
    "dq_scaling_tile16.hip",
    "dq_grouping.hip", "dq_bitrate.hip", "dq_sort.hip",
    "dq_scaling_mixed.hip",
    "dq_rht_scaling.hip", "dq_rht_compress_philox.hip", "dq_rht_compress_bf16.hip", "dq_rht_compress_f32.hip", "dq_rht_decompress.hip",
    "dq_superchunk.hip",
    "dq_hadamard.hip",
    "dq_packing.hip",
    "dq_eden.hip",
    "dq_streams.hip",
    "dq_io_floor.hip",
]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    # the kernels are checked bit-for-bit: only explicit fmaf may fuse
    "-ffp-contract=off",
    # keep hipcc from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd, what):
    t0 = time.time()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "is not a recognized feature for this target" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError("%s failed (%d):\n%s\n%s" % (what, proc.returncode, " ".join(cmd), out))
    if out.strip():
        print(out)
    return time.time() - t0


def _newest_header():
    return max(os.path.getmtime(os.path.join(CSRC, f)) for f in os.listdir(CSRC) if f.endswith((".cuh", ".h")))


def build_kernels(verbose=True, jobs=6, only_changed=False):
    """only_changed: keep an object file that is newer than its source and every header (for edit-compile loops;
    the default recompiles everything)"""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = _hipcc()
    headers = _newest_header() if only_changed else 0.0

    def one(src):
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        if only_changed and os.path.exists(obj) and \
                os.path.getmtime(obj) > max(headers, os.path.getmtime(os.path.join(CSRC, src))):
            return obj
        dt = _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj], "hipcc " + src)
        if verbose:
            print("  hipcc %-28s %.1fs" % (src, dt))
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(one, HIP_SOURCES))
    dt = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs, "link " + LIB_NAME)
    if verbose:
        print("  link  %-28s %.1fs" % (LIB_NAME, dt))
    return LIB_PATH


def extension_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(PKG_DIR, "eden_utils" + suffix)


def build_extension(verbose=True):
    import torch
    from torch.utils import cpp_extension as ce

    out = extension_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared",
           "-DTORCH_EXTENSION_NAME=eden_utils", "-DTORCH_API_INCLUDE_EXTENSION_H",
           # c10's HIP stream / caching-allocator headers pull in the HIP runtime API (declarations only)
           "-D__HIP_PLATFORM_AMD__=1", "-I" + os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "include"),
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    cmd += ["-I" + p for p in ce.include_paths()]
    cmd += ["-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(PKG_DIR, "..", "include")]
    cmd += [os.path.join(CSRC, "eden_utils_module.cpp"), "-o", out]
    cmd += ["-L" + PKG_DIR, "-l:" + LIB_NAME, "-Wl,-rpath,$ORIGIN",
            "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_python",
            "-Wl,-rpath," + torch_lib]
    dt = _run(cmd, "g++ eden_utils_module.cpp")
    if verbose:
        print("  g++   %-28s %.1fs" % (os.path.basename(out), dt))
    return out


PROBE_SRC = os.path.join(PKG_DIR, "..", "tests", "cxx", "launchers_probe.cpp")
PROBE_PATH = os.path.join(PKG_DIR, "..", "tests", "cxx", "liblaunchers_probe.so")


def launchers_probe_command(out, throw=False):
    """the compile line of the C++ launcher header's test caller: plain C++ for the host, the HIP headers only for
    their types"""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [os.path.join(rocm, "bin", "amdclang++"), "-O1", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Werror",
           "-D__HIP_PLATFORM_AMD__=1", "-I" + os.path.join(rocm, "include"), "-I" + os.path.join(PKG_DIR, "..", "include")]
    if throw:
        cmd.append("-DDYNAMIQ_LAUNCHERS_THROW")
    cmd += [PROBE_SRC, "-o", out, "-L" + PKG_DIR, "-l:" + LIB_NAME, "-Wl,-rpath," + PKG_DIR,
            "-Wl,-rpath,$ORIGIN/../../dynamiq_sigcomm_artifact_amd"]
    return cmd


def build_launchers_probe(verbose=True):
    dt = _run(launchers_probe_command(PROBE_PATH), "amdclang++ launchers_probe.cpp")
    if verbose:
        print("  clang %-28s %.1fs" % (os.path.basename(PROBE_PATH), dt))
    return PROBE_PATH


def build_all(verbose=True):
    lib = build_kernels(verbose)
    ext = build_extension(verbose)
    build_launchers_probe(verbose)
    return lib, ext


if __name__ == "__main__":
    only = sys.argv[1] if len(sys.argv) > 1 else "all"
    if only in ("all", "kernels"):
        build_kernels(only_changed="--changed" in sys.argv)
    if only in ("all", "ext"):
        build_extension()
    if only in ("all", "probe"):
        build_launchers_probe()
