"""Build recipe of the native parts: libflashgs_hip.so (HIP kernels behind the C ABI) and the
``flash_gaussian_splatting`` Python extension that mirrors FlashGS's op surface.

Everything is compiled for gfx950 only and lands in-tree (``flashgs_amd/lib/`` and the
repository root), so a copy of the tree carries the binaries with it.

    python -m flashgs_amd.build              # both
    python -m flashgs_amd.build --lib        # only the C-ABI library
    python -m flashgs_amd.build --asan-host  # flashgs_amd/lib/asan/host_checks: the library's host code and the .ply
                                             # reader under the address and undefined-behaviour sanitizers (CPU only)
"""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libflashgs_hip.so")
CAL_PATH = os.path.join(LIB_DIR, "libflashgs_calibrate.so")     # microbenchmarks for bench.py --calibrate
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# Packed fp32 instructions are switched off for every kernel of this library.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# preprocess.hip feeds bit-exact tile keys: one IEEE operation per source operation, no fusing.
SOURCES = {
    "common.hip": [],
    "preprocess.hip": ["-ffp-contract=off"],
    "sort.hip": [],
    "render.hip": ["-ffp-contract=fast"],
}


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_lib():
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = []
    for src, extra in SOURCES.items():
        obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        _run([HIPCC] + HIP_FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs)
    _run([HIPCC] + HIP_FLAGS + ["-shared", os.path.join(CSRC, "calibrate.hip"), "-o", CAL_PATH])
    return LIB_PATH


ASAN_DIR = os.path.join(LIB_DIR, "asan")
ASAN_CHECKS = os.path.join(ASAN_DIR, "host_checks")
# sanitizers on the host code only: each -fsanitize= directly behind -Xarch_host
ASAN_HOST = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
             "-Xarch_host", "-fno-sanitize-recover=undefined", "-g", "-fno-omit-frame-pointer"]


def build_asan_host():
    """host_checks.cpp linked with the library's own translation units, host code instrumented.
    Run it as ``ASAN_OPTIONS=detect_leaks=0 flashgs_amd/lib/asan/host_checks`` (the HIP runtime keeps
    allocations of its own until the process ends); it launches nothing and needs no GPU."""
    os.makedirs(ASAN_DIR, exist_ok=True)
    objs = []
    for src, extra in SOURCES.items():
        obj = os.path.join(ASAN_DIR, src.replace(".hip", ".o"))
        _run([HIPCC] + HIP_FLAGS + ASAN_HOST + extra + ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    main = os.path.join(ASAN_DIR, "host_checks.o")
    _run([HIPCC, "-x", "hip"] + HIP_FLAGS + ASAN_HOST + ["-I", os.path.join(ROOT, "include"), "-c",
                                                        os.path.join(CSRC, "host_checks.cpp"), "-o", main])
    _run([HIPCC, "--offload-arch=gfx950", "-fno-gpu-sanitize", "-fsanitize=address", "-fsanitize=undefined", "-o", ASAN_CHECKS, main] + objs)
    return ASAN_CHECKS


def ext_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX")
    return os.path.join(ROOT, "flash_gaussian_splatting" + suffix)


def build_ext():
    """The pybind11/torch extension named like the reference's (setup.py:32-48 of FlashGS)."""
    import torch
    from torch.utils import cpp_extension as ce

    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"], "-isystem", os.path.join(ROCM, "include")]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    out = ext_path()
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-variable",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=flash_gaussian_splatting",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
           "-I", os.path.join(ROOT, "include")] + inc + [
           os.path.join(CSRC, "pybind.cpp"), "-o", out,
           "-L", LIB_DIR, "-lflashgs_hip", "-Wl,-rpath,$ORIGIN/flashgs_amd/lib",
           "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-Wl,-rpath," + torch_lib,
           "-L", os.path.join(ROCM, "lib"), "-lamdhip64"]
    _run(cmd)
    return out


def build_all():
    build_lib()
    if os.path.exists(os.path.join(CSRC, "pybind.cpp")):
        build_ext()


if __name__ == "__main__":
    if "--lib" in sys.argv:
        build_lib()
    elif "--asan-host" in sys.argv:
        build_asan_host()
    else:
        build_all()
