"""Builds libpla_gfx950.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc.

The library is built in-tree at ``pla_amd/lib/libpla_gfx950.so`` so that it
travels with the source tree; nothing is JIT-compiled at import time.
Run ``python -m pla_amd.build`` to (re)build.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libpla_gfx950.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = ["api.hip", "decode_k_last.hip", "decode_kda_mega.hip", "decode_kda_replay.hip", "commit_plan.hip", "prefill_gdn.hip", "prefill_kda.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wno-inline-asm",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 library cannot be built")
    return exe


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, proc.stdout, proc.stderr))
    return obj


def build_library(verbose=True):
    """Compile every HIP source and link the shared library. Always recompiles."""
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    from .autotune import write_header
    write_header()                       # the tuned table is compiled in from pla_amd/lut/*.csv
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-Wno-inline-asm", "-o", tmp, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (proc.stdout, proc.stderr))
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


BINDING_SRC = os.path.join(CSRC, "decode_binding.cpp")
PREFILL_BINDING_SRC = os.path.join(CSRC, "prefill_binding.cpp")

# compiled host modules: package directory (relative to pla_amd) -> (source, extra defines)
BINDINGS = {
    "decode": (BINDING_SRC, []),
    os.path.join("prefill", "flashqla"): (PREFILL_BINDING_SRC, ["-DPLA_BIND_FLASHQLA"]),
    os.path.join("prefill", "flashkdapro"): (PREFILL_BINDING_SRC, ["-DPLA_BIND_FLASHKDAPRO"]),
}


def binding_path(package="decode"):
    import sysconfig
    return os.path.join(HERE, package, "_C" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_binding(verbose=True, package="decode"):
    """Compile pla_amd/<package>/_C (pybind11 over the C ABI; host code only, g++) against this interpreter's torch.

    The module links libpla_gfx950.so by a path relative to itself; torch's libraries are found because importing
    torch precedes importing the module (the reference's extensions rely on the same order).
    """
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise RuntimeError("g++ not found; pla_amd.%s._C cannot be built" % package.replace(os.sep, "."))
    src, defines = BINDINGS[package]
    out = binding_path(package)
    tmp = out + ".tmp"
    incs = cpp_extension.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include"]
    libdirs = cpp_extension.library_paths() + [LIB_DIR]
    up = "/".join([".."] * (package.count(os.sep) + 1))
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wno-attributes",
           "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H", "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), *defines,
           *["-I" + p for p in incs], src, "-o", tmp,
           *["-L" + p for p in libdirs], "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
           "-lpla_gfx950", "-Wl,-rpath,$ORIGIN/%s/lib" % up]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building pla_amd.%s._C failed:\n%s\n%s" % (package.replace(os.sep, "."), proc.stdout, proc.stderr[-4000:]))
    os.replace(tmp, out)
    if verbose:
        print("built", out)
    return out


def build_bindings(verbose=True):
    """All compiled host modules (three g++ runs side by side)."""
    with ThreadPoolExecutor(max_workers=len(BINDINGS)) as pool:
        return list(pool.map(lambda package: build_binding(verbose, package), BINDINGS))


if __name__ == "__main__":
    build_library()
    build_bindings()
    sys.exit(0)
