"""Builds libtagi_hip.so (the HIP kernels and their C ABI) in-tree for gfx950.

    python -m cutagi_amd.build          # or: python cutagi_amd/build.py

hipcc cross-compiles without a GPU. The library has no dependency besides the
HIP runtime.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtagi_hip.so")
SOURCES = ["tagi_gemm.hip", "tagi_gemv.hip", "tagi_gemv16.hip", "tagi_small.hip", "tagi_elementwise.hip",
           "tagi_conv2d.hip", "tagi_layers.hip", "tagi_conv_idx.cpp", "tagi_capi.hip"]
# packed fp32 VALU ops are kept off for gfx950 (device pass only; the host pass
# does not know the feature and says so)
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]


def _compile(src, objdir, extra):
    obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
    cmd = ["hipcc"] + FLAGS + extra + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines()
                    if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(extra_flags=(), objdir=None, lib=LIB):
    objdir = objdir or os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=6) as pool:
        objs = list(pool.map(lambda s: _compile(s, objdir, list(extra_flags)), SOURCES))
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs,
                   check=True)
    return lib


HOST_SOURCES = ["states.cpp", "layers.cpp", "blocks.cpp", "sequential.cpp", "bindings.cpp"]


def build_host():
    """The C++ host classes (BaseLayer / Linear / Conv2d / Sequential / OutputUpdater
    mirrors) and their pybind11 module `cutagi`, linked against libtagi_hip.so."""
    import sysconfig
    import pybind11
    host = os.path.join(HERE, "host")
    objdir = os.path.join(HERE, "build", "host")
    os.makedirs(objdir, exist_ok=True)
    ext = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(HERE, "cutagi" + ext)
    flags = ["-O2", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
             "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"],
             "-fvisibility=hidden"]

    def comp(src):
        obj = os.path.join(objdir, src.replace(".cpp", ".o"))
        subprocess.run(["g++"] + flags + ["-c", os.path.join(host, src), "-o", obj], check=True)
        return obj

    with ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(comp, HOST_SOURCES))
    subprocess.run(["g++", "-shared", "-o", out] + objs +
                   ["-L" + HERE, "-ltagi_hip", "-L/opt/rocm/lib", "-lamdhip64",
                    "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    return out


if __name__ == "__main__":
    print(build())
    print(build_host())
