"""Compiles the gfx950 engine into dciknn_cuda_amd/libdci_hip.so with hipcc.

Usage: python -m dciknn_cuda_amd.build   (cross-compiles; no GPU needed)
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libdci_hip.so")
SOURCES = ["api.hip", "project.hip", "segsort.hip", "query.hip", "traverse_block.hip", "traverse_dense.hip", "exhaustive.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    # packed fp32 VALU ops are not to be generated on these machines
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(src):
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, r


def build_library(verbose=False):
    """(Re)compile every source and link the shared library; returns its path."""
    with ThreadPoolExecutor(max_workers=4) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = []
    for src, obj, r in results:
        noise = "\n".join(l for l in r.stderr.splitlines()
                          if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, r.stderr))
        if verbose and noise.strip():
            print(noise, file=sys.stderr)
        objs.append(obj)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr)
    return LIB


EXT = os.path.join(HERE, "_dci_cuda.so")


def build_extension(verbose=False):
    """Compile the torch C++ extension `_dci_cuda` (host side, g++) against libdci_hip.so."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    if not os.path.exists(LIB):
        build_library(verbose)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_dci_cuda",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-DPYBIND11_COMPILER_TYPE=\"_gcc\"",
           "-DPYBIND11_STDLIB=\"_libstdcpp\"", "-DPYBIND11_BUILD_ABI=\"_cxxabi1011\"",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wno-deprecated-declarations"]
    for inc in ce.include_paths() + ["/opt/rocm/include", sysconfig.get_paths()["include"]]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "_dci_cuda.cpp"), "-o", EXT,
            "-L" + tlib, "-L" + HERE, "-ldci_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch", "-ltorch_python", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building _dci_cuda failed:\n%s" % r.stderr[-4000:])
    if verbose and r.stderr.strip():
        print(r.stderr[-2000:], file=sys.stderr)
    return EXT


STAMP = os.path.join(HERE, "build_stamp.txt")


def source_digest():
    """Hash of every source file the two libraries are built from."""
    import hashlib
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h", ".cpp")):
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def build_all(verbose=False):
    out = build_library(verbose), build_extension(verbose)
    with open(STAMP, "w") as f:
        f.write(source_digest() + "\n")
    return out


def is_stale():
    """True when the libraries were built from other sources than the tree holds now."""
    try:
        with open(STAMP) as f:
            return f.read().strip() != source_digest()
    except OSError:
        return False      # no stamp: built by other means, nothing to compare with


def ensure_built():
    """Build the two libraries if either is missing (tests, smoke and benchmark call
    this; they never rebuild what is there)."""
    if not (os.path.exists(LIB) and os.path.exists(EXT)):
        build_all()
    elif is_stale():
        print("dciknn_cuda_amd: libdci_hip.so / _dci_cuda.so are older than the sources in csrc/; "
              "run `python -m dciknn_cuda_amd.build` to test what the tree holds", file=sys.stderr)
    return LIB, EXT


if __name__ == "__main__":
    print(build_all(verbose=True))
