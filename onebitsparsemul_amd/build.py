"""Builds the native pieces in-tree with hipcc / g++ for gfx950 (no JIT cache, no install step).

    python -m onebitsparsemul_amd.build            # libonebitmul.so (+ .a) and the torch binding
"""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB = os.path.join(PKG, "libonebitmul.so")
STATIC_LIB = os.path.join(PKG, "libonebitmul.a")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops is switched off for every device compile of this project.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", INCLUDE, "-I", CSRC]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_library():
    objs = []
    for src in ("onebit_kernels.hip", "onebit_capi.hip", "onebit_diag.hip"):
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        _run([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    if os.path.exists(STATIC_LIB):
        os.remove(STATIC_LIB)
    _run(["ar", "rcs", STATIC_LIB, *objs])
    return LIB


def binding_path():
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(PKG, "onebit_sparse_cuda" + suffix)


def build_binding():
    """pybind11 module `onebit_sparse_cuda` (same module and function name as the reference's extension)."""
    import torch
    from torch.utils import cpp_extension

    out = binding_path()
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"], "-isystem", "/opt/rocm/include", "-I", INCLUDE]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=onebit_sparse_cuda", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *inc, os.path.join(CSRC, "torch_binding.cpp"), "-o", out,
           "-L", PKG, "-lonebitmul", "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
           "-ltorch_python", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    _run(cmd)
    return out


CONSUMER_SRC = os.path.join(ROOT, "tests", "consumer", "libso_test.cpp")
CONSUMER_BIN = os.path.join(ROOT, "tests", "consumer", "libso_test")


def build_consumer(out=CONSUMER_BIN):
    """The C++ consumer of the boundary (the reference's `lib_test` target, makefile:22-23): declares the entry point
    with C++ linkage as the reference's header does and links with -lonebitmul."""
    _run([HIPCC, "-O1", "-std=c++17", CONSUMER_SRC, "-o", out, "-L", PKG, "-lonebitmul",
          "-Wl,-rpath,$ORIGIN/../../onebitsparsemul_amd"])
    return out


def build_all():
    build_library()
    build_binding()
    build_consumer()


if __name__ == "__main__":
    build_all()
    print("built", LIB, binding_path())
    sys.exit(0)
