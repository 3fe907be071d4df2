"""TEST INFRASTRUCTURE - ctypes front end of the CPU oracle (oracle/onebit_oracle.c).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the
shipped library never does. Every function here forwards to the C restatement, whose comments cite the
reference lines it follows. Arrays are numpy; nothing here touches a GPU.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
# ONEBIT_ORACLE_LIBRARY overrides the default build, e.g. the sanitizer build `make -C oracle asan` (run the CPU
# tests with it under LD_PRELOAD of gcc's libasan.so)
_LIB_PATH = os.environ.get("ONEBIT_ORACLE_LIBRARY") or os.path.join(_DIR, "libonebit_oracle.so")

LAYOUT_REFERENCE = 0
LAYOUT_CUTLASS = 1
LAYOUT_LOGICAL = 2
F32 = 0
F16 = 1


def build(force=False):
    """Compile the C oracle with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(
            os.path.join(_DIR, "onebit_oracle.c")):
        subprocess.run(["make", "-C", _DIR, "-B", "libonebit_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        L.ob_half_to_float.restype = f32
        L.ob_half_to_float.argtypes = [ctypes.c_uint16]
        L.ob_float_to_half.restype = ctypes.c_uint16
        L.ob_float_to_half.argtypes = [f32]
        L.ob_binary_quant.argtypes = [vp, i64, vp]
        L.ob_pack_binary.argtypes = [vp, i32, i32, vp]
        L.ob_unpack_binary.argtypes = [vp, i32, i32, vp]
        for name in ("ob_meta_offset_reference", "ob_meta_offset_cutlass"):
            getattr(L, name).restype = i64
            getattr(L, name).argtypes = [i64, i64, i64]
        L.ob_sparse_from_dense.argtypes = [vp, i32, i32, vp, vp, i32]
        L.ob_sparse_to_dense.argtypes = [vp, vp, i32, i32, vp, i32]
        L.ob_mask_creator.argtypes = [vp, i64, vp]
        L.ob_decompress_operands.argtypes = [vp, vp, i32, i32, i32, vp]
        L.ob_host_gemm.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, i32, i32]
        L.ob_reference_matmul.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, i32, i32, i32]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def half_to_float(h):
    return lib().ob_half_to_float(int(h))


def float_to_half(f):
    return lib().ob_float_to_half(float(f))


def binary_quant(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().ob_binary_quant(_p(x), x.size, _p(out))
    return out


def pack_binary(bits):
    bits = _c(bits, np.uint8)
    rows, cols = bits.shape
    out = np.empty((rows, cols // 8), np.uint8)
    if lib().ob_pack_binary(_p(bits), rows, cols, _p(out)):
        raise ValueError("last dimension must be a multiple of 8")
    return out


def unpack_binary(packed):
    packed = _c(packed, np.uint8)
    rows, pc = packed.shape
    out = np.empty((rows, pc * 8), np.uint8)
    lib().ob_unpack_binary(_p(packed), rows, pc, _p(out))
    return out


def meta_offset(r, c, m, layout=LAYOUT_REFERENCE):
    f = lib().ob_meta_offset_reference if layout == LAYOUT_REFERENCE else lib().ob_meta_offset_cutlass
    return f(r, c, m)


def sparse_from_dense(dense, layout=LAYOUT_REFERENCE):
    dense = _c(dense, np.float32)
    m, k = dense.shape
    sparse = np.empty((m, k // 2), np.float32)
    meta = np.zeros((m, k // 16), np.int16)
    rc = lib().ob_sparse_from_dense(_p(dense), m, k, _p(sparse), _p(meta), layout)
    if rc:
        raise ValueError(f"shape ({m}, {k}) rejected (code {rc})")
    return sparse, meta


def sparse_to_dense(sparse, meta, layout=LAYOUT_REFERENCE):
    sparse = _c(sparse, np.float32)
    meta = _c(meta, np.int16)
    m, ks = sparse.shape
    dense = np.empty((m, 2 * ks), np.float32)
    if lib().ob_sparse_to_dense(_p(sparse), _p(meta), m, ks, _p(dense), layout):
        raise ValueError("bad shape")
    return dense


def mask_creator(w):
    w = _c(w, np.float32)
    mask = np.empty(w.shape, np.float32)
    lib().ob_mask_creator(_p(w), w.size, _p(mask))
    return mask


def decompress_operands(a, e, m, k, layout=LAYOUT_REFERENCE):
    """(a bits, e metadata) in the C entry point's formats -> dense int8 (m, k) in {-1, 0, +1}."""
    a = _c(a, np.uint8).reshape(-1)
    e = _c(e, np.int16).reshape(-1)
    assert a.size == m * k // 16 and e.size == m * k // 16
    dense = np.empty((m, k), np.int8)
    if lib().ob_decompress_operands(_p(a), _p(e), m, k, layout, _p(dense)):
        raise ValueError("bad shape")
    return dense


def host_gemm(a_dense, b_half, c=None, alpha=1.0, beta=0.0, d_dtype=F16, acc="f32"):
    """Reference host GEMM on the decompressed A. b_half: float16 (k, n). acc: 'f32' (sequential fp32,
    the reference's host GEMM) or 'f64'. Returns d as float16 or float32."""
    a_dense = _c(a_dense, np.int8)
    b_half = _c(b_half, np.float16)
    m, k = a_dense.shape
    n = b_half.shape[1]
    c_dtype = F32
    cbuf = None
    if c is not None:
        c_dtype = F16 if c.dtype == np.float16 else F32
        cbuf = _c(c, np.float16 if c_dtype == F16 else np.float32)
    d = np.empty((m, n), np.float16 if d_dtype == F16 else np.float32)
    rc = lib().ob_host_gemm(_p(a_dense), _p(b_half.view(np.uint16)), _p(cbuf) if cbuf is not None else None, _p(d), m,
                            n, k, alpha, beta, c_dtype, d_dtype, 0 if acc == "f32" else 1)
    if rc:
        raise RuntimeError("host gemm failed")
    return d


def reference_matmul(a, b_half, e, m, n, k, c=None, alpha=1.0, beta=0.0, d_dtype=F16, layout=LAYOUT_REFERENCE,
                     acc="f32"):
    dense = decompress_operands(a, e, m, k, layout)
    return host_gemm(dense, b_half, c, alpha, beta, d_dtype, acc)


def blas_matmul(a_dense, b_half, c=None, alpha=1.0, beta=0.0, dtype=np.float64):
    """Same product through numpy's BLAS (any summation order); for sizes where the sequential loop is slow."""
    acc = a_dense.astype(dtype) @ b_half.astype(dtype)
    out = dtype(alpha) * acc
    if c is not None and beta != 0.0:
        out = out + dtype(beta) * c.astype(dtype)
    return out


def cpu_baseline_gemm(a, b_half, e, m, n, k, row_begin, row_end, layout=LAYOUT_REFERENCE, threads=None, repeats=1):
    """The reference's CPU path (onebit_sparse_mul/__init__.py:67-97: decompress the weight, then a dense
    torch.matmul) on rows [row_begin, row_end) of A, in fp32 on the host's cores. Returns (seconds of one
    matmul, averaged over `repeats`; seconds of the decompression; result slab as float32 numpy)."""
    import time

    import torch

    if threads:
        torch.set_num_threads(threads)
    t0 = time.perf_counter()
    dense = decompress_operands(a, e, m, k, layout)[row_begin:row_end]
    t1 = time.perf_counter()
    a_t = torch.from_numpy(dense).to(torch.float32)
    b_t = torch.from_numpy(np.ascontiguousarray(b_half)).to(torch.float32)
    torch.matmul(a_t[:64], b_t)  # warm-up of the BLAS threads
    t2 = time.perf_counter()
    for _ in range(repeats):
        out = torch.matmul(a_t, b_t)
    t3 = time.perf_counter()
    return (t3 - t2) / repeats, t1 - t0, out.numpy()
