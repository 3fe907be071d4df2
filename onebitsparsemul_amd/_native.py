"""ctypes loader of libonebitmul.so (the C ABI of include/onebit_sparse_tensor.h). There is no fallback:
if the library is missing or a call fails, an exception is raised."""
import ctypes
import os

import torch

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "libonebitmul.so")

F32, F16 = 0, 1
META_REFERENCE, META_CUTLASS, META_LOGICAL = 0, 1, 2

EXPORTS = (
    "onebit_sparse_matmul", "onebit_sparse_matmul_ex", "onebit_sparse_prepared_bytes", "onebit_sparse_prepare",
    "onebit_sparse_matmul_prepared", "onebit_sparse_matmul_prepared_static", "onebit_sparse_linear_prepared", "onebit_sparse_pack", "onebit_sparse_last_error", "onebit_sparse_set_tile_config",
    "onebit_sparse_set_skinny_enabled", "onebit_sparse_set_skinny_rows", "onebit_sparse_set_split_k", "onebit_sparse_set_pad_b", "onebit_sparse_describe_launch", "onebit_sparse_set_weight_cache", "onebit_sparse_clear_weight_cache", "onebit_sparse_release_buffers",
    "onebit_sparse_measure_smfmac_rate", "onebit_sparse_device_info",
    "onebit_sparse_describe_launch_for", "onebit_sparse_measure_smfmac_rate_shape",
    "onebit_sparse_linear_prepared_grouped",
)


class LinearProblem(ctypes.Structure):
    """onebit_linear_problem of include/onebit_sparse_tensor.h"""
    _fields_ = [("prepared", ctypes.c_void_p), ("x", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("m", ctypes.c_int), ("k", ctypes.c_int)]

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: run `python -m onebitsparsemul_amd.build` (needs hipcc)")
        L = ctypes.CDLL(LIB_PATH)
        vp, i32, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.onebit_sparse_matmul.restype = None
        L.onebit_sparse_matmul.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32]
        L.onebit_sparse_matmul_ex.restype = i32
        L.onebit_sparse_matmul_ex.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, i32, i32, vp]
        L.onebit_sparse_prepared_bytes.restype = ctypes.c_size_t
        L.onebit_sparse_prepared_bytes.argtypes = [i32, i32]
        L.onebit_sparse_prepare.restype = i32
        L.onebit_sparse_prepare.argtypes = [vp, vp, i32, i32, i32, vp, vp]
        L.onebit_sparse_matmul_prepared.restype = i32
        L.onebit_sparse_matmul_prepared.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, i32, vp]
        L.onebit_sparse_matmul_prepared_static.restype = i32
        L.onebit_sparse_matmul_prepared_static.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32, f32, i32, i32, vp]
        L.onebit_sparse_linear_prepared.restype = i32
        L.onebit_sparse_linear_prepared.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]
        L.onebit_sparse_linear_prepared_grouped.restype = i32
        L.onebit_sparse_linear_prepared_grouped.argtypes = [ctypes.POINTER(LinearProblem), i32, i32, i32, i32, vp]
        L.onebit_sparse_pack.restype = i32
        L.onebit_sparse_pack.argtypes = [vp, i32, i32, i32, vp, vp, i32, vp]
        L.onebit_sparse_last_error.restype = ctypes.c_char_p
        L.onebit_sparse_last_error.argtypes = []
        L.onebit_sparse_set_tile_config.restype = None
        L.onebit_sparse_set_tile_config.argtypes = [i32]
        L.onebit_sparse_set_skinny_enabled.restype = None
        L.onebit_sparse_set_skinny_enabled.argtypes = [i32]
        L.onebit_sparse_set_skinny_rows.restype = None
        L.onebit_sparse_set_skinny_rows.argtypes = [i32]
        L.onebit_sparse_set_split_k.restype = None
        L.onebit_sparse_set_split_k.argtypes = [i32]
        L.onebit_sparse_set_pad_b.restype = None
        L.onebit_sparse_set_pad_b.argtypes = [i32]
        L.onebit_sparse_set_weight_cache.restype = i32
        L.onebit_sparse_set_weight_cache.argtypes = [i32]
        L.onebit_sparse_clear_weight_cache.restype = i32
        L.onebit_sparse_clear_weight_cache.argtypes = []
        L.onebit_sparse_release_buffers.restype = i32
        L.onebit_sparse_release_buffers.argtypes = []
        L.onebit_sparse_describe_launch.restype = i32
        L.onebit_sparse_describe_launch.argtypes = [i32, i32, i32, i32, ctypes.POINTER(ctypes.c_int)]
        L.onebit_sparse_describe_launch_for.restype = i32
        L.onebit_sparse_describe_launch_for.argtypes = [i32, i32, i32, i32, i32, ctypes.POINTER(ctypes.c_int)]
        L.onebit_sparse_measure_smfmac_rate_shape.restype = i32
        L.onebit_sparse_measure_smfmac_rate_shape.argtypes = [i32, i32, i32, ctypes.POINTER(ctypes.c_double)]
        L.onebit_sparse_device_info.restype = i32
        L.onebit_sparse_device_info.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.onebit_sparse_measure_smfmac_rate.restype = i32
        L.onebit_sparse_measure_smfmac_rate.argtypes = [i32, i32, ctypes.POINTER(ctypes.c_double)]
        _lib = L
    return _lib


def last_error():
    return lib().onebit_sparse_last_error().decode()


def _check(rc):
    if rc != 0:
        raise RuntimeError(f"libonebitmul: {last_error()} (status {rc})")


def _dtype_code(t):
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.float16:
        return F16
    raise TypeError(f"C / D must be float32 or float16, got {t.dtype}")


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require_cuda(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("all operands must live on the GPU")
        if not t.is_contiguous():
            raise ValueError("all operands must be contiguous")
        if dev is not None and t.device != dev:
            raise ValueError("all operands must be on the same device")
        dev = t.device
    return dev


class _on_device:
    """Make `dev` the current device for the duration of a library call; free when it already is (the usual case:
    entering torch.cuda.device() costs more than the call it guards)."""

    def __init__(self, dev):
        self._guard = None if dev.index == torch.cuda.current_device() else torch.cuda.device(dev)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            self._guard.__exit__(*exc)
        return False


def prepared_bytes(m, k):
    return lib().onebit_sparse_prepared_bytes(m, k)


def _prepared_bytes_fast(m, k):
    """onebit_sparse_prepared_bytes without the library call (hot path of the per-call checks): one 1536-byte
    block per 32 rows and 256 columns."""
    return ((m + 31) // 32) * ((k + 255) // 256) * 1536


def prepare(a, meta, m, k, layout=META_REFERENCE):
    """Reorder (a bits, metadata) into the operand the kernels consume. Returns a uint8 device tensor."""
    dev = _require_cuda(a, meta)
    if a.numel() * a.element_size() != m * k // 16 or meta.numel() * meta.element_size() != m * k // 8:
        raise ValueError("operand sizes do not match m, k")
    out = torch.empty(prepared_bytes(m, k), dtype=torch.uint8, device=dev)
    with _on_device(dev):
        _check(lib().onebit_sparse_prepare(a.data_ptr(), meta.data_ptr(), m, k, layout, out.data_ptr(), _stream(a)))
    return out


STATIC_SCRATCH_BYTES = 64 << 20


def matmul_prepared(prepared, b, d, m, n, k, c=None, alpha=1.0, beta=0.0, static_scratch=False):
    """D = alpha * A * B + beta * C on the prepared weight. static_scratch=True takes the entry point that never
    allocates device memory (its internal buffers live in a fixed array of STATIC_SCRATCH_BYTES)."""
    dev = _require_cuda(prepared, b, d, c)
    if b.dtype != torch.float16 or tuple(b.shape) != (k, n):
        raise ValueError("B must be float16 of shape (k, n)")
    if tuple(d.shape) != (m, n) or (c is not None and tuple(c.shape) != (m, n)):
        raise ValueError("C / D must have shape (m, n)")
    if prepared.numel() != _prepared_bytes_fast(m, k):
        raise ValueError("prepared operand does not match m, k")
    entry = lib().onebit_sparse_matmul_prepared_static if static_scratch else lib().onebit_sparse_matmul_prepared
    with _on_device(dev):
        _check(entry(
            prepared.data_ptr(), b.data_ptr(), c.data_ptr() if c is not None else None, d.data_ptr(), m, n, k,
            alpha, beta, _dtype_code(c) if c is not None else F32, _dtype_code(d), _stream(b)))
    return d


def linear_prepared(prepared, x, y, m, k, bias=None):
    """y (tokens, m) = x (tokens, k) @ W.T (+ bias), x fp16 and y fp16 / fp32, both token-major and contiguous."""
    dev = _require_cuda(prepared, x, y, bias)
    tokens = x.shape[0]
    if x.dtype != torch.float16 or tuple(x.shape) != (tokens, k):
        raise ValueError("x must be float16 of shape (tokens, k)")
    if tuple(y.shape) != (tokens, m) or (bias is not None and tuple(bias.shape) != (m,)):
        raise ValueError("y must have shape (tokens, m) and bias (m,)")
    if prepared.numel() != _prepared_bytes_fast(m, k):
        raise ValueError("prepared operand does not match m, k")
    with _on_device(dev):
        _check(lib().onebit_sparse_linear_prepared(
            prepared.data_ptr(), x.data_ptr(), bias.data_ptr() if bias is not None else None, y.data_ptr(), tokens, m, k,
            _dtype_code(bias) if bias is not None else F16, _dtype_code(y), _stream(x)))
    return y


def linear_prepared_grouped(problems):
    """Several products y_i = x_i @ W_i.T (+ bias_i) with the same token count in one call (one launch per 16 problems
    when tokens <= 64). problems: sequence of (prepared, x, y, m, k, bias or None); all y of one dtype, all biases of one."""
    if not problems:
        return
    tokens = problems[0][1].shape[0]
    table = (LinearProblem * len(problems))()
    dev = None
    bias_code, y_code = F16, None
    for i, (prepared, x, y, m, k, bias) in enumerate(problems):
        dev = _require_cuda(prepared, x, y, bias)
        if x.dtype != torch.float16 or tuple(x.shape) != (tokens, k):
            raise ValueError("every x must be float16 of shape (tokens, k) with the same token count")
        if tuple(y.shape) != (tokens, m) or (bias is not None and tuple(bias.shape) != (m,)):
            raise ValueError("y must have shape (tokens, m) and bias (m,)")
        if prepared.numel() != _prepared_bytes_fast(m, k):
            raise ValueError("prepared operand does not match m, k")
        if y_code is not None and _dtype_code(y) != y_code:
            raise TypeError("all results must have the same dtype")
        y_code = _dtype_code(y)
        if bias is not None:
            code = _dtype_code(bias)
            if any(p[5] is not None and _dtype_code(p[5]) != code for p in problems[:i]):
                raise TypeError("all biases must have the same dtype")
            bias_code = code
        table[i] = LinearProblem(prepared.data_ptr(), x.data_ptr(), bias.data_ptr() if bias is not None else None,
                                 y.data_ptr(), m, k)
    with _on_device(dev):
        _check(lib().onebit_sparse_linear_prepared_grouped(table, len(problems), tokens, bias_code, y_code,
                                                           _stream(problems[0][1])))


def _check_stored_operands(a, meta, c, d, m, n, k):
    """Sizes of the reference-format operands: a wrong-sized tensor would be read or written out of bounds."""
    if m % 64 or k % 32 or m <= 0 or k <= 0 or n <= 0:
        raise ValueError("m must be a positive multiple of 64, k of 32, n positive")
    if a.dtype != torch.uint8 or a.numel() != m * k // 16:
        raise ValueError(f"A must be uint8 with m*k/16 = {m * k // 16} bytes (one bit per kept value)")
    if meta.dtype != torch.int16 or meta.numel() != m * k // 16:
        raise ValueError(f"meta must be int16 with m*k/16 = {m * k // 16} elements")
    if tuple(d.shape) != (m, n) or (c is not None and tuple(c.shape) != (m, n)):
        raise ValueError("C / D must have shape (m, n)")


def matmul_ex(a, b, meta, d, m, n, k, c=None, alpha=1.0, beta=0.0, layout=META_REFERENCE):
    dev = _require_cuda(a, b, meta, d, c)
    if b.dtype != torch.float16 or tuple(b.shape) != (k, n):
        raise ValueError("B must be float16 of shape (k, n)")
    _check_stored_operands(a, meta, c, d, m, n, k)
    with _on_device(dev):
        _check(lib().onebit_sparse_matmul_ex(
            a.data_ptr(), b.data_ptr(), c.data_ptr() if c is not None else None, d.data_ptr(), meta.data_ptr(), m, n,
            k, alpha, beta, _dtype_code(c) if c is not None else F32, _dtype_code(d), layout, _stream(b)))
    return d


def matmul_legacy(a, b, c, d, meta, m, n, k):
    """The 8-argument entry point: fp32 C/D, alpha = 1, beta = 0, default stream."""
    dev = _require_cuda(a, b, c, d, meta)
    if b.dtype != torch.float16 or tuple(b.shape) != (k, n):
        raise ValueError("B must be float16 of shape (k, n)")
    _check_stored_operands(a, meta, c, d, m, n, k)
    if d.dtype != torch.float32 or c.dtype != torch.float32:
        raise TypeError("the 8-argument entry point takes float32 C and D")
    with _on_device(dev):
        lib().onebit_sparse_matmul(a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), meta.data_ptr(), m, n, k)
    return d


def set_tile_config(cfg):
    lib().onebit_sparse_set_tile_config(cfg)


def set_skinny_enabled(flag):
    lib().onebit_sparse_set_skinny_enabled(1 if flag else 0)


def set_skinny_rows(rows):
    lib().onebit_sparse_set_skinny_rows(rows)


def set_split_k(splits):
    lib().onebit_sparse_set_split_k(splits)


def set_pad_b(enabled):
    lib().onebit_sparse_set_pad_b(1 if enabled else 0)


SMFMAC_32X32X32, SMFMAC_16X16X64 = 0, 1


def measure_smfmac_rate(random_operands=True, iterations=50000, shape=SMFMAC_32X32X32):
    """Sustained register-only rate of one SMFMAC instruction on the current GPU, dense-equivalent TFLOP/s (diagnostic)."""
    out = ctypes.c_double(0.0)
    rc = lib().onebit_sparse_measure_smfmac_rate_shape(shape, 1 if random_operands else 0, iterations, ctypes.byref(out))
    if rc != 0:
        raise RuntimeError(f"libonebitmul: measuring the SMFMAC rate failed (status {rc})")
    return out.value


def pack_weight(weight, prune=True, layout=META_REFERENCE):
    """dense fp16 (m, k) on the GPU -> (a uint8 (k/2, m/8), meta int16 (m, k/16)), the stored operands."""
    dev = _require_cuda(weight)
    if weight.dtype != torch.float16 or weight.dim() != 2:
        raise TypeError("weight must be a 2-dimensional float16 tensor")
    m, k = weight.shape
    a = torch.empty((k // 2, m // 8), dtype=torch.uint8, device=dev)
    meta = torch.empty((m, k // 16), dtype=torch.int16, device=dev)
    with _on_device(dev):
        _check(lib().onebit_sparse_pack(weight.data_ptr(), m, k, 1 if prune else 0, a.data_ptr(), meta.data_ptr(), layout,
                                        _stream(weight)))
    return a, meta


def device_info():
    """(compute units, peak engine clock in kHz) of the current device."""
    cus, khz = ctypes.c_int(0), ctypes.c_int(0)
    _check(lib().onebit_sparse_device_info(ctypes.byref(cus), ctypes.byref(khz)))
    return cus.value, khz.value


def describe_launch(m, n, k, b_aligned=True, compute_units=256):
    """What a prepared call of this shape would launch on a GPU with `compute_units` compute units (host-only; None = the
    current device's count, which is what the calls themselves plan for): dict(kernel, rows or tile, splits, pad_b)."""
    plan = (ctypes.c_int * 4)()
    if compute_units is None:
        _check(lib().onebit_sparse_describe_launch(m, n, k, 1 if b_aligned else 0, plan))
    else:
        _check(lib().onebit_sparse_describe_launch_for(m, n, k, 1 if b_aligned else 0, compute_units, plan))
    if plan[0]:
        return dict(kernel="skinny_kernel", rows=plan[1], splits=plan[2])
    return dict(kernel="gemm_kernel", tile=plan[1], splits=plan[2], pad_b=bool(plan[3]))


def set_weight_cache(entries):
    """Opt-in cache of reordered weights for the one-call entry points (0 = off, the default)."""
    _check(lib().onebit_sparse_set_weight_cache(entries))


def release_buffers():
    """Free the library-owned buffers of the one-call / K-split / padded-B paths (after a device synchronization)."""
    _check(lib().onebit_sparse_release_buffers())


def clear_weight_cache():
    _check(lib().onebit_sparse_clear_weight_cache())
