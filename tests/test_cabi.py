"""The C ABI of libonebitmul.so as far as it can be exercised without a GPU: the library loads, exports every
symbol that include/onebit_sparse_tensor.h and include/onebit_sparse_tuning.h declare, validates its arguments and reports HIP failures as
status codes (or, for the 8-argument symbol, as exit(EXIT_FAILURE) like the reference)."""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "onebit_sparse_tensor.h")
TUNING_HEADER = os.path.join(ROOT, "include", "onebit_sparse_tuning.h")

from onebitsparsemul_amd import _native  # noqa: E402


def _declared_functions(*headers):
    names = set()
    for header in headers or (HEADER, TUNING_HEADER):
        text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
        names |= set(re.findall(r"\b(onebit_sparse_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_native.LIB_PATH)
    declared = _declared_functions()
    assert "onebit_sparse_matmul" in declared and len(declared) >= 8
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert sorted(_native.EXPORTS) == declared
    # objects compiled against the reference's C++ header link against the mangled name
    assert hasattr(lib, "_Z20onebit_sparse_matmulPvS_S_S_S_iii")


def test_drop_in_header_holds_no_hooks_or_diagnostics():
    """what a maintainer of the reference installs declares the product's entry points only"""
    product = _declared_functions(HEADER)
    assert not [n for n in product if "_set_tile" in n or "_set_skinny" in n or "_set_split" in n or "_set_pad" in n
                or "describe" in n or "measure" in n or "device_info" in n]
    assert "onebit_sparse_matmul" in product and "onebit_sparse_matmul_prepared_static" in product


@pytest.mark.parametrize("header", ["onebit_sparse_tensor.h", "onebit_sparse_tuning.h"])
def test_header_is_plain_c(header):
    src = f'#include "{header}"\nint main(void){{return onebit_sparse_prepared_bytes(64,32)==0;}}\n'
    out = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                          "-x", "c", "-"], input=src.encode(), capture_output=True)
    assert out.returncode == 0, out.stderr.decode()


def test_prepared_bytes():
    lib = _native.lib()
    assert lib.onebit_sparse_prepared_bytes(64, 32) == 2 * 1 * 1536
    assert lib.onebit_sparse_prepared_bytes(8192, 8192) == 8192 * 8192 * 3 // 16   # 1.5 bits per weight
    assert lib.onebit_sparse_prepared_bytes(11008, 4096) == 11008 * 4096 * 3 // 16
    assert lib.onebit_sparse_prepared_bytes(0, 32) == 0


@pytest.mark.parametrize("m,n,k", [(10, 10, 10), (64, 8, 16), (32, 8, 32), (64, 0, 32), (-64, 8, 32), (64, 8, 48)])
def test_shape_validation(m, n, k):
    lib = _native.lib()
    fake = ctypes.c_void_p(0x1000)
    rc = lib.onebit_sparse_matmul_ex(fake, fake, fake, fake, fake, m, n, k, 1.0, 0.0, 0, 0, 0, None)
    assert rc == 1
    assert _native.last_error() != ""
    rc = lib.onebit_sparse_matmul_prepared(fake, fake, fake, fake, m, n, k, 1.0, 0.0, 0, 0, None)
    assert rc == 1


def test_argument_validation():
    lib = _native.lib()
    fake = ctypes.c_void_p(0x1000)
    assert lib.onebit_sparse_matmul_ex(None, fake, fake, fake, fake, 64, 8, 32, 1.0, 0.0, 0, 0, 0, None) == 1
    assert lib.onebit_sparse_matmul_ex(fake, fake, None, fake, fake, 64, 8, 32, 1.0, 1.0, 0, 0, 0, None) == 1  # beta, no C
    assert lib.onebit_sparse_matmul_ex(fake, fake, fake, fake, fake, 64, 8, 32, 1.0, 0.0, 2, 0, 0, None) == 1   # dtype
    assert lib.onebit_sparse_matmul_ex(fake, fake, fake, fake, fake, 64, 8, 32, 1.0, 0.0, 0, 0, 7, None) == 1   # layout
    assert lib.onebit_sparse_prepare(fake, fake, 64, 32, 0, None, None) == 1
    assert lib.onebit_sparse_prepare(fake, fake, 64, 32, 3, fake, None) == 1
    assert "layout" in _native.last_error()


def test_offset_limits_are_refused_with_a_message():
    """shapes beyond the kernels' 32-bit offsets are refused before anything is launched (no GPU needed)"""
    lib = _native.lib()
    fake = ctypes.c_void_p(0x1000)
    m, k = 1 << 20, 1 << 15                      # 32768 row blocks x 128 chunks x 1536 bytes = 6 GiB of prepared operand
    assert _native.prepared_bytes(m, k) >= 1 << 32
    assert lib.onebit_sparse_matmul_prepared(fake, fake, fake, fake, m, 128, k, 1.0, 0.0, 0, 0, None) == 1
    assert "4 GiB" in _native.last_error()
    assert lib.onebit_sparse_linear_prepared(fake, fake, None, fake, 128, m, k, 1, 1, None) == 1
    assert "4 GiB" in _native.last_error()
    assert lib.onebit_sparse_matmul_prepared_static(fake, fake, fake, fake, m, 128, k, 1.0, 0.0, 0, 0, None) in (1, 2)
    # the token-major form addresses a tile's token rows with 32-bit offsets: k is limited
    assert lib.onebit_sparse_linear_prepared(fake, fake, None, fake, 128, 64, 1 << 23, 1, 1, None) == 1
    assert "token-major" in _native.last_error()
    # x must be 16-byte aligned
    assert lib.onebit_sparse_linear_prepared(fake, ctypes.c_void_p(0x1008), None, fake, 8, 64, 64, 1, 1, None) == 1
    assert "aligned" in _native.last_error()


@pytest.mark.skipif(torch.cuda.is_available(), reason="needs a host without a GPU (pointers are fake)")
def test_no_device_is_reported_not_fatal():
    lib = _native.lib()
    fake = ctypes.c_void_p(0x1000)
    rc = lib.onebit_sparse_matmul_ex(fake, fake, fake, fake, fake, 64, 8, 32, 1.0, 0.0, 0, 0, 0, None)
    assert rc == 2
    assert "HIP error" in _native.last_error()


def test_legacy_symbol_exits_on_error():
    """csrc/kernel_lib.cu:11-20: print one line to stderr and exit(EXIT_FAILURE)."""
    code = ("import ctypes,sys; L=ctypes.CDLL(sys.argv[1]); p=ctypes.c_void_p(0x1000);"
            "L.onebit_sparse_matmul(p,p,p,p,p,10,10,10); print('survived')")
    out = subprocess.run([sys.executable, "-c", code, _native.LIB_PATH], capture_output=True, text=True)
    assert out.returncode == 1
    assert "survived" not in out.stdout
    assert "onebit_sparse_matmul error" in out.stderr


def test_python_wrappers_reject_host_tensors():
    a = torch.zeros(16, 8, dtype=torch.uint8)
    meta = torch.zeros(64, 2, dtype=torch.int16)
    with pytest.raises(ValueError):
        _native.prepare(a, meta, 64, 32)


def test_binding_module_loads_and_validates():
    from onebitsparsemul_amd import onebit_sparse_cuda
    assert onebit_sparse_cuda.onebit_mul.__doc__.strip().endswith("A32 = Sparse W1 * A16 matmul.")
    a = torch.zeros(16, 8, dtype=torch.uint8)
    b = torch.zeros(32, 8, dtype=torch.float16)
    meta = torch.zeros(64, 2, dtype=torch.int16)
    c = torch.zeros(64, 8, dtype=torch.float32)
    with pytest.raises(RuntimeError):
        onebit_sparse_cuda.onebit_mul(a, b, meta, c)  # host tensors are rejected, nothing is computed on the CPU


@pytest.fixture
def _default_hooks():
    def reset():
        _native.set_tile_config(-1)
        _native.set_skinny_enabled(True)
        _native.set_skinny_rows(-1)
        _native.set_split_k(-1)
        _native.set_pad_b(True)
    reset()
    yield
    reset()


def test_launch_plan_of_the_benchmark_shapes(_default_hooks):
    """kernel choice of the C ABI (host logic, no GPU): the five benchmark configurations and the cases around them"""
    plan = _native.describe_launch
    # large squares: at least one round of 512 x 128 tiles, which then run on the 16x16x64 SMFMAC with one wavefront per
    # SIMD (code 15); one pass, B read in place
    for size in (4096, 8192, 16384, 25600):
        assert plan(size, size, size) == dict(kernel="gemm_kernel", tile=15, splits=1, pad_b=False)
    assert plan(28672, 512, 8192)["tile"] == 15                                                   # 224 tiles: 0.875 of a round
    # a last round of 512 x 128 tiles that would be mostly empty: 256 x 128 on four wavefronts (code 4)
    assert plan(6144, 6144, 6144)["tile"] == 4 and plan(11008, 2048, 4096)["tile"] == 4
    # the prefill shape has one 256 x 128 tile per CU: its eight-wavefront form (code 10)
    assert plan(4096, 2048, 4096) == dict(kernel="gemm_kernel", tile=10, splits=1, pad_b=False)
    # small squares: 128 x 128 / 64 x 128 tiles, no K split
    assert plan(2048, 2048, 2048) == dict(kernel="gemm_kernel", tile=13, splits=1, pad_b=False)   # two K groups
    assert plan(512, 512, 512) == dict(kernel="gemm_kernel", tile=12, splits=1, pad_b=False)
    # decode shapes: the split-K kernel, row group by M
    for n in (1, 4, 16):
        assert plan(11008, n, 4096) == dict(kernel="skinny_kernel", rows=64, splits=1)
        assert plan(4096, n, 11008) == dict(kernel="skinny_kernel", rows=32, splits=1)
    assert plan(28672, 16, 8192) == dict(kernel="skinny_kernel", rows=128, splits=1)
    assert plan(28672, 32, 8192) == dict(kernel="skinny_kernel", rows=128, splits=1)
    assert plan(16384, 32, 4096) == dict(kernel="skinny_kernel", rows=64, splits=1)
    assert plan(4096, 64, 4096) == dict(kernel="skinny_kernel", rows=32, splits=1)
    assert plan(11008, 64, 4096) == dict(kernel="skinny_kernel", rows=64, splits=1)   # 33 ... 64 columns: at most 64 rows
    assert plan(28672, 64, 8192) == dict(kernel="skinny_kernel", rows=64, splits=1)
    # few row groups over a long K: K split over workgroups as well, one workgroup per compute unit, 64-row groups
    assert plan(4096, 16, 16384) == dict(kernel="skinny_kernel", rows=64, splits=4)
    assert plan(2048, 16, 28672) == dict(kernel="skinny_kernel", rows=64, splits=8)
    assert plan(8192, 16, 28672) == dict(kernel="skinny_kernel", rows=64, splits=2)
    assert plan(8192, 64, 8192) == dict(kernel="skinny_kernel", rows=64, splits=2)
    assert plan(11008, 32, 28672) == dict(kernel="skinny_kernel", rows=128, splits=2)   # 64 rows: 172 groups, no room
    assert plan(4096, 16, 11008) == dict(kernel="skinny_kernel", rows=32, splits=1)     # B too small to pay for it
    assert plan(8192, 16, 16384) == dict(kernel="skinny_kernel", rows=32, splits=1)
    assert plan(65536, 64, 8192)["kernel"] == "gemm_kernel"      # from about 48k rows on the main kernel is faster
    assert plan(4096, 65, 4096)["kernel"] == "gemm_kernel"
    # fewer than 256 tiles of 512 x 128: tile and split from the cost model
    assert plan(4096, 3072, 4096) == dict(kernel="gemm_kernel", tile=9, splits=1, pad_b=False)    # 192 large tiles: eight wavefronts
    assert plan(4096, 1536, 4096) == dict(kernel="gemm_kernel", tile=10, splits=1, pad_b=False)   # 192 of 256 x 128
    assert plan(11008, 768, 4096)["tile"] == 9 and plan(28672, 192, 8192)["tile"] == 10
    assert plan(4096, 384, 11008) == dict(kernel="gemm_kernel", tile=13, splits=2, pad_b=False)   # 96 tiles, 43 chunks
    assert plan(4096, 512, 4096) == dict(kernel="gemm_kernel", tile=14, splits=1, pad_b=False)    # 64 x 128, two K groups
    # few tiles over a long K: split over workgroups; many tiles: never
    few = plan(4096, 128, 4096)
    assert few["kernel"] == "gemm_kernel" and few["splits"] > 1
    assert plan(4096, 256, 11008)["splits"] > 1
    # B rows that are not 16-byte aligned: padded copy, except for tiny operands
    assert plan(4096, 1001, 4096)["pad_b"] is True
    assert plan(4096, 1000, 4096, b_aligned=False)["pad_b"] is True
    assert plan(4096, 1000, 4096)["pad_b"] is False
    assert plan(256, 72, 128, b_aligned=False)["pad_b"] is False


def test_hooks_act_on_the_calling_thread_only(_default_hooks):
    """a hook set on one thread leaves the launches of every other thread alone"""
    import threading
    _native.set_skinny_enabled(False)
    _native.set_tile_config(4)
    seen = {}

    def worker():
        seen["plan"] = _native.describe_launch(11008, 16, 4096)
        _native.set_skinny_rows(32)  # stays in the worker
        seen["own"] = _native.describe_launch(28672, 16, 8192)

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert seen["plan"] == dict(kernel="skinny_kernel", rows=64, splits=1)     # the defaults, not this thread's hooks
    assert seen["own"] == dict(kernel="skinny_kernel", rows=32, splits=1)
    assert _native.describe_launch(11008, 16, 4096)["kernel"] == "gemm_kernel"  # this thread's hooks still hold
    _native.set_skinny_enabled(True)
    _native.set_tile_config(-1)
    assert _native.describe_launch(28672, 16, 8192) == dict(kernel="skinny_kernel", rows=128, splits=1)


def test_launch_plan_scales_with_the_compute_units(_default_hooks):
    """the explicit-count form plans for a smaller or partitioned GPU: fewer resident workgroups, other row groups"""
    full = _native.describe_launch(28672, 16, 8192, compute_units=256)
    small = _native.describe_launch(28672, 16, 8192, compute_units=64)
    assert full == dict(kernel="skinny_kernel", rows=128, splits=1) and small["kernel"] == "skinny_kernel"
    assert _native.describe_launch(2048, 16, 28672, compute_units=64)["splits"] <= 2   # one workgroup per compute unit
    lib = _native.lib()
    out = (ctypes.c_int * 4)()
    assert lib.onebit_sparse_describe_launch_for(64, 8, 32, 1, 0, out) == 1
    assert "compute_units" in _native.last_error()


def test_launch_plan_follows_the_hooks(_default_hooks):
    plan = _native.describe_launch
    _native.set_skinny_enabled(False)
    assert plan(11008, 16, 4096)["kernel"] == "gemm_kernel"
    _native.set_skinny_enabled(True)
    _native.set_skinny_rows(32)
    assert plan(28672, 16, 8192) == dict(kernel="skinny_kernel", rows=32, splits=1)
    _native.set_tile_config(4)
    _native.set_split_k(3)
    assert plan(8192, 8192, 8192) == dict(kernel="gemm_kernel", tile=4, splits=3, pad_b=False)
    _native.set_split_k(1000)
    assert plan(8192, 8192, 8192)["splits"] == 32          # at most one split per 256 of K
    _native.set_pad_b(False)
    assert plan(4096, 1001, 4096)["pad_b"] is False


def test_describe_launch_validates():
    lib = _native.lib()
    out = (ctypes.c_int * 4)()
    assert lib.onebit_sparse_describe_launch(60, 8, 32, 1, out) == 1
    assert lib.onebit_sparse_describe_launch(64, 8, 32, 1, None) == 1


def test_python_side_size_formula_matches_the_library():
    for m, k in ((64, 32), (64, 256), (96, 288), (4096, 11008), (28672, 8192)):
        assert _native._prepared_bytes_fast(m, k) == _native.prepared_bytes(m, k)
