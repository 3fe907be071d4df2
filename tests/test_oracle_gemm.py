"""Pins the oracle's host GEMM and epilogue (oracle/onebit_oracle.c: ob_host_gemm, ob_reference_matmul) with
special cases that reduce to closed forms or to numpy, chosen so that a dropped term, a wrong sign, a wrong
position or a transposed operand fails at least one of them."""
import numpy as np
import pytest


def _operands_from_dense(oracle_lib, dense):
    sparse, meta = oracle_lib.sparse_from_dense(dense)
    bits = oracle_lib.binary_quant(sparse)
    a = oracle_lib.pack_binary(np.ascontiguousarray(bits.T))
    return a, meta


def _random_pm1_dense(rng, m, k):
    dense = np.zeros((m, k // 4, 4), dtype=np.float32)
    pick = np.array([(0, 1), (0, 2), (1, 2), (0, 3), (1, 3), (2, 3)])[rng.integers(0, 6, size=(m, k // 4))]
    np.put_along_axis(dense, pick, rng.choice([-1.0, 1.0], size=(m, k // 4, 2)).astype(np.float32), axis=-1)
    return dense.reshape(m, k)


def test_benchmark_dataset_closed_form(oracle_lib):
    """The reference benchmark's own data (tests/kernel_test.cu:302-306,398-400): every value bit 1 and every
    metadata element 0x4444 => A = repeat([1, 1, 0, 0]) => D[i, :] = sum of the rows t of B with t % 4 < 2."""
    m, n, k = 64, 24, 96
    a = np.full(m * k // 16, 0xFF, dtype=np.uint8)
    e = np.full((m, k // 16), 0x4444, dtype=np.int16)  # constant tensor: identical in every layout
    rng = np.random.default_rng(1)
    b = rng.integers(-8, 9, size=(k, n)).astype(np.float16)
    d = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32)
    want = b.astype(np.float64)[np.arange(k) % 4 < 2].sum(axis=0)
    assert np.array_equal(d, np.tile(want, (m, 1)).astype(np.float32))


def test_identity_b_returns_decompressed_a(oracle_lib):
    rng = np.random.default_rng(2)
    m, k = 64, 64
    dense = _random_pm1_dense(rng, m, k)
    a, e = _operands_from_dense(oracle_lib, dense)
    d = oracle_lib.reference_matmul(a, np.eye(k, dtype=np.float16), e, m, k, k, d_dtype=oracle_lib.F32)
    assert np.array_equal(d, dense)


def test_not_transposed_and_sign(oracle_lib):
    # one kept +1 at (row 3, col 5) and one kept -1 at (row 3, col 6) among a regular background
    m, k, n = 64, 32, 8
    dense = np.tile(np.array([1, 1, 0, 0], dtype=np.float32), (m, k // 4))
    dense[3, 4:8] = [0, 1, -1, 0]
    a, e = _operands_from_dense(oracle_lib, dense)
    b = np.zeros((k, n), dtype=np.float16)
    b[5, 2] = 3
    b[6, 2] = 10
    b[6, 7] = 1
    d = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32)
    want = dense.astype(np.float64) @ b.astype(np.float64)
    assert np.array_equal(d, want.astype(np.float32))
    assert d[3, 2] == 3 - 10 and d[3, 7] == -1 and d[0, 2] == 3 and d[0, 7] == 0


@pytest.mark.parametrize("m,n,k", [(64, 1, 32), (64, 5, 64), (128, 33, 160), (192, 64, 512)])
def test_against_numpy_small_integers_exact(oracle_lib, m, n, k):
    rng = np.random.default_rng(m + n + k)
    dense = _random_pm1_dense(rng, m, k)
    a, e = _operands_from_dense(oracle_lib, dense)
    b = rng.integers(-8, 9, size=(k, n)).astype(np.float16)
    want = dense.astype(np.float64) @ b.astype(np.float64)
    for acc in ("f32", "f64"):
        d32 = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32, acc=acc)
        assert np.array_equal(d32.astype(np.float64), want)
        d16 = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F16, acc=acc)
        assert np.array_equal(d16, want.astype(np.float16))


def test_normal_b_tolerance_and_epilogue(oracle_lib):
    rng = np.random.default_rng(9)
    m, n, k = 128, 48, 1024
    dense = _random_pm1_dense(rng, m, k)
    a, e = _operands_from_dense(oracle_lib, dense)
    b = rng.standard_normal((k, n)).astype(np.float16)
    c16 = rng.standard_normal((m, n)).astype(np.float16)
    c32 = rng.standard_normal((m, n)).astype(np.float32)
    exact = dense.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(exact).max()
    d = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32, acc="f32")
    assert np.abs(d - exact).max() <= 1e-5 * scale          # fp32 sequential accumulation of 512 terms
    d = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32, acc="f64")
    assert np.abs(d - exact).max() <= 1e-6 * scale
    for c in (c16, c32):
        want = 0.5 * exact + 1.0 * c.astype(np.float64)
        d = oracle_lib.reference_matmul(a, b, e, m, n, k, c=c, alpha=0.5, beta=1.0, d_dtype=oracle_lib.F32, acc="f64")
        assert np.abs(d - want).max() <= 1e-6 * scale
        d16 = oracle_lib.reference_matmul(a, b, e, m, n, k, c=c, alpha=0.5, beta=1.0, d_dtype=oracle_lib.F16, acc="f64")
        assert np.abs(d16.astype(np.float64) - want).max() <= 5e-4 * np.abs(want).max() + 1e-7
    # beta == 0: C is not read (NaNs in C must not leak)
    nan_c = np.full((m, n), np.nan, dtype=np.float32)
    d = oracle_lib.reference_matmul(a, b, e, m, n, k, c=nan_c, alpha=1.0, beta=0.0, d_dtype=oracle_lib.F32)
    assert np.isfinite(d).all()


def test_linearity_in_b(oracle_lib):
    rng = np.random.default_rng(4)
    m, n, k = 64, 16, 256
    dense = _random_pm1_dense(rng, m, k)
    a, e = _operands_from_dense(oracle_lib, dense)
    b1 = rng.integers(-4, 5, size=(k, n)).astype(np.float16)
    b2 = rng.integers(-4, 5, size=(k, n)).astype(np.float16)
    f = lambda b: oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32)
    assert np.array_equal(f(b1 + b2), f(b1) + f(b2))


def test_blas_helper_agrees(oracle_lib):
    rng = np.random.default_rng(6)
    m, n, k = 64, 40, 320
    dense = _random_pm1_dense(rng, m, k)
    a, e = _operands_from_dense(oracle_lib, dense)
    b = rng.integers(-8, 9, size=(k, n)).astype(np.float16)
    d = oracle_lib.reference_matmul(a, b, e, m, n, k, d_dtype=oracle_lib.F32)
    assert np.array_equal(oracle_lib.blas_matmul(oracle_lib.decompress_operands(a, e, m, k), b), d.astype(np.float64))
