"""A compiled C++ consumer of the boundary, the counterpart of the reference's link test (tests/libso_test.cu:3-22,
built by makefile:22-23 with -lonebitmul): tests/consumer/libso_test.cpp declares onebit_sparse_matmul as the
reference's header does (include/onebit_sparse_tensor.h:5, C++ linkage), so linking it proves that libonebitmul.so
resolves the C++-mangled name, and running it multiplies real operands through that symbol.

Without a GPU: the program compiles and links against the library, and its only undefined onebit symbol is the mangled
one. With a GPU (-m gpu): the prebuilt program (onebitsparsemul_amd.build.build_consumer, part of build()) runs a
512^3 product with integer B and its output file equals the oracle's host GEMM bit for bit."""
import os
import subprocess

import numpy as np
import pytest

import oracle
from onebitsparsemul_amd import build as native_build
from onebitsparsemul_amd import synthetic

MANGLED = "_Z20onebit_sparse_matmulPvS_S_S_S_iii"


def test_consumer_compiles_and_links_against_the_mangled_symbol(tmp_path):
    out = native_build.build_consumer(str(tmp_path / "libso_test"))
    undefined = subprocess.run(["nm", "-D", "--undefined-only", out], capture_output=True, text=True, check=True).stdout
    onebit = [line.split()[-1] for line in undefined.splitlines() if "onebit" in line]
    assert onebit == [MANGLED], onebit
    defined = subprocess.run(["nm", "-D", "--defined-only", native_build.LIB], capture_output=True, text=True,
                             check=True).stdout
    assert any(line.split()[-1] == MANGLED for line in defined.splitlines())


@pytest.mark.gpu
def test_consumer_runs_and_matches_the_oracle(tmp_path):
    binary = native_build.CONSUMER_BIN
    assert os.path.exists(binary), f"{binary} is missing: run `python -m onebitsparsemul_amd.build`"
    m = n = k = 512
    a, meta = synthetic.make_weight(m, k, seed=0x0B5A0006)
    b = synthetic.make_b(k, n, seed=6, kind="int")
    paths = {name: str(tmp_path / f"{name}.bin") for name in ("a", "b", "e", "d")}
    a.numpy().tofile(paths["a"])
    b.numpy().tofile(paths["b"])
    meta.numpy().tofile(paths["e"])
    run = subprocess.run([binary, str(m), str(n), str(k), paths["a"], paths["b"], paths["e"], paths["d"]],
                         capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stderr
    got = np.fromfile(paths["d"], dtype=np.float32).reshape(m, n)
    want = oracle.reference_matmul(a.numpy(), b.numpy(), meta.numpy(), m, n, k, d_dtype=oracle.F32)
    assert np.array_equal(got, want)
    assert run.stdout.strip() == f"sum {float(want.astype(np.float64).sum()):.1f}"
