"""The entry point that allocates nothing (onebit_sparse_matmul_prepared_static) against the entry point it is a
variant of (onebit_sparse_matmul_prepared), through the C ABI.

Both run the same kernels with the same plan, so the results must be identical bit for bit, for integer and for
N(0,1) operands alike; the shapes are chosen so that the two internal buffers (fp32 partial sums of a K split, the
padded copy of B) are both in use, the second call is smaller than the first (it sees what the first left in the
array), and the first call is also checked against the CPU oracle.
"""
import numpy as np
import pytest
import torch

import oracle
from onebitsparsemul_amd import _native, synthetic

pytestmark = pytest.mark.gpu


def _both(prep, b, m, n, k, c=None, alpha=1.0, beta=0.0, dtype=torch.float16):
    want = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    got = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    _native.matmul_prepared(prep, b, want, m, n, k, c=c, alpha=alpha, beta=beta)
    _native.matmul_prepared(prep, b, got, m, n, k, c=c, alpha=alpha, beta=beta, static_scratch=True)
    torch.cuda.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


def test_two_calls_in_a_row_second_smaller():
    for hook in (_native.set_tile_config, _native.set_skinny_rows, _native.set_split_k):
        hook(-1)
    _native.set_skinny_enabled(True)
    _native.set_pad_b(True)
    # (m, n, k): K split over workgroups and a padded copy of B in the first two, the split-K kernel with a K split over
    # workgroups in the third, a split of the main kernel alone in the fourth, no buffer at all in the last
    shapes = ((2048, 130, 8192), (1024, 100, 8192), (2048, 16, 16384), (512, 72, 4096), (1024, 16, 4096))
    plans = [_native.describe_launch(m, n, k) for (m, n, k) in shapes]
    assert plans[0]["splits"] > 1 and plans[0]["pad_b"] and plans[1]["splits"] > 1 and plans[1]["pad_b"]
    assert plans[2]["kernel"] == "skinny_kernel" and plans[2]["splits"] > 1   # the split-K kernel's own K split
    assert plans[3]["splits"] > 1 and plans[4] == dict(kernel="skinny_kernel", rows=32, splits=1)
    for kind in ("int", "normal"):
        for i, (m, n, k) in enumerate(shapes):
            a, meta = synthetic.make_weight(m, k, seed=40 + i)
            b = synthetic.make_b(k, n, seed=50 + i, kind=kind)
            c = synthetic.make_c(m, n, seed=60 + i)
            prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
            got, want = _both(prep, b.cuda(), m, n, k)
            assert np.array_equal(got, want), f"{kind} {(m, n, k)}"
            got2, want2 = _both(prep, b.cuda(), m, n, k, c=c.cuda(), alpha=0.5, beta=1.0, dtype=torch.float32)
            assert np.array_equal(got2, want2), f"{kind} {(m, n, k)} epilogue"
            if kind == "int":
                ref = oracle.reference_matmul(a.numpy(), b.numpy(), meta.numpy(), m, n, k, d_dtype=oracle.F16)
                assert np.array_equal(got, ref), f"oracle {(m, n, k)}"


def test_refuses_shapes_beyond_the_static_workspace():
    _native.set_split_k(-1)
    m, n, k = 8192, 520, 8192
    _native.set_split_k(8)  # 8 x 8192 x 520 x 4 bytes = 136 MB of partial sums
    try:
        prep = torch.zeros(_native.prepared_bytes(m, k), dtype=torch.uint8, device="cuda")
        b = torch.zeros((k, n), dtype=torch.float16, device="cuda")
        d = torch.zeros((m, n), dtype=torch.float16, device="cuda")
        with pytest.raises(RuntimeError, match="static workspace"):
            _native.matmul_prepared(prep, b, d, m, n, k, static_scratch=True)
        _native.matmul_prepared(prep, b, d, m, n, k)  # the allocating entry point takes the same shape
        torch.cuda.synchronize()
    finally:
        _native.set_split_k(-1)
