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
    plans = [_native.describe_launch(m, n, k, compute_units=None) for (m, n, k) in shapes]  # for this GPU
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


def test_static_entry_point_is_capturable_without_a_warm_up():
    """A call that allocated would invalidate the capture: the non-allocating entry point is captured in a HIP graph
    with no eager call before it, on a shape that needs both internal buffers (K split over workgroups and a padded copy
    of B), and every replay equals the eager result of the allocating entry point."""
    for hook in (_native.set_tile_config, _native.set_skinny_rows, _native.set_split_k):
        hook(-1)
    m, n, k = 2048, 130, 8192
    plan = _native.describe_launch(m, n, k, compute_units=None)
    assert plan["splits"] > 1 and plan["pad_b"]
    a, meta = synthetic.make_weight(m, k, seed=71)
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    b = torch.zeros((k, n), dtype=torch.float16, device="cuda")
    d = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    # The entry point's first call on a device looks up the address of the static array (set-up, not an allocation);
    # that happens here, outside the capture, through a shape that uses no internal buffer at all.
    small = torch.zeros((64, 16), dtype=torch.float32, device="cuda")
    _native.matmul_prepared(torch.zeros(_native.prepared_bytes(64, 256), dtype=torch.uint8, device="cuda"),
                            torch.zeros((256, 16), dtype=torch.float16, device="cuda"), small, 64, 16, 256, static_scratch=True)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            _native.matmul_prepared(prep, b, d, m, n, k, static_scratch=True)
    for replay in range(3):
        values = synthetic.make_b(k, n, seed=200 + replay, kind="int").cuda()
        b.copy_(values)
        d.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(d)
        _native.matmul_prepared(prep, values, eager, m, n, k)
        torch.cuda.synchronize()
        assert torch.equal(d, eager) and bool(torch.isfinite(d).all())
    ref = oracle.reference_matmul(a.numpy(), values.cpu().numpy(), meta.numpy(), m, n, k, d_dtype=oracle.F32)
    assert np.array_equal(d.cpu().numpy(), ref)


def test_allocating_entry_point_refuses_to_grow_under_capture_and_release_buffers():
    """The allocating entry point cannot grow its buffers inside a capture: it refuses with a message, and the same call
    works afterwards outside. onebit_sparse_release_buffers frees the buffers; the next split call allocates them again
    and still matches the oracle."""
    for hook in (_native.set_tile_config, _native.set_skinny_rows, _native.set_split_k):
        hook(-1)
    m, n, k = 1024, 72, 8192
    assert _native.describe_launch(m, n, k, compute_units=None)["splits"] > 1
    a, meta = synthetic.make_weight(m, k, seed=72)
    bi = synthetic.make_b(k, n, seed=73, kind="int")
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    b = bi.cuda()
    d = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    ref = oracle.reference_matmul(a.numpy(), bi.numpy(), meta.numpy(), m, n, k, d_dtype=oracle.F32)
    torch.cuda.synchronize()
    _native.release_buffers()  # whatever earlier tests left: this stream's K-split buffer has to be allocated anew
    stream = torch.cuda.Stream()  # a fresh stream owns no library buffer yet
    refused = None
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            try:
                _native.matmul_prepared(prep, b, d, m, n, k)
            except RuntimeError as err:
                refused = str(err)
    assert refused is not None and "being captured" in refused
    del graph
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        _native.matmul_prepared(prep, b, d, m, n, k)  # the same call outside the capture allocates and runs
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy(), ref)
    _native.release_buffers()
    d.fill_(float("nan"))
    with torch.cuda.stream(stream):
        _native.matmul_prepared(prep, b, d, m, n, k)  # allocates again after the release
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy(), ref)


def test_weight_cache_refuses_a_miss_under_capture():
    """A weight that is not in the opt-in cache yet would have to be reordered into newly allocated memory: inside a
    capture the one-call entry point refuses with a message; after one call outside, the same call is captured, replayed
    and matches the oracle."""
    m, n, k = 256, 16, 512
    a, meta = synthetic.make_weight(m, k, seed=81)
    bi = synthetic.make_b(k, n, seed=82, kind="int")
    ad, md, bd = a.cuda(), meta.cuda(), bi.cuda()
    d = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    ref = oracle.reference_matmul(a.numpy(), bi.numpy(), meta.numpy(), m, n, k, d_dtype=oracle.F32)
    torch.cuda.synchronize()
    _native.set_weight_cache(2)
    try:
        stream = torch.cuda.Stream()
        refused = None
        with torch.cuda.stream(stream):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                try:
                    _native.matmul_ex(ad, bd, md, d, m, n, k)
                except RuntimeError as err:
                    refused = str(err)
        assert refused is not None and "being captured" in refused
        del graph
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            _native.matmul_ex(ad, bd, md, d, m, n, k)  # a miss outside the capture: reordered and cached
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                _native.matmul_ex(ad, bd, md, d, m, n, k)  # a hit: nothing to allocate
        d.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(d.cpu().numpy(), ref)
    finally:
        _native.set_weight_cache(0)
