"""Linear-layer form of the prepared product (token-major x and y, fused bias) against the oracle."""
import numpy as np
import pytest
import torch

import oracle
from onebitsparsemul_amd import _native, synthetic

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _defaults():
    _native.set_tile_config(-1)
    _native.set_skinny_enabled(True)
    _native.set_skinny_rows(-1)
    _native.set_split_k(-1)
    yield
    _native.set_tile_config(-1)
    _native.set_skinny_enabled(True)
    _native.set_skinny_rows(-1)
    _native.set_split_k(-1)


def _expected(dense, x, bias, y_dtype):
    """y = (W x^T)^T + bias with the oracle's host GEMM (fp32 accumulation; exact for small integers)."""
    d = oracle.host_gemm(dense, np.ascontiguousarray(x.T), d_dtype=oracle.F32, acc="f32").T
    if bias is not None:
        d = d + bias.astype(np.float32)[None, :]
    return d.astype(y_dtype)


@pytest.mark.parametrize("rows", [-1, 32, 64, 128])
@pytest.mark.parametrize("tokens", [1, 5, 16, 17, 32, 33, 64])
@pytest.mark.parametrize("m,k", [(256, 512), (192, 1056), (1024, 4096), (448, 8480)])
def test_linear_form_small_token_counts(rows, tokens, m, k):
    _native.set_skinny_rows(rows)
    a, meta = synthetic.make_weight(m, k, seed=m + k + tokens)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), m, k)
    x = synthetic.make_b(tokens, k, seed=tokens, kind="int")           # (tokens, k) small integers
    bias = synthetic.make_b(1, m, seed=tokens + 1, kind="int").reshape(m)
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    for y_dtype, b in ((torch.float32, bias), (torch.float16, None), (torch.float16, bias.float())):
        y = torch.full((tokens, m), float("nan"), dtype=y_dtype, device="cuda")
        _native.linear_prepared(prep, x.cuda(), y, m, k, bias=b.cuda() if b is not None else None)
        torch.cuda.synchronize()
        want = _expected(dense, x.numpy().astype(np.float32), b.numpy() if b is not None else None,
                         np.float32 if y_dtype == torch.float32 else np.float16)
        assert np.array_equal(y.cpu().numpy(), want), (y_dtype, b is not None)


@pytest.mark.parametrize("tile", [-1, 4, 6, 9, 10, 11, 12, 13, 14, 15])
@pytest.mark.parametrize("tokens,m,k", [(65, 256, 512), (128, 192, 1056), (200, 1024, 2048), (1000, 640, 544), (16, 256, 800),
                                        (520, 4096, 512)])
def test_linear_form_main_kernel(tile, tokens, m, k):
    _native.set_tile_config(tile)
    _native.set_skinny_enabled(False)
    a, meta = synthetic.make_weight(m, k, seed=m + k + tokens)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), m, k)
    x = synthetic.make_b(tokens, k, seed=tokens, kind="int")
    bias = synthetic.make_b(1, m, seed=tokens + 1, kind="int").reshape(m)
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    for y_dtype, b in ((torch.float32, bias), (torch.float16, None), (torch.float16, bias.float())):
        y = torch.full((tokens, m), float("nan"), dtype=y_dtype, device="cuda")
        _native.linear_prepared(prep, x.cuda(), y, m, k, bias=b.cuda() if b is not None else None)
        torch.cuda.synchronize()
        want = _expected(dense, x.numpy().astype(np.float32), b.numpy() if b is not None else None,
                         np.float32 if y_dtype == torch.float32 else np.float16)
        assert np.array_equal(y.cpu().numpy(), want), (y_dtype, b is not None)


@pytest.mark.parametrize("splits", [-1, 2, 3, 16])
@pytest.mark.parametrize("tokens,m,k", [(128, 256, 4096), (72, 192, 2080), (264, 1024, 1024)])
def test_linear_form_k_split_over_workgroups(splits, tokens, m, k):
    _native.set_split_k(splits)
    _native.set_skinny_enabled(False)
    a, meta = synthetic.make_weight(m, k, seed=splits + m + k)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), m, k)
    x = synthetic.make_b(tokens, k, seed=tokens, kind="int")
    bias = synthetic.make_b(1, m, seed=tokens + 1, kind="int").reshape(m)
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    for y_dtype, b in ((torch.float32, bias), (torch.float16, None), (torch.float16, bias.float())):
        y = torch.full((tokens, m), float("nan"), dtype=y_dtype, device="cuda")
        _native.linear_prepared(prep, x.cuda(), y, m, k, bias=b.cuda() if b is not None else None)
        torch.cuda.synchronize()
        want = _expected(dense, x.numpy().astype(np.float32), b.numpy() if b is not None else None,
                         np.float32 if y_dtype == torch.float32 else np.float16)
        assert np.array_equal(y.cpu().numpy(), want), (y_dtype, b is not None)
    # result 2 bytes past a 16-byte boundary: the element form of the reduction
    store = torch.full((tokens * m + 1,), float("nan"), dtype=torch.float16, device="cuda")
    y = store[1:].view(tokens, m)
    _native.linear_prepared(prep, x.cuda(), y, m, k, bias=bias.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), _expected(dense, x.numpy().astype(np.float32), bias.numpy(), np.float16))


@pytest.mark.parametrize("tokens", [8, 300])
def test_linear_form_result_not_16_byte_aligned(tokens):
    m, k = 320, 1024
    a, meta = synthetic.make_weight(m, k, seed=3)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), m, k)
    x = synthetic.make_b(tokens, k, seed=4, kind="int")
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    store = torch.full((tokens * m + 1,), float("nan"), dtype=torch.float16, device="cuda")
    y = store[1:].view(tokens, m)  # 2 bytes past a 16-byte boundary
    _native.linear_prepared(prep, x.cuda(), y, m, k)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), _expected(dense, x.numpy().astype(np.float32), None, np.float16))
    # aligned result, bias 2 bytes past a 16-byte boundary
    bias = synthetic.make_b(1, m + 1, seed=5, kind="int").reshape(m + 1).cuda()[1:]
    y2 = torch.full((tokens, m), float("nan"), dtype=torch.float16, device="cuda")
    _native.linear_prepared(prep, x.cuda(), y2, m, k, bias=bias)
    torch.cuda.synchronize()
    assert np.array_equal(y2.cpu().numpy(), _expected(dense, x.numpy().astype(np.float32), bias.cpu().numpy(), np.float16))


def test_linear_form_rejects_misaligned_x():
    m, k, tokens = 64, 256, 4
    a, meta = synthetic.make_weight(m, k, seed=3)
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    store = torch.zeros(tokens * k + 1, dtype=torch.float16, device="cuda")
    y = torch.empty((tokens, m), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        _native.linear_prepared(prep, store[1:].view(tokens, k), y, m, k)


@pytest.mark.parametrize("lead", [(7,), (3, 70), (2, 2, 9)])
@pytest.mark.parametrize("x_dtype", [torch.float16, torch.float32])
def test_layer_forward_with_bias(lead, x_dtype):
    """BinaryLinear_2_4.forward goes through the linear form: any leading shape, fp16 or fp32 activations, bias fused"""
    import onebitsparsemul_amd as ob
    out_f, in_f = 640, 512
    torch.manual_seed(0)
    layer = ob.BinaryLinear_2_4(in_f, out_f)
    layer.pack(torch.randn(out_f, in_f).half())
    layer.bias = torch.randint(-3, 4, (out_f,)).to(torch.float16)
    x = torch.randint(-4, 5, lead + (in_f,)).to(x_dtype)
    want = ob.py_binary_gemm(x.reshape(-1, in_f).float(), layer.packed_binary_sparse, layer.meta) + layer.bias.float()
    layer = layer.cuda()
    layer.bias = layer.bias.cuda()
    got = layer(x.cuda())
    torch.cuda.synchronize()
    assert got.dtype == x_dtype and tuple(got.shape) == lead + (out_f,)
    assert torch.equal(got.cpu().float().reshape(-1, out_f), want)
    # a view that does not start on a 16-byte boundary
    store = torch.zeros(x.numel() + 1, dtype=torch.float16, device="cuda")
    store[1:] = x.reshape(-1).cuda().half()
    got2 = layer(store[1:].view(*lead, in_f))
    assert torch.equal(got2.cpu().float().reshape(-1, out_f), want)


def test_linear_form_at_8192_identity_and_linearity():
    """full size: x = I returns the transposed decompressed weight exactly; linearity on integer tokens, exact"""
    m = k = tokens = 8192
    a, meta = synthetic.make_weight(m, k, seed=0x0B5A0200)
    dense = torch.from_numpy(oracle.decompress_operands(a.numpy(), meta.numpy(), m, k))
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    eye = torch.eye(k, dtype=torch.float16, device="cuda")
    y = torch.empty((tokens, m), dtype=torch.float16, device="cuda")
    _native.linear_prepared(prep, eye, y, m, k)
    torch.cuda.synchronize()
    del eye
    assert torch.equal(y.to(torch.int8), dense.cuda().T)
    x1 = synthetic.make_b(tokens, k, seed=1, kind="int", device="cuda")
    x2 = synthetic.make_b(tokens, k, seed=2, kind="int", device="cuda")
    outs = []
    for x in (x1, x2, x1 + x2):
        o = torch.empty((tokens, m), dtype=torch.float32, device="cuda")
        _native.linear_prepared(prep, x, o, m, k)
        outs.append(o)
    torch.cuda.synchronize()
    assert torch.equal(outs[0] + outs[1], outs[2])
    # and equal to the plain form on the transposed operand
    d = torch.empty((m, tokens), dtype=torch.float32, device="cuda")
    _native.matmul_prepared(prep, x1.T.contiguous(), d, m, tokens, k)
    torch.cuda.synchronize()
    assert torch.equal(d.T, outs[0])


@pytest.mark.parametrize("tokens,m,k", [(16, 1024, 2048), (300, 512, 512), (128, 256, 8192)])
def test_linear_form_in_a_hip_graph(tokens, m, k):
    """the layer's call captured in a HIP graph (after one eager call on the capture stream, which sizes the K-split
    buffer): every replay, with new activations written in between, equals the eager result; split-K kernel, main
    kernel, and its K split over workgroups"""
    a, meta = synthetic.make_weight(m, k, seed=m + tokens)
    prep = _native.prepare(a.cuda(), meta.cuda(), m, k)
    bias = synthetic.make_b(1, m, seed=3, kind="int").reshape(m).cuda()
    x = torch.zeros((tokens, k), dtype=torch.float16, device="cuda")
    y = torch.zeros((tokens, m), dtype=torch.float32, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())  # prep, bias, x and y were produced on the current stream
    with torch.cuda.stream(stream):
        _native.linear_prepared(prep, x, y, m, k, bias=bias)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            _native.linear_prepared(prep, x, y, m, k, bias=bias)
    for replay in range(4):
        values = synthetic.make_b(tokens, k, seed=100 + replay, kind="int").cuda()
        x.copy_(values)
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(y)
        _native.linear_prepared(prep, values, eager, m, k, bias=bias)
        torch.cuda.synchronize()
        assert torch.equal(y, eager) and bool(torch.isfinite(y).all())


def test_layer_forward_of_an_empty_batch():
    import onebitsparsemul_amd as ob
    layer = ob.BinaryLinear_2_4(64, 128)
    layer.pack(torch.randn(128, 64).half())
    layer = layer.cuda()
    out = layer(torch.empty((0, 64), dtype=torch.float16, device="cuda"))
    assert tuple(out.shape) == (0, 128) and out.dtype == torch.float16
    out = layer(torch.empty((2, 0, 64), dtype=torch.float16, device="cuda"))
    assert tuple(out.shape) == (2, 0, 128)


def test_layer_result_dtype_follows_the_activations():
    """float16 activations: float16 result; other activation dtypes (and out_dtype=float32): the kernel's fp32 result,
    so sums beyond float16's range survive. Integer operands: exact against the oracle."""
    import onebitsparsemul_amd as ob
    in_f, out_f, tokens = 2048, 256, 9
    a, meta = synthetic.make_weight(out_f, in_f, seed=77)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), out_f, in_f)
    x = synthetic.make_b(tokens, in_f, seed=78, kind="int").float() * 256.0  # sums of 1024 terms of up to 2048: beyond 65504
    want = _expected(dense, x.numpy(), None, np.float32)
    assert np.abs(want).max() > 65504.0
    for out_dtype, x_dtype, got_dtype in ((None, torch.float32, torch.float32), (None, torch.bfloat16, torch.bfloat16),
                                          (torch.float32, torch.float16, torch.float32)):
        layer = ob.BinaryLinear_2_4(in_f, out_f, out_dtype=out_dtype)
        layer.packed_binary_sparse, layer.meta, layer.vaild = a, meta, True
        layer = layer.cuda()
        got = layer(x.to(x_dtype).cuda())
        torch.cuda.synchronize()
        assert got.dtype == got_dtype
        if got_dtype == torch.float32:
            assert np.array_equal(got.cpu().numpy(), want)
        else:  # the fp32 sums rounded once to the activation dtype
            assert torch.equal(got.cpu(), torch.from_numpy(want).to(got_dtype))
    # float16 in, float16 out (the default): the same sums overflow to infinity, as a float16 result must
    layer = ob.BinaryLinear_2_4(in_f, out_f)
    layer.packed_binary_sparse, layer.meta, layer.vaild = a, meta, True
    got = layer.cuda()(x.half().cuda())
    assert got.dtype == torch.float16 and torch.equal(got.cpu(), torch.from_numpy(want).half())


def test_one_call_entry_points_reject_wrong_sized_operands():
    m, n, k = 128, 8, 64
    a, meta = synthetic.make_weight(m, k, seed=1)
    b = synthetic.make_b(k, n, seed=2, kind="int")
    ad, md, bd = a.cuda(), meta.cuda(), b.cuda()
    d = torch.empty((m, n), dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError):
        _native.matmul_ex(ad[:-1].contiguous(), bd, md, d, m, n, k)          # A too small
    with pytest.raises(ValueError):
        _native.matmul_ex(ad, bd, md[:, :-1].contiguous(), d, m, n, k)       # metadata too small
    with pytest.raises(ValueError):
        _native.matmul_ex(ad, bd, md, d[:-1], m, n, k)                       # D too small
    with pytest.raises(ValueError):
        _native.matmul_ex(ad, bd, md.view(torch.uint8), d, m, n, k)          # metadata of the wrong dtype
    with pytest.raises(ValueError):
        _native.matmul_legacy(ad, bd, d, d[:-1], md, m, n, k)
    with pytest.raises(TypeError):
        _native.matmul_legacy(ad, bd, d.half(), d.half(), md, m, n, k)       # the 8-argument symbol is fp32 only
    _native.matmul_ex(ad, bd, md, d, m, n, k)
    torch.cuda.synchronize()
    assert np.array_equal(d.cpu().numpy(), oracle.reference_matmul(a.numpy(), b.numpy(), meta.numpy(), m, n, k, d_dtype=oracle.F32))
