"""The grouped linear-layer entry point (onebit_sparse_linear_prepared_grouped) through the C ABI: several products
y_i = x_i W_i^T + bias_i with one token count in one call, against the oracle (bit-exact on integer activations) and
against the single form (identical results). Covers the q / k / v case (one x, three weights), problems with different
m and k (the down projection next to gate / up), every row group, token counts of each image width, more problems
than one launch holds, and token counts beyond the split-K kernel's range (a sequence of single calls)."""
import numpy as np
import pytest
import torch

import oracle
from onebitsparsemul_amd import _native, synthetic

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _defaults():
    def reset():
        _native.set_tile_config(-1)
        _native.set_skinny_enabled(True)
        _native.set_skinny_rows(-1)
        _native.set_split_k(-1)
    reset()
    yield
    reset()


def _problem(m, k, tokens, seed, x=None, bias_dtype=torch.float16, y_dtype=torch.float16):
    a, meta = synthetic.make_weight(m, k, seed=seed)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), m, k)
    if x is None:
        x = synthetic.make_b(tokens, k, seed=seed + 1, kind="int")
    bias = synthetic.make_b(1, m, seed=seed + 2, kind="int").reshape(m).to(bias_dtype)
    want = (x.numpy().astype(np.float32) @ dense.astype(np.float32).T + bias.numpy().astype(np.float32)[None, :])
    want = want.astype(np.float16 if y_dtype == torch.float16 else np.float32)
    return dict(prep=_native.prepare(a.cuda(), meta.cuda(), m, k), x=x, bias=bias, want=want, m=m, k=k)


def _run(problems, tokens, y_dtype=torch.float16, shared_x=None):
    xs = [shared_x if shared_x is not None else p["x"].cuda() for p in problems]
    ys = [torch.full((tokens, p["m"]), float("nan"), dtype=y_dtype, device="cuda") for p in problems]
    _native.linear_prepared_grouped([(p["prep"], x, y, p["m"], p["k"], p["bias"].cuda() if p["bias"] is not None else None)
                                     for p, x, y in zip(problems, xs, ys)])
    torch.cuda.synchronize()
    return [y.cpu().numpy() for y in ys]


@pytest.mark.parametrize("rows", [-1, 32, 64, 128])
@pytest.mark.parametrize("tokens", [1, 7, 16, 24, 40, 64])
def test_qkv_one_x_three_weights(rows, tokens):
    _native.set_skinny_rows(rows)
    k = 1024
    x = synthetic.make_b(tokens, k, seed=tokens, kind="int")
    problems = [_problem(m, k, tokens, seed=10 * i + tokens, x=x) for i, m in enumerate((1024, 256, 320))]
    got = _run(problems, tokens, shared_x=x.cuda())
    for g, p in zip(got, problems):
        assert np.array_equal(g, p["want"])


@pytest.mark.parametrize("y_dtype,bias_dtype", [(torch.float16, torch.float32), (torch.float32, torch.float16)])
def test_different_shapes_and_a_problem_without_bias(y_dtype, bias_dtype):
    tokens = 16
    shapes = ((704, 512), (192, 2080), (2048, 544), (64, 4096), (1088, 32))
    problems = [_problem(m, k, tokens, seed=100 + i, bias_dtype=bias_dtype, y_dtype=y_dtype) for i, (m, k) in enumerate(shapes)]
    problems[2]["bias"] = None
    a_dense = problems[2]["want"]  # recompute without the bias
    a, meta = synthetic.make_weight(2048, 544, seed=102)
    dense = oracle.decompress_operands(a.numpy(), meta.numpy(), 2048, 544)
    problems[2]["want"] = (problems[2]["x"].numpy().astype(np.float32) @ dense.astype(np.float32).T).astype(a_dense.dtype)
    got = _run(problems, tokens, y_dtype=y_dtype)
    for g, p in zip(got, problems):
        assert np.array_equal(g, p["want"])
    # identical to the single form, N(0,1) activations included (same sums in the same order)
    _native.set_split_k(1)
    for p in problems:
        xn = synthetic.make_b(tokens, p["k"], seed=7, kind="normal").cuda()
        single = torch.empty((tokens, p["m"]), dtype=y_dtype, device="cuda")
        _native.linear_prepared(p["prep"], xn, single, p["m"], p["k"], bias=p["bias"].cuda() if p["bias"] is not None else None)
        p["xn"], p["single"] = xn, single
    ys = [torch.empty((tokens, p["m"]), dtype=y_dtype, device="cuda") for p in problems]
    _native.linear_prepared_grouped([(p["prep"], p["xn"], y, p["m"], p["k"], p["bias"].cuda() if p["bias"] is not None else None)
                                     for p, y in zip(problems, ys)])
    torch.cuda.synchronize()
    for p, y in zip(problems, ys):
        assert torch.equal(y, p["single"])


def test_more_problems_than_one_launch_and_many_tokens():
    tokens = 8
    problems = [_problem(128 + 64 * (i % 3), 256 + 32 * (i % 5), tokens, seed=200 + i) for i in range(19)]
    for g, p in zip(_run(problems, tokens), problems):
        assert np.array_equal(g, p["want"])
    # beyond the split-K kernel's token range the call is a sequence of single calls
    tokens = 200
    problems = [_problem(m, 512, tokens, seed=300 + i) for i, m in enumerate((256, 640))]
    for g, p in zip(_run(problems, tokens), problems):
        assert np.array_equal(g, p["want"])


def test_argument_checks():
    p = _problem(256, 512, 16, seed=1)
    y = torch.empty((16, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        _native.linear_prepared_grouped([(p["prep"], p["x"].cuda(), y, 256, 512, None),
                                         (p["prep"], p["x"].cuda()[:8].contiguous(), y[:8].contiguous(), 256, 512, None)])
    lib = _native.lib()
    table = (_native.LinearProblem * 1)(_native.LinearProblem(p["prep"].data_ptr(), p["x"].cuda().data_ptr() + 2, None,
                                                              y.data_ptr(), 256, 512))
    assert lib.onebit_sparse_linear_prepared_grouped(table, 1, 16, 1, 1, None) == 1
    assert "aligned" in _native.last_error()
    assert lib.onebit_sparse_linear_prepared_grouped(table, 0, 16, 1, 1, None) == 1
    assert lib.onebit_sparse_linear_prepared_grouped(None, 1, 16, 1, 1, None) == 1


def test_layers_forward_grouped_equals_the_layers_one_by_one():
    import onebitsparsemul_amd as ob
    torch.manual_seed(5)
    layers = []
    for out_features in (256, 128, 128):
        layer = ob.BinaryLinear_2_4(512, out_features)
        layer.pack(torch.randn(out_features, 512).half())
        layers.append(layer.cuda())
    layers[1].bias = torch.randn(128, dtype=torch.float16, device="cuda")
    x = torch.randn(2, 5, 512, dtype=torch.float16, device="cuda")
    grouped = ob.forward_grouped(layers, x)
    for layer, got in zip(layers, grouped):
        want = layer(x)
        assert got.shape == want.shape == (2, 5, layer.outfeatures) and torch.equal(got, want)
    # one input per layer, float32 activations (float32 results), and a token count beyond the split-K kernel's range
    xs = [torch.randn(70, 512, device="cuda") for _ in layers]
    for layer, x, got in zip(layers, xs, ob.forward_grouped(layers, xs)):
        want = layer(x)
        assert got.dtype == torch.float32 and torch.equal(got, want)
