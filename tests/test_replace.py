"""Model replacement helper (reference: tests/python/test_model_replace.py): layer swapping and accounting on
the CPU; the forward pass of a replaced model is checked on the GPU."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle
import onebitsparsemul_amd as ob
from onebitsparsemul_amd import replace


class _Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.up = nn.Linear(64, 128, bias=False)
        self.down = nn.Linear(128, 64, bias=True)
        self.odd = nn.Linear(64, 10, bias=True)  # 10 output features: the packed format does not admit it

    def forward(self, x):
        return self.down(torch.relu(self.up(x))), self.odd(x)


class _Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.blocks = nn.ModuleList([_Block(), _Block()])
        self.head = nn.Linear(64, 64, bias=False)

    def forward(self, x):
        for blk in self.blocks:
            x, _ = blk(x)
        return self.head(x)


def _expected_dense(weight):
    """2:4 magnitude mask, then sign with zero -> -1: the weight a replaced layer represents"""
    mask = ob.mask_creator(weight)
    return torch.where(weight > 0, 1.0, -1.0) * mask


def test_replace_swaps_admissible_layers_and_accounts():
    torch.manual_seed(0)
    net = _Net()
    originals = {n: m.weight.detach().clone() for n, m in net.named_modules() if isinstance(m, nn.Linear)}
    stats = replace.replace_linear_layers(net, skip=("head",))
    assert sorted(stats["replaced"]) == ["blocks.0.down", "blocks.0.up", "blocks.1.down", "blocks.1.up"]
    assert sorted(stats["kept"]) == ["blocks.0.odd", "blocks.1.odd", "head"]
    assert stats["weight_params"] == 4 * 64 * 128 and stats["bias_params"] == 2 * 64
    assert stats["packed_weight_gib"] == pytest.approx(stats["fp16_weight_gib"] * 1.5 / 16)
    for name in stats["replaced"]:
        layer = net.get_submodule(name)
        assert isinstance(layer, ob.BinaryLinear_2_4) and layer.vaild
        w = originals[name]
        assert layer.packed_binary_sparse.shape == (w.shape[1] // 2, w.shape[0] // 8)
        assert layer.meta.shape == (w.shape[0], w.shape[1] // 16)
        dense = ob.dequant_desparse_tile(layer.packed_binary_sparse, layer.meta)
        assert torch.equal(dense.float(), _expected_dense(w).float())
    assert isinstance(net.blocks[0].odd, nn.Linear) and isinstance(net.head, nn.Linear)
    assert net.blocks[0].down.bias is not None and net.blocks[0].up.bias is None
    # the packed buffers travel in the state dict
    keys = net.state_dict().keys()
    assert "blocks.0.up.packed_binary_sparse" in keys and "blocks.0.up.meta" in keys and "blocks.0.down.bias" in keys


def test_set_module_nested():
    net = _Net()
    replace.set_module(net, "blocks.1.up", nn.Identity())
    assert isinstance(net.blocks[1].up, nn.Identity)


@pytest.mark.gpu
def test_replaced_model_forward_matches_dense_reference():
    torch.manual_seed(1)
    net = _Net().half().cuda()
    ref = _Net().half().cuda()
    ref.load_state_dict(net.state_dict())
    for name, module in ref.named_modules():
        if isinstance(module, nn.Linear) and module.weight.shape[0] % 64 == 0 and name != "head":
            module.weight.data = _expected_dense(module.weight.data.cpu()).half().cuda()
    stats = replace.replace_linear_layers(net, skip=("head",))
    assert len(stats["replaced"]) == 4
    x = torch.randn(3, 5, 64, dtype=torch.float16, device="cuda")
    with torch.no_grad():
        got = net(x).float().cpu().numpy()
        want = ref(x).float().cpu().numpy()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 2e-2 * np.abs(want).max()  # two chained fp16 layers with fp16 rounding between


class _TwoLayer(nn.Module):
    def __init__(self, d_in=256, d_hidden=512, d_out=192):
        super().__init__()
        self.up = nn.Linear(d_in, d_hidden, bias=False)
        self.down = nn.Linear(d_hidden, d_out, bias=True)

    def forward(self, x):
        return self.down(torch.relu(self.up(x)))


def _oracle_weight(weight_fp16):
    """What a replaced layer must hold, by the oracle's restatement of the reference pipeline
    (onebit_sparse_mul/__init__.py:130-145): magnitude mask, 2:4 compression, sign quantisation, transposed bit
    packing; returns the stored operands and their decompressed form (-1 / 0 / +1)."""
    w = weight_fp16.float().numpy()
    out_f, in_f = w.shape
    sparse, meta = oracle.sparse_from_dense(w * oracle.mask_creator(w))
    a = oracle.pack_binary(np.ascontiguousarray(oracle.binary_quant(sparse).T))
    return a, meta, oracle.decompress_operands(a, meta, out_f, in_f)


def _oracle_linear(dense, x_fp16, bias_fp16, acc):
    """y = x W^T + bias through the oracle's host GEMM on the decompressed weight, fp32 (or fp64) sums, one rounding
    to float16 at the end (what the layer returns for float16 activations)."""
    d = oracle.host_gemm(dense, np.ascontiguousarray(x_fp16.T), d_dtype=oracle.F32, acc=acc).T.astype(np.float64)
    if bias_fp16 is not None:
        d = d + bias_fp16.astype(np.float64)[None, :]
    return d


@pytest.mark.gpu
def test_replaced_model_matches_the_oracle_layer_by_layer():
    """Counterpart of the reference's model script (tests/python/test_model_replace.py:22-56) with a check it does
    not have: every replaced layer's stored operands equal the oracle's, and its GPU forward equals the oracle's host
    GEMM on the same input - bit for bit on integer activations, within 1e-3 on N(0,1) activations."""
    torch.manual_seed(5)
    net = _TwoLayer().half()
    with torch.no_grad():
        net.down.bias.copy_(torch.randint(-3, 4, net.down.bias.shape).half())
    expected = {name: _oracle_weight(getattr(net, name).weight.detach()) for name in ("up", "down")}
    bias = net.down.bias.detach().numpy().copy()
    net = net.cuda()
    stats = replace.replace_linear_layers(net)
    assert sorted(stats["replaced"]) == ["down", "up"]
    for name, (a, meta, _) in expected.items():
        layer = getattr(net, name)
        assert np.array_equal(layer.packed_binary_sparse.cpu().numpy(), a)       # GPU packer = oracle pipeline
        assert np.array_equal(layer.meta.cpu().numpy(), meta)
    seen = {}
    hooks = [getattr(net, name).register_forward_hook(
        lambda mod, inp, out, name=name: seen.__setitem__(name, (inp[0].detach().cpu(), out.detach().cpu())))
        for name in ("up", "down")]
    # integer activations: every sum is an integer below 2^24, so the only rounding is the final one to float16
    x = torch.randint(-2, 3, (3, 7, 256)).half().cuda()
    with torch.no_grad():
        net(x)
    torch.cuda.synchronize()
    for name, b in (("up", None), ("down", bias)):
        inp, out = seen[name]
        want = _oracle_linear(expected[name][2], inp.reshape(-1, inp.shape[-1]).numpy(), b, "f32")
        assert np.array_equal(out.reshape(-1, out.shape[-1]).numpy(), want.astype(np.float16)), name
    # N(0,1) activations: each layer against the oracle on the input that layer actually received
    x = torch.randn(4, 33, 256).half().cuda()
    with torch.no_grad():
        y = net(x)
    torch.cuda.synchronize()
    assert torch.isfinite(y).all()
    for name, b in (("up", None), ("down", bias)):
        inp, out = seen[name]
        want = _oracle_linear(expected[name][2], inp.reshape(-1, inp.shape[-1]).numpy(), b, "f64")
        got = out.reshape(-1, out.shape[-1]).double().numpy()
        assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max(), name
    for h in hooks:
        h.remove()
