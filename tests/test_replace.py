"""Model replacement helper (reference: tests/python/test_model_replace.py): layer swapping and accounting on
the CPU; the forward pass of a replaced model is checked on the GPU."""
import numpy as np
import pytest
import torch
import torch.nn as nn

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
