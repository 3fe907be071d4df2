"""The package's host-side format code (PyTorch tensors, mirrors the reference's Python module) against the
oracle, plus its error behaviour. CPU only."""
import json
import os

import numpy as np
import pytest
import torch

import onebitsparsemul_amd as ob
from onebitsparsemul_amd import _semi_structured_conversions as conv
from onebitsparsemul_amd import synthetic

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kat_reference_tests.json")


def _random_dense(rng, m, k, degenerate=False):
    dense = np.zeros((m, k // 4, 4), dtype=np.float32)
    if degenerate:
        flags = rng.integers(0, 2, size=dense.shape).astype(bool)
    else:
        flags = np.zeros(dense.shape, dtype=bool)
        pick = np.array([(0, 1), (0, 2), (1, 2), (0, 3), (1, 3), (2, 3)])[rng.integers(0, 6, size=(m, k // 4))]
        np.put_along_axis(flags, pick, True, axis=-1)
    vals = rng.integers(1, 9, size=dense.shape) * rng.choice([-1, 1], size=dense.shape)
    return np.where(flags, vals, 0).astype(np.float32).reshape(m, k)


@pytest.mark.parametrize("m,ncols", [(64, 2), (192, 6), (11008, 4)])
def test_offsets_match_oracle(oracle_lib, m, ncols):
    got = conv._calculate_meta_reordering_scatter_offsets(m, ncols, torch.int16, "cpu").view(m, ncols).numpy()
    rows = sorted(set(list(range(0, min(m, 130))) + [m - 1, m - 64, m // 2]))
    for r in rows:
        for c in range(ncols):
            assert got[r, c] == oracle_lib.meta_offset(r, c, m)


@pytest.mark.parametrize("degenerate", [False, True])
@pytest.mark.parametrize("dtype", [torch.int32, torch.half])
def test_from_dense_and_back_match_oracle(oracle_lib, degenerate, dtype):
    rng = np.random.default_rng(21 + degenerate)
    dense = _random_dense(rng, 128, 96, degenerate)
    sparse, meta = conv.sparse_semi_structured_from_dense_cutlass(torch.from_numpy(dense).to(dtype))
    o_sparse, o_meta = oracle_lib.sparse_from_dense(dense)
    assert sparse.dtype == dtype and meta.dtype == torch.int16 and tuple(meta.shape) == (128, 6)
    assert np.array_equal(sparse.to(torch.float32).numpy(), o_sparse)
    assert np.array_equal(meta.numpy(), o_meta)
    back = conv.sparse_semi_structured_to_dense_cutlass(sparse, meta)
    assert np.array_equal(back.to(torch.float32).numpy(), oracle_lib.sparse_to_dense(o_sparse, o_meta))


def test_kat_through_package():
    with open(GOLDEN) as f:
        kat = json.load(f)
    w = torch.zeros((64, 32), dtype=torch.int32)
    w[:, 0::4] = 1
    w[:, 1::4] = 1
    w[0, :16] = torch.tensor(kat["dense_rows"][0], dtype=torch.int32)
    w[1, :16] = torch.tensor(kat["dense_rows"][1], dtype=torch.int32)
    mask = conv.mask_creator(w)
    assert mask[0, :16].int().tolist() == kat["mask_rows"][0]
    assert mask[1, :16].int().tolist() == kat["mask_rows"][1]
    sparse, meta = conv.sparse_semi_structured_from_dense_cutlass(w)
    assert sparse[0, :8].tolist() == kat["sparse_rows"][0]
    binary = ob.binary_quant(sparse)
    assert binary[:2, :8].tolist() == kat["binary_rows"]
    assert ob.pack_binary(binary)[:2, 0].tolist() == kat["packed_bytes"]
    assert int(meta[0, 0]) == kat["meta_row0_first_element"]
    assert conv.mask_creator(torch.ones(2, 8))[0, :4].int().tolist() == kat["all_ones_weight_mask_first_group"]


def test_pack_unpack_match_oracle(oracle_lib):
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2, size=(24, 64)).astype(np.uint8)
    packed = ob.pack_binary(torch.from_numpy(bits))
    assert packed.dtype == torch.uint8
    assert np.array_equal(packed.numpy(), oracle_lib.pack_binary(bits))
    assert np.array_equal(ob.unpack_binary(packed).numpy(), bits)
    with pytest.raises(ValueError):
        ob.pack_binary(torch.zeros(2, 12, dtype=torch.uint8))


def test_mask_creator_matches_oracle(oracle_lib):
    rng = np.random.default_rng(13)
    w = rng.integers(-3, 4, size=(64, 64)).astype(np.float32)  # many ties
    got = conv.mask_creator(torch.from_numpy(w)).numpy()
    assert np.array_equal(got, oracle_lib.mask_creator(w))
    assert np.all(got.reshape(-1, 4).sum(-1) == 2)
    with pytest.raises(ValueError):
        conv.mask_creator(torch.ones(3, 3))


def test_linear_layer_pack_and_dequant(oracle_lib):
    rng = np.random.default_rng(17)
    out_f, in_f = 128, 96
    w = rng.standard_normal((out_f, in_f)).astype(np.float32)
    layer = ob.BinaryLinear_2_4(in_f, out_f)
    with pytest.raises(NotImplementedError):
        layer(torch.zeros(1, in_f))
    layer.pack(torch.from_numpy(w).half())
    assert tuple(layer.packed_binary_sparse.shape) == (in_f // 2, out_f // 8)
    assert tuple(layer.meta.shape) == (out_f, in_f // 16)
    wh = w.astype(np.float16).astype(np.float32)
    want = np.sign(wh * oracle_lib.mask_creator(wh)).astype(np.int8)
    dense = oracle_lib.decompress_operands(layer.packed_binary_sparse.numpy(), layer.meta.numpy(), out_f, in_f)
    assert np.array_equal(dense, want)
    tile = ob.dequant_desparse_tile(layer.packed_binary_sparse, layer.meta)
    assert np.array_equal(tile.numpy().astype(np.int8), want)
    x = torch.from_numpy(rng.integers(-4, 5, size=(5, in_f)).astype(np.float32))
    y = ob.py_binary_gemm(x, layer.packed_binary_sparse, layer.meta)
    assert np.array_equal(y.numpy(), x.numpy() @ want.T.astype(np.float32))
    # registered buffers: the packed weight survives a state_dict round trip
    other = ob.BinaryLinear_2_4(in_f, out_f)
    other.load_state_dict(layer.state_dict())
    assert other.vaild and torch.equal(other.meta, layer.meta)
    with pytest.raises(ValueError):
        ob.BinaryLinear_2_4(100, 64)


def test_error_behaviour():
    with pytest.raises(RuntimeError):
        conv.sparse_semi_structured_from_dense_cutlass(torch.zeros(64, 32, 2, dtype=torch.half))
    with pytest.raises(RuntimeError):
        conv.sparse_semi_structured_from_dense_cutlass(torch.zeros(32, 32, dtype=torch.half))   # rows % 64
    with pytest.raises(RuntimeError):
        conv.sparse_semi_structured_from_dense_cutlass(torch.zeros(64, 48, dtype=torch.half))   # cols % 32
    with pytest.raises(RuntimeError):
        conv.sparse_semi_structured_from_dense_cutlass(torch.zeros(64, 32, dtype=torch.float64))
    with pytest.raises(RuntimeError):
        conv.sparse_semi_structured_to_dense_cutlass(torch.zeros(64, 16, dtype=torch.half),
                                                     torch.zeros(64, 3, dtype=torch.int16))
    with pytest.raises(RuntimeError):
        conv.sparse_semi_structured_to_dense_cutlass(torch.zeros(64, 16, dtype=torch.half),
                                                     torch.zeros(64, 2, dtype=torch.int32))
    with pytest.raises(ValueError):
        ob.py_binary_gemm(torch.zeros(2, 32), torch.zeros(16, 8, dtype=torch.int8), torch.zeros(64, 2, dtype=torch.int16))


def test_synthetic_weight_is_valid_2to4(oracle_lib):
    a, meta = synthetic.make_weight(128, 64, seed=7)
    dense = oracle_lib.decompress_operands(a.numpy(), meta.numpy(), 128, 64)
    assert np.all((dense != 0).reshape(128, 16, 4).sum(-1) == 2)
    a2, meta2 = synthetic.make_weight(128, 64, seed=7)
    assert torch.equal(a, a2) and torch.equal(meta, meta2)
    assert set(np.unique(dense).tolist()) == {-1, 0, 1}


def test_layer_is_valid_only_after_its_buffers_were_loaded():
    """A state dict without the packed weight must not mark the layer as holding one (strict=False loads)."""
    import onebitsparsemul_amd as ob
    layer = ob.BinaryLinear_2_4(64, 64)
    layer.load_state_dict({}, strict=False)
    assert not layer.vaild
    donor = ob.BinaryLinear_2_4(64, 64)
    donor.pack(torch.randn(64, 64))
    layer.load_state_dict(donor.state_dict())
    assert layer.vaild and torch.equal(layer.meta, donor.meta)
    with pytest.raises(ValueError):
        ob.BinaryLinear_2_4(64, 64, out_dtype=torch.bfloat16)
