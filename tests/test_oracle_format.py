"""Pins the CPU oracle's format functions (oracle/onebit_oracle.c) against everything that fixes them
without running the reference: the known-answer values of the reference's own tests, closed forms and
invariants of the layout, and PyTorch's own library copy of the CUTLASS conversion routines."""
import json
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kat_reference_tests.json")


@pytest.fixture(scope="module")
def kat():
    with open(GOLDEN) as f:
        return json.load(f)


def test_half_conversion_matches_ieee(oracle_lib):
    hs = np.arange(0, 65536, 7, dtype=np.uint16)
    ref = hs.view(np.float16).astype(np.float32)
    got = np.array([oracle_lib.half_to_float(h) for h in hs], dtype=np.float32)
    keep = ~np.isnan(ref)
    assert np.array_equal(got.view(np.uint32)[keep], ref.view(np.uint32)[keep])
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(3000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1, 300, 7e4)] +
                       [np.array([65504, 65519.99, 65520, 2.9802322e-8, 2.9802326e-8, 0.0, -0.0, 2049, 2051],
                                 dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([oracle_lib.float_to_half(v) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_kat_pack_bytes(oracle_lib, kat):
    # tests/python/test_sparse.py:60-64: sign rows -> bytes 112 and 165 (element 8c+i -> bit i)
    bits = np.array(kat["binary_rows"], dtype=np.uint8)
    packed = oracle_lib.pack_binary(bits)
    assert packed[:, 0].tolist() == kat["packed_bytes"]
    assert np.array_equal(oracle_lib.unpack_binary(packed), bits)


def test_kat_binary_quant(oracle_lib, kat):
    sparse = np.array(kat["sparse_rows"], dtype=np.float32)
    assert np.array_equal(oracle_lib.binary_quant(sparse), np.array(kat["binary_rows"], dtype=np.uint8))
    # zero quantises to bit 0 (= -1): "value > 0" (onebit_sparse_mul/__init__.py:22-23)
    assert oracle_lib.binary_quant(np.array([[0.0, -0.0, 1e-30, -3.0]], dtype=np.float32)).tolist() == [[0, 0, 1, 0]]


def test_kat_compress_rows(oracle_lib, kat):
    # embed the two documented rows as rows 0 and 1 of a (64, 32) matrix
    dense = np.zeros((64, 32), dtype=np.float32)
    dense[:, 0::4] = 1
    dense[:, 1::4] = 1
    dense[0, :16] = kat["dense_rows"][0]
    dense[1, :16] = kat["dense_rows"][1]
    sparse, meta = oracle_lib.sparse_from_dense(dense)
    assert sparse[0, :8].tolist() == kat["sparse_rows"][0]
    assert sparse[1, :8].tolist() == kat["sparse_rows"][1]
    # meta.view(m, -1)[0, 0] of the reordered tensor is logical element (0, 0): offset(0, 0) == 0
    assert oracle_lib.meta_offset(0, 0, 64) == 0
    assert int(meta.reshape(-1)[0]) == kat["meta_row0_first_element"]
    assert np.array_equal(oracle_lib.sparse_to_dense(sparse, meta), dense)


def test_mask_tie_rule_is_what_the_reference_expression_gives_on_this_torch(oracle_lib):
    """The reference prunes `torch.argsort(|w|, dim=1)[:, :2]` of every group of four (unstable sort,
    _semi_structured_conversions.py:308-309). On the CPU build of PyTorch in this image that call returns the
    stable order for every one of the 256 rank patterns of four magnitudes (checked here with PyTorch's own
    routine, for the dtypes a weight can have and for small and large row counts), so the oracle's rule - among
    equal magnitudes the lower index is pruned first - is the reference's result in this environment."""
    import itertools
    import torch
    patterns = torch.tensor(list(itertools.product(range(4), repeat=4)), dtype=torch.float32)
    for repeats in (1, 300):
        x = patterns.repeat(repeats, 1)
        for dtype in (torch.float32, torch.float16, torch.bfloat16):
            unstable = torch.argsort(x.to(dtype), dim=1)[:, :2]
            mask = torch.ones_like(x).scatter_(1, unstable, 0.0)
            got = oracle_lib.mask_creator(x.numpy())
            assert np.array_equal(got, mask.numpy())


def test_kat_mask(oracle_lib, kat):
    for row, mask in zip(kat["dense_rows"], kat["mask_rows"]):
        got = oracle_lib.mask_creator(np.array([row], dtype=np.float32))
        assert got[0].astype(int).tolist() == mask
    ones = oracle_lib.mask_creator(np.ones((2, 8), dtype=np.float32))
    assert ones[0, :4].astype(int).tolist() == kat["all_ones_weight_mask_first_group"]
    # all-ones weight after masking: every group keeps positions 2, 3 -> nibble 0xE -> element 0xEEEE = -4370
    dense = np.tile(np.array([0, 0, 1, 1], dtype=np.float32), (64, 8))
    _, meta = oracle_lib.sparse_from_dense(dense)
    assert set(meta.reshape(-1).tolist()) == {kat["all_ones_weight_meta_element"]}


def _closed_form_reference(r, c, m):
    b = [(r >> i) & 1 for i in range(6)]
    return (c // 2) * 2 * m + (r // 64) * 128 + (
        b[1] << 6 | b[5] << 5 | b[4] << 4 | b[3] << 3 | b[0] << 2 | (c % 2) << 1 | b[2])


@pytest.mark.parametrize("m,ncols", [(64, 2), (128, 4), (256, 6), (11008, 2)])
def test_reference_offsets_closed_form_and_bijection(oracle_lib, m, ncols):
    offs = np.array([[oracle_lib.meta_offset(r, c, m) for c in range(ncols)] for r in range(m)])
    want = np.array([[_closed_form_reference(r, c, m) for c in range(ncols)] for r in range(m)])
    assert np.array_equal(offs, want)
    assert sorted(offs.reshape(-1).tolist()) == list(range(m * ncols))  # bijection
    # every (64 rows x 2 columns) block fills one 128-element window
    for rb in range(0, m, 64):
        for cp in range(0, ncols, 2):
            blk = offs[rb:rb + 64, cp:cp + 2].reshape(-1)
            assert blk.min() % 128 == 0 and blk.max() - blk.min() == 127


def test_reference_offsets_not_bijective_outside_domain(oracle_lib):
    # m = 32 (accepted by the reference's own check) writes out of range: documents why m % 64 is required
    offs = [oracle_lib.meta_offset(r, c, 32) for r in range(32) for c in range(2)]
    assert max(offs) >= 32 * 2


@pytest.mark.parametrize("m,ncols", [(32, 2), (64, 4), (256, 8)])
def test_cutlass_offsets_match_torch_library(oracle_lib, m, ncols):
    # torch ships its own restatement of CUTLASS reorder_meta (a library routine, not the reference)
    from torch.sparse._semi_structured_conversions import _calculate_meta_reordering_scatter_offsets as torch_offsets
    want = torch_offsets(m, ncols, torch.int16, "cpu").view(m, ncols).numpy()
    got = np.array([[oracle_lib.meta_offset(r, c, m, oracle_lib.LAYOUT_CUTLASS) for c in range(ncols)]
                    for r in range(m)])
    assert np.array_equal(got, want)


def _random_dense(rng, m, k, degenerate=False):
    dense = np.zeros((m, k), dtype=np.float32)
    groups = dense.reshape(m, k // 4, 4)
    if degenerate:
        flags = rng.integers(0, 2, size=groups.shape).astype(bool)  # 0..4 non-zeros per group
    else:
        flags = np.zeros(groups.shape, dtype=bool)
        pick = np.array([(0, 1), (0, 2), (1, 2), (0, 3), (1, 3), (2, 3)])[rng.integers(0, 6, size=groups.shape[:2])]
        np.put_along_axis(flags, pick, True, axis=-1)
    vals = rng.integers(1, 9, size=groups.shape) * rng.choice([-1, 1], size=groups.shape)
    groups[...] = np.where(flags, vals, 0)
    return dense


@pytest.mark.parametrize("degenerate", [False, True])
def test_compress_matches_torch_library_in_cutlass_layout(oracle_lib, degenerate):
    """The nibble encoding (all 16 non-zero patterns), value gather and int16 packing are the part of the
    reference that is identical to torch.sparse._semi_structured_conversions (the reference only changes the
    row permutation of the reorder), so torch's routine pins them, in the CUTLASS layout."""
    from torch.sparse._semi_structured_conversions import (
        sparse_semi_structured_from_dense_cutlass as torch_from_dense,
        sparse_semi_structured_to_dense_cutlass as torch_to_dense,
    )
    rng = np.random.default_rng(11 + degenerate)
    dense = _random_dense(rng, 64, 128, degenerate)
    sparse, meta = oracle_lib.sparse_from_dense(dense, oracle_lib.LAYOUT_CUTLASS)
    t_sparse, t_meta = torch_from_dense(torch.from_numpy(dense).to(torch.half))
    assert np.array_equal(sparse, t_sparse.numpy().astype(np.float32))
    assert np.array_equal(meta, t_meta.numpy())
    back = oracle_lib.sparse_to_dense(sparse, meta, oracle_lib.LAYOUT_CUTLASS)
    t_back = torch_to_dense(t_sparse, t_meta).numpy().astype(np.float32)
    assert np.array_equal(back, t_back)
    if not degenerate:
        assert np.array_equal(back, dense)


def test_reference_layout_is_permutation_of_logical(oracle_lib):
    rng = np.random.default_rng(5)
    dense = _random_dense(rng, 128, 96)
    s_ref, meta_ref = oracle_lib.sparse_from_dense(dense, oracle_lib.LAYOUT_REFERENCE)
    s_log, meta_log = oracle_lib.sparse_from_dense(dense, oracle_lib.LAYOUT_LOGICAL)
    assert np.array_equal(s_ref, s_log)
    flat = meta_ref.reshape(-1)
    for r in (0, 1, 2, 5, 37, 64, 127):
        for c in range(6):
            assert flat[_closed_form_reference(r, c, 128)] == meta_log[r, c]
    # legal nibbles only, idx0 < idx1
    words = meta_log.astype(np.int64) & 0xFFFF
    for g in range(4):
        nib = (words >> (4 * g)) & 15
        assert set(np.unique(nib).tolist()) <= {0x4, 0x8, 0x9, 0xC, 0xD, 0xE}
        assert np.all((nib & 3) < (nib >> 2))
    assert np.array_equal(oracle_lib.sparse_to_dense(s_ref, meta_ref), dense)


def test_decompress_operands_is_the_entry_points_format(oracle_lib):
    """a = column-major bits of the (m, k/2) sign matrix, i.e. pack_binary(signs.T) flattened
    (onebit_sparse_mul/__init__.py:139-143 with csrc/kernel_lib.cu:37)."""
    rng = np.random.default_rng(8)
    m, k = 128, 64
    dense = _random_dense(rng, m, k)
    sparse, meta = oracle_lib.sparse_from_dense(dense)
    bits = oracle_lib.binary_quant(sparse)                   # (m, k/2)
    a = oracle_lib.pack_binary(np.ascontiguousarray(bits.T))  # (k/2, m/8)
    got = oracle_lib.decompress_operands(a, meta, m, k)
    assert np.array_equal(got, np.sign(dense).astype(np.int8))
    # brute force on single elements: bit (r, j) is bit (r + j m) % 8 of byte (r + j m) / 8
    flat = a.reshape(-1)
    for r, j in ((0, 0), (7, 0), (8, 3), (127, 31), (65, 17)):
        pos = r + j * m
        assert (flat[pos // 8] >> (pos % 8)) & 1 == bits[r, j]
