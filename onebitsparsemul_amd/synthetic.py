"""Synthetic operands of the benchmark configurations, generated directly in the stored formats.

A: per aligned group of four along K one of the six two-of-four patterns, uniformly; each kept value +-1 with
probability 1/2. Stored as one-bit values (column-major) and reordered int16 metadata, exactly what
BinaryLinear_2_4.pack() produces. B: fp16 N(0,1) or small integers in [-8, 8] (the reference benchmark's
range, tests/kernel_test.cu:325-332)."""
import torch

from ._semi_structured_conversions import _calculate_meta_reordering_scatter_offsets

_LEGAL_NIBBLES = (0x4, 0x8, 0x9, 0xC, 0xD, 0xE)


def make_weight(m, k, seed, device="cpu"):
    """Returns (a, meta): a uint8 (k/2, m/8) one-bit values, meta int16 (m, k/16) reordered."""
    if m % 64 or k % 32:
        raise ValueError("m must be a multiple of 64 and k of 32")
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    nib_idx = torch.randint(0, 6, (m, k // 16, 4), generator=g, device=device)
    nib = torch.tensor(_LEGAL_NIBBLES, device=device, dtype=torch.int64)[nib_idx]
    word = nib[..., 0] | (nib[..., 1] << 4) | (nib[..., 2] << 8) | (nib[..., 3] << 12)
    word = torch.where(word >= 0x8000, word - 0x10000, word).to(torch.int16)
    offsets = _calculate_meta_reordering_scatter_offsets(m, k // 16, torch.int16, device)
    meta = torch.empty(m * (k // 16), dtype=torch.int16, device=device)
    meta[offsets] = word.reshape(-1)
    del nib_idx, nib, word, offsets
    # bits of the (k/2, m) transposed value matrix, packed along m (LSB first) -> (k/2, m/8)
    a = torch.randint(0, 256, (k // 2, m // 8), generator=g, device=device, dtype=torch.uint8)
    return a, meta.view(m, k // 16)


def make_b(k, n, seed, kind="normal", device="cpu"):
    g = torch.Generator(device=device)
    g.manual_seed(seed + 1)
    if kind == "normal":
        return torch.randn((k, n), generator=g, device=device, dtype=torch.float32).to(torch.float16)
    if kind == "int":
        return torch.randint(-8, 9, (k, n), generator=g, device=device).to(torch.float16)
    raise ValueError(kind)


def make_c(m, n, seed, dtype=torch.float16, device="cpu"):
    g = torch.Generator(device=device)
    g.manual_seed(seed + 2)
    return torch.randn((m, n), generator=g, device=device, dtype=torch.float32).to(dtype)
