"""2:4 semi-structured format used by the one-bit sparse GEMM (host side, PyTorch tensors).

Same functions, argument meaning and error behaviour as the reference module
onebit_sparse_mul/_semi_structured_conversions.py (:21-48 offsets, :54-179 compress, :186-283 decompress,
:286-314 mask), written from the format definition rather than from that code:

* a group of four dense values keeps two; its metadata nibble is ``idx0 | idx1 << 2`` with idx0 < idx1 the
  kept positions; four nibbles make one int16 (group g at bits 4g), one int16 covers 16 dense columns;
* the metadata matrix (m, k/16) is stored reordered: every block of 64 rows x 2 metadata columns occupies
  128 consecutive int16, at position  b1<<6 | b5<<5 | b4<<4 | b3<<3 | b0<<2 | (c&1)<<1 | b2  for row bits
  b0..b5, blocks ordered column-pair-major, then by row block.

Only the 16-bit-metadata path (dense dtype half / bfloat16 / int32) exists here: it is the only one the
one-bit pipeline uses. The reorder is a bijection only for m % 64 == 0 and k % 32 == 0, and that is what
this module demands (the reference checks m % 32, k % 16 and then writes out of range for such shapes).
"""
import torch

# nibble for each pattern of non-zero flags (bit i of the index = dense[i] != 0). Patterns with exactly two
# flags encode their positions; the others use the fixed choices of the reference (:110-124).
_NIBBLE_OF_PATTERN = (
    0xE,  # 0000
    0x8,  # 1000  (only position 0)
    0x9,  # 0100
    0x4,  # 1100
    0xE,  # 0010
    0x8,  # 1010
    0x9,  # 0110
    0x4,  # 1110
    0xE,  # 0001
    0xC,  # 1001
    0xD,  # 0101
    0x4,  # 1101
    0xE,  # 0011
    0xC,  # 1011
    0xD,  # 0111
    0x4,  # 1111
)

_SUPPORTED = (torch.half, torch.bfloat16, torch.int32)


def _check_dense(dense):
    if dense.dim() != 2:
        raise RuntimeError(f"Expected 2-dimensional dense tensor, got {dense.dim()}-dimensional tensor")
    if dense.dtype not in _SUPPORTED:
        raise RuntimeError(f"Invalid datatype {dense.dtype} of dense matrix (supported: half, bfloat16, int32)")
    m, k = dense.shape
    if m % 64 != 0:
        raise RuntimeError(f"Number of rows of dense matrix {m} must be divisible by 64")
    if k % 32 != 0:
        raise RuntimeError(f"Number of columns of dense matrix {k} must be divisible by 32")
    return m, k


def _calculate_meta_reordering_scatter_offsets(m, meta_ncols, meta_dtype, device):
    """Flat int16 offsets, in row-major order of the logical (m, meta_ncols) metadata matrix, of every
    element inside the reordered buffer (reference :21-48)."""
    if meta_dtype != torch.int16:
        raise RuntimeError("only int16 metadata is supported")
    r = torch.arange(m, device=device, dtype=torch.int64)[:, None]
    c = torch.arange(meta_ncols, device=device, dtype=torch.int64)[None, :]
    inner = (((r >> 1) & 1) << 6) | (((r >> 3) & 7) << 3) | ((r & 1) << 2) | ((c & 1) << 1) | ((r >> 2) & 1)
    return ((c >> 1) * (2 * m) + (r >> 6) * 128 + inner).reshape(-1)


def sparse_semi_structured_from_dense_cutlass(dense):
    """dense (m, k) with at most two non-zeros per aligned group of four -> (sparse (m, k/2), meta (m, k/16)
    int16, reordered). Groups with fewer or more than two non-zeros get the reference's fixed encodings."""
    m, k = _check_dense(dense)
    device = dense.device
    groups = dense.reshape(m, k // 4, 4)
    flags = (groups != 0).to(torch.int64)
    pattern = flags[..., 0] | (flags[..., 1] << 1) | (flags[..., 2] << 2) | (flags[..., 3] << 3)
    nibble = torch.tensor(_NIBBLE_OF_PATTERN, dtype=torch.int64, device=device)[pattern]
    idx = torch.stack((nibble & 3, nibble >> 2), dim=-1)
    sparse = torch.gather(groups, -1, idx).reshape(m, k // 2)
    quads = nibble.reshape(m, k // 16, 4)
    word = quads[..., 0] | (quads[..., 1] << 4) | (quads[..., 2] << 8) | (quads[..., 3] << 12)
    word = torch.where(word >= 0x8000, word - 0x10000, word).to(torch.int16)
    offsets = _calculate_meta_reordering_scatter_offsets(m, k // 16, torch.int16, device)
    meta_reordered = torch.empty(m * (k // 16), dtype=torch.int16, device=device)
    meta_reordered[offsets] = word.reshape(-1)
    return sparse, meta_reordered.view(m, k // 16)


def meta_to_logical(meta_reordered):
    """Undo the reordering: (m, k/16) reordered -> logical row-major metadata."""
    m, ncols = meta_reordered.shape
    offsets = _calculate_meta_reordering_scatter_offsets(m, ncols, meta_reordered.dtype, meta_reordered.device)
    return meta_reordered.reshape(-1)[offsets].view(m, ncols)


def sparse_semi_structured_to_dense_cutlass(sparse, meta_reordered):
    """Inverse of the function above: (sparse (m, k/2), reordered meta (m, k/16)) -> dense (m, k)."""
    if sparse.dim() != 2:
        raise RuntimeError(f"Expected 2-dimensional sparse tensor, got {sparse.dim()}-dimensional tensor")
    if meta_reordered.dim() != 2:
        raise RuntimeError(f"Expected 2-dimensional meta tensor, got {meta_reordered.dim()}-dimensional tensor")
    m, ks = sparse.shape
    if meta_reordered.device != sparse.device:
        raise RuntimeError(
            f"Expected meta matrix to be on {sparse.device} device, got matrix on {meta_reordered.device} device")
    if meta_reordered.dtype != torch.int16:
        raise RuntimeError(f"Invalid datatype {meta_reordered.dtype} of meta matrix")
    if meta_reordered.shape[0] != m:
        raise RuntimeError(
            f"Number of rows of meta matrix {meta_reordered.shape[0]} must be equal to number of rows of sparse matrix {m}")
    if meta_reordered.shape[1] * 8 != ks:
        raise RuntimeError(
            f"Number of columns of sparse matrix {ks} different from the {meta_reordered.shape[1] * 8}, "
            "expected according to the number of columns of meta matrix")
    if m % 64 != 0 or ks % 16 != 0:
        raise RuntimeError("sparse matrix must have a multiple of 64 rows and of 16 columns")
    word = meta_to_logical(meta_reordered).to(torch.int64) & 0xFFFF
    shifts = torch.arange(0, 16, 2, device=sparse.device, dtype=torch.int64)
    pos = (word[..., None] >> shifts) & 3                      # (m, k/16, 8): position of kept value j
    group = torch.arange(ks, device=sparse.device, dtype=torch.int64) // 2  # dense group of kept value
    cols = pos.reshape(m, ks) + 4 * group[None, :]
    dense = torch.zeros((m, 2 * ks), dtype=sparse.dtype, device=sparse.device)
    dense.scatter_(1, cols, sparse)
    return dense


def mask_creator(tensor):
    """2:4 magnitude mask: 1 for the two largest |w| of every group of four (flattened order), 0 elsewhere.
    Ties are broken towards the higher index (the lower index is pruned first); the reference leaves the
    order among equal magnitudes to an unstable argsort (:308-309)."""
    if tensor.numel() % 4 != 0:
        raise ValueError(f"Tensor of size {tensor.shape} can't be evenly divided into 4 groups")
    mag = tensor.detach().abs().reshape(-1, 4)
    order = torch.argsort(mag, dim=1, stable=True)[:, :2]
    mask = torch.ones(mag.shape, device=tensor.device)
    mask.scatter_(1, order, 0.0)
    return mask.reshape(tensor.shape)
