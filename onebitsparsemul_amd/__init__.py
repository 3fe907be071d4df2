"""onebitsparsemul_amd - one-bit 2:4 sparse GEMM for MI355X (gfx950).

Python surface of the reference package ``onebit_sparse_mul`` (onebit_sparse_mul/__init__.py:12-145) on top
of libonebitmul.so: same callables, same argument meaning, intended semantics where the reference's own code
is inconsistent (result allocated on the operands' device, metadata passed in the binding's argument order,
``y = x @ W.T`` in the linear layer). GPU work always goes through the HIP library; nothing falls back to a
host computation.
"""
import torch
import torch.nn as nn

from . import _native
from ._semi_structured_conversions import (
    mask_creator,
    sparse_semi_structured_from_dense_cutlass,
    sparse_semi_structured_to_dense_cutlass,
)

__all__ = [
    "cuda_binary_mul", "cuda_binary_mul_", "binary_quant", "pack_binary", "unpack_binary", "dequant_desparse_tile",
    "py_binary_gemm", "BinaryLinear_2_4", "PreparedWeight", "mask_creator", "sparse_semi_structured_from_dense_cutlass",
    "sparse_semi_structured_to_dense_cutlass", "set_weight_cache", "clear_weight_cache",
]


def _binding():
    """The compiled torch binding `onebit_sparse_cuda` (reference: onebit_sparse_mul/torch_kernel_cuda.cpp)."""
    from . import onebit_sparse_cuda  # noqa: PLC0415  (compiled module, built in-tree)
    return onebit_sparse_cuda


def set_weight_cache(entries):
    """Let `cuda_binary_mul` / `onebit_mul` / the C entry points keep the reordered copy of up to `entries` weights
    per GPU, keyed by the weight tensors' addresses (0, the default, keeps nothing: the reference's behaviour).
    Only for weights that are neither modified nor freed while cached; see include/onebit_sparse_tensor.h."""
    _native.set_weight_cache(entries)


def clear_weight_cache():
    _native.clear_weight_cache()


def _problem_shape(A, B, meta):
    m, k = meta.shape[0], meta.shape[1] * 16
    if A.dtype != torch.uint8 or A.numel() != m * k // 16:
        raise ValueError(f"A must be uint8 with m*k/16 = {m * k // 16} bytes (shape (k/2, m/8)), got {tuple(A.shape)}")
    if B.dim() != 2 or B.shape[0] != k:
        raise ValueError(f"B must have shape (k={k}, n), got {tuple(B.shape)}")
    return m, B.shape[1], k


def cuda_binary_mul(A, B, meta):
    """C = W @ B with W the one-bit 2:4 weight stored as (A bits, meta); returns fp32 (m, n) on B's device.
    Reference: onebit_sparse_mul/__init__.py:12-15."""
    m, n, _ = _problem_shape(A, B, meta)
    C = torch.empty((m, n), dtype=torch.float32, device=B.device)
    _binding().onebit_mul(A, B, meta, C)
    return C


def cuda_binary_mul_(A, B, C, meta):
    """In-place form: writes into C (fp32 or fp16, (m, n)). Reference: onebit_sparse_mul/__init__.py:17-19."""
    _binding().onebit_mul(A, B, meta, C)
    return C


def binary_quant(tensor):
    """value > 0 -> 1, else 0. Reference: onebit_sparse_mul/__init__.py:22-23."""
    return (tensor > 0).to(torch.int64)


def pack_binary(tensor):
    """(rows, cols) of 0/1 -> (rows, cols/8) uint8; element 8c+i of a row is bit i of byte c.
    Reference: onebit_sparse_mul/__init__.py:25-34."""
    rows, cols = tensor.shape
    if cols % 8:
        raise ValueError("last dimension must be a multiple of 8")
    weights = (1 << torch.arange(8, device=tensor.device, dtype=torch.int64))
    return (tensor.reshape(rows, cols // 8, 8).to(torch.int64) * weights).sum(-1).to(torch.uint8)


def unpack_binary(packed_tensor):
    """Inverse of pack_binary; returns uint8 0/1. Reference: onebit_sparse_mul/__init__.py:36-45."""
    rows, pcols = packed_tensor.shape
    shifts = torch.arange(8, device=packed_tensor.device, dtype=torch.int64)
    bits = (packed_tensor.to(torch.int64)[..., None] >> shifts) & 1
    return bits.reshape(rows, pcols * 8).to(torch.uint8)


def dequant_desparse_tile(packed_sparse_tile, meta_tile):
    """(k/2, m/8) packed bits + (m, k/16) reordered metadata -> dense (m, k) weight with values in {-1, 0, +1}.
    Reference: onebit_sparse_mul/__init__.py:47-65 (whose shapes do not compose; this is the intended result)."""
    bits = unpack_binary(packed_sparse_tile).T.contiguous()  # (m, k/2)
    values = torch.where(bits == 1, 1, -1).to(torch.int32)
    return sparse_semi_structured_to_dense_cutlass(values, meta_tile)


def py_binary_gemm(x, packed_sparse_tensor, sparse_meta):
    """Host check: x (batch, k) @ W.T with W = dequant_desparse_tile(...), as torch.matmul on the dense weight.
    Reference: onebit_sparse_mul/__init__.py:67-97."""
    if packed_sparse_tensor.dtype != torch.uint8:
        raise ValueError("packed_sparse_tensor must be `torch.uint8`")
    if sparse_meta.dtype != torch.int16:
        raise ValueError("Sparse Meta must be `torch.int16`")
    if packed_sparse_tensor.shape[0] * 2 != x.shape[1]:
        raise ValueError("x.shape[1] must equal 2 * packed_sparse_tensor.shape[0] (the weight's in-features)")
    dense = dequant_desparse_tile(packed_sparse_tensor, sparse_meta)
    return torch.matmul(x, dense.to(x.dtype).T)


class PreparedWeight:
    """A packed weight reordered once for the gfx950 kernels (see include/onebit_sparse_tensor.h)."""

    def __init__(self, packed_binary_sparse, meta, layout=_native.META_REFERENCE):
        self.m = meta.shape[0]
        self.k = meta.shape[1] * 16
        self.buffer = _native.prepare(packed_binary_sparse, meta, self.m, self.k, layout)

    def matmul(self, b, out=None, c=None, alpha=1.0, beta=0.0, out_dtype=torch.float16):
        n = b.shape[1]
        if out is None:
            out = torch.empty((self.m, n), dtype=out_dtype, device=b.device)
        return _native.matmul_prepared(self.buffer, b, out, self.m, n, self.k, c=c, alpha=alpha, beta=beta)

    def linear(self, x, bias=None, out=None, out_dtype=torch.float16):
        """y (tokens, m) = x (tokens, k) @ W.T (+ bias): the layer's form, x and y token-major, no transposes."""
        if x.data_ptr() % 16:
            x = x.clone()  # a view that starts inside a 16-byte unit
        if out is None:
            out = torch.empty((x.shape[0], self.m), dtype=out_dtype, device=x.device)
        return _native.linear_prepared(self.buffer, x, out, self.m, self.k, bias=bias)


class BinaryLinear_2_4(nn.Module):
    """1-bit 2:4 sparse linear layer: y = x @ W.T (+ bias when one has been assigned), W (outfeatures, infeatures)
    stored at 1.5 bits per weight. Reference: onebit_sparse_mul/__init__.py:101-145."""

    def __init__(self, infeatures: int, outfeatures: int, out_dtype=None):
        """out_dtype: dtype of the kernel's result. None (default): float16 for float16 activations (the sums are
        accumulated in fp32 and rounded once; a sum of infeatures/2 terms of +-x can exceed float16's range for large
        activations) and float32 for every other activation dtype, so that the only precision loss is the cast of x
        to float16. torch.float32 returns the reference layer's fp32 product for float16 activations as well
        (onebit_sparse_mul/__init__.py:12-14: cuda_binary_mul returns an fp32 C)."""
        super().__init__()
        if infeatures % 32 != 0 or outfeatures % 64 != 0:
            raise ValueError("`infeatures` must be divisible by 32 and `outfeatures` by 64.")
        if out_dtype not in (None, torch.float16, torch.float32):
            raise ValueError("out_dtype must be None, torch.float16 or torch.float32")
        self.infeatures = infeatures
        self.outfeatures = outfeatures
        self.out_dtype = out_dtype
        self.register_buffer("packed_binary_sparse", torch.zeros((infeatures // 2, outfeatures // 8), dtype=torch.uint8))
        self.register_buffer("meta", torch.zeros((outfeatures, infeatures // 16), dtype=torch.int16))
        self.vaild = False
        self._prepared = None
        self.bias = None  # optional (outfeatures,) tensor added to the output; the model script assigns it

    def pack(self, weight):
        """weight (outfeatures, infeatures): prune to 2:4 by magnitude, keep the signs.
        Reference: onebit_sparse_mul/__init__.py:130-145."""
        if tuple(weight.shape) != (self.outfeatures, self.infeatures):
            raise ValueError(f"weight must have shape ({self.outfeatures}, {self.infeatures})")
        if weight.is_cuda and weight.dtype == torch.float16:
            # one fused HIP kernel (mask, compress, quantise, transpose-pack, reorder); same result as below
            self.packed_binary_sparse, self.meta = _native.pack_weight(weight.contiguous(), prune=True)
            self.vaild = True
            self._prepared = None
            return
        w = weight * mask_creator(weight).to(weight.dtype)
        if w.dtype not in (torch.half, torch.bfloat16, torch.int32):
            w = w.to(torch.half)
        sparse, meta = sparse_semi_structured_from_dense_cutlass(w)
        bits = binary_quant(sparse).T.contiguous()
        self.packed_binary_sparse = pack_binary(bits)
        self.meta = meta
        self.vaild = True
        self._prepared = None

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)
        # a packed weight is there only if both buffers came from the state dict
        if prefix + "packed_binary_sparse" in state_dict and prefix + "meta" in state_dict:
            self.vaild = True
        self._prepared = None

    def forward(self, x):
        if not self.vaild:
            raise NotImplementedError("the BinaryLinear_2_4 layer holds no packed weight: call pack() first")
        if self._prepared is None or self._prepared.buffer.device != x.device:
            self._prepared = PreparedWeight(self.packed_binary_sparse.to(x.device), self.meta.to(x.device))
        lead = x.shape[:-1]
        if x.numel() == 0:  # an empty batch: nothing to launch
            return x.new_zeros(*lead, self.outfeatures)
        tokens = x.reshape(-1, self.infeatures).to(torch.float16).contiguous()
        bias = self.bias
        if bias is not None and (bias.dtype not in (torch.float16, torch.float32) or bias.device != x.device):
            bias = bias.to(device=x.device, dtype=torch.float32)
        out_dtype = self.out_dtype or (torch.float16 if x.dtype == torch.float16 else torch.float32)
        # one kernel: reads the tokens where they lie, adds the bias, writes (tokens, outfeatures)
        y = self._prepared.linear(tokens, bias=bias.contiguous() if bias is not None else None, out_dtype=out_dtype)
        y = y.reshape(*lead, self.outfeatures)
        return y if self.out_dtype is not None else y.to(x.dtype)


def forward_grouped(layers, xs):
    """The forward passes of several BinaryLinear_2_4 layers on inputs with the same number of tokens, in one library
    call (one kernel launch per 16 layers for up to 64 tokens): the q / k / v or gate / up projections of a decoder
    layer. xs: one tensor for all layers, or one per layer. Returns the list of outputs, each what layer(x) returns."""
    if isinstance(xs, torch.Tensor):
        xs = [xs] * len(layers)
    if len(xs) != len(layers):
        raise ValueError("one input per layer (or one for all)")
    if not layers:
        return []
    flat, prepared = {}, []
    for layer, x in zip(layers, xs):
        if not layer.vaild:
            raise NotImplementedError("a BinaryLinear_2_4 layer holds no packed weight: call pack() first")
        if layer._prepared is None or layer._prepared.buffer.device != x.device:
            layer._prepared = PreparedWeight(layer.packed_binary_sparse.to(x.device), layer.meta.to(x.device))
        if id(x) not in flat:  # inputs shared by several layers are made contiguous fp16 once
            t = x.reshape(-1, layer.infeatures).to(torch.float16).contiguous()
            flat[id(x)] = t.clone() if t.data_ptr() % 16 else t
        prepared.append(flat[id(x)])
    tokens = prepared[0].shape[0]
    out_dtypes = {layer.out_dtype or (torch.float16 if x.dtype == torch.float16 else torch.float32)
                  for layer, x in zip(layers, xs)}
    bias_dtypes = {layer.bias.dtype if layer.bias.dtype in (torch.float16, torch.float32) else torch.float32
                   for layer in layers if layer.bias is not None}
    if tokens == 0 or len(out_dtypes) > 1 or len(bias_dtypes) > 1 or any(t.shape[0] != tokens for t in prepared):
        return [layer(x) for layer, x in zip(layers, xs)]  # nothing to share: the layers one by one
    out_dtype = out_dtypes.pop()
    problems, ys = [], []
    for layer, x, t in zip(layers, xs, prepared):
        bias = layer.bias
        if bias is not None:
            bias = bias.to(device=x.device, dtype=bias_dtypes and next(iter(bias_dtypes))).contiguous()
        y = torch.empty((tokens, layer.outfeatures), dtype=out_dtype, device=x.device)
        problems.append((layer._prepared.buffer, t, y, layer.outfeatures, layer.infeatures, bias))
        ys.append(y)
    _native.linear_prepared_grouped(problems)
    outs = []
    for layer, x, y in zip(layers, xs, ys):
        y = y.reshape(*x.shape[:-1], layer.outfeatures)
        outs.append(y if layer.out_dtype is not None else y.to(x.dtype))
    return outs
