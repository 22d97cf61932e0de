"""A linear map y = x W + b as a part: weight stored [in, out] (GPT-2's Conv1D) or [out, in],
kept [out, in] for the matrix kernels, with the epilogue (activation, residual sum) fused."""

from __future__ import annotations

from ..ops import kernels
from ..weights.spec import MATRIX, VECTOR, Normal, TensorSpec
from .base import Part


class Linear(Part):
    def __init__(self, in_features: int, out_features: int, *, bias: bool = True, stored_in_out: bool = True,
                 weight_std: float = 0.02, bias_std: float = 0.01):
        self.in_features, self.out_features = in_features, out_features
        self.has_bias, self.stored_in_out = bias, stored_in_out
        self.weight_std, self.bias_std = weight_std, bias_std
        self.weight = None
        self.bias = None
        self._split_blocks = {}
        self._accepts_packed = {}

    def tensor_specs(self):
        shape = (self.in_features, self.out_features) if self.stored_in_out else (self.out_features, self.in_features)
        specs = {"weight": TensorSpec(shape, MATRIX, Normal(self.weight_std), keep_transposed=self.stored_in_out)}
        if self.has_bias:
            specs["bias"] = TensorSpec((self.out_features,), VECTOR, Normal(self.bias_std))
        return specs

    def forward(self, x, activation=None, residual=None, out_dtype=None, packed_out=False):
        return kernels.linear(x, self.weight, self.bias, activation=activation, residual=residual, out_dtype=out_dtype, packed_out=packed_out)

    def accepts_packed_rows(self, rows: int, dtype, pending: bool = False) -> bool:
        """Whether ``forward`` (or, with ``pending``, ``forward_pending``) of so many rows reads them in
        the packed layout (kernels.PackedRows): where the product takes the kernel for few rows."""
        key = (rows, dtype, pending)
        answer = self._accepts_packed.get(key)
        if answer is None:
            answer = kernels.takes_packed_rows(rows, self.weight, dtype)
            if pending and rows <= 64 and kernels.split_blocks(self.weight, dtype, rows) > 1:
                answer = True   # the partial products of few rows come from that kernel whatever the matrix
            self._accepts_packed[key] = answer
        return answer

    def forward_pending(self, x, residual):
        """residual + x W + b, as float32 rows or, where few rows meet few output columns and a long
        K, as rows whose sums are pending: the product cut along K into partial products, which
        whoever reads the rows next adds up (kernels.PendingRows)."""
        rows = x.shape[0]
        bucket = 0 if rows <= 64 else -(-rows // 128)  # the answer is the same inside a bucket
        k_blocks = self._split_blocks.get((bucket, x.dtype))
        if k_blocks is None:
            k_blocks = self._split_blocks[bucket, x.dtype] = kernels.split_blocks(self.weight, x.dtype, rows)
        if k_blocks > 1:
            return kernels.PendingRows(residual, kernels.linear_split(x, self.weight, k_blocks), self.bias)
        return self.forward(x, residual=residual)


class BranchProduct:
    """The last product of a branch whose sum with the stream is taken by the norm behind it: x W^T in float32, as plain rows
    or, where few rows meet few output columns and a long K (the library says: ``kernels.split_blocks``), cut along K into
    partial products [n, rows, out] that the norm adds up on its way in. With a residual the sum is taken inside the product, and
    so is a bias's.
    Up to FEW_ROWS rows the product stays whole: measured on MI355X at width 768, a decode step of 64 rows gains 5 % from the
    cut (0.990 -> 0.939 ms), one of 8 rows or of a single row loses 3 % (the norm's extra trips to memory cost more than the
    product saves)."""

    FEW_ROWS = 16

    def __init__(self):
        self._split_blocks = {}

    def blocks(self, x, weight) -> int:
        """Into how many partial products the product of these rows is cut (1: it stays whole)."""
        rows = x.shape[0]
        if rows <= self.FEW_ROWS:
            return 1
        bucket = 0 if rows <= 64 else -(-rows // 128)   # the answer is the same inside a bucket
        k_blocks = self._split_blocks.get((bucket, x.dtype))
        if k_blocks is None:
            k_blocks = self._split_blocks[bucket, x.dtype] = kernels.split_blocks(weight, x.dtype, rows)
        return k_blocks

    def __call__(self, x, weight, residual=None, bias=None):
        import torch

        if residual is None and bias is None:
            k_blocks = self.blocks(x, weight)
            if k_blocks > 1:
                return kernels.linear_split(x, weight, k_blocks)
        return kernels.linear(x, weight, bias, residual=residual, out_dtype=torch.float32)

    def later(self, x, weight, bias=None, spare: int = 0):
        """For a branch whose sum with the stream is taken by a kernel that also takes a bias and partial products
        (``kernels.branch_join``): ``kernels.BranchRows`` of the product, cut along K where that pays, and the bias, not yet added. ``spare``:
        so many more matrices of the product's shape are kept behind the partial products for the caller to fill (they join the sum)."""
        import torch

        k_blocks = self.blocks(x, weight)
        if k_blocks == 1 and not spare:
            return kernels.BranchRows(kernels.linear(x, weight, out_dtype=torch.float32), bias)
        out = torch.empty((k_blocks + spare, x.shape[0], weight.rows if isinstance(weight, kernels.PackedMatrix) else weight.shape[0]),
                          dtype=torch.float32, device=x.device if hasattr(x, "device") else x.data.device)
        if k_blocks == 1:
            kernels.linear(x, weight, out_dtype=torch.float32, out=out[0])
        else:
            kernels.linear_split(x, weight, k_blocks, out=out)
        return kernels.BranchRows(out, bias)


def fuse_rows(matrices, multiple: int = 16):
    """The matrices of several products over the same input laid behind each other ([out, in] each), zero rows added up to a multiple
    of ``multiple`` outputs: the products of many rows stream only matrices whose outputs are a multiple of 8, and the ones of few
    rows take 16 outputs a block. The caller reads the columns it knows of the fused product and leaves the rest alone."""
    import torch

    fused = torch.cat(list(matrices), dim=0)
    spare = -fused.shape[0] % multiple
    if spare:
        fused = torch.cat([fused, torch.zeros((spare, fused.shape[1]), dtype=fused.dtype, device=fused.device)], dim=0)
    return fused.contiguous()
