"""Dense feed-forward: up projection, activation, down projection, residual sum
(engine/src/transformer_block.c:64-71). The activation is fused into the up product and the
residual sum into the down product."""

from __future__ import annotations

import torch

from ..ops import kernels
from .base import FeedForward, register_part
from .linear import BranchProduct, Linear
from .norms import LayerNorm

ACTIVATIONS = ("gelu_new", "gelu")


class DenseMLP(FeedForward):
    def __init__(self, width: int, inner: int, activation: str, down_std: float = 0.02,
                 up_name: str = "c_fc.", down_name: str = "c_proj."):
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {ACTIVATIONS}")
        self.width, self.inner, self.activation = width, inner, activation
        self.up = Linear(width, inner)
        self.down = Linear(inner, width, weight_std=down_std)
        self._names = (up_name, down_name)

    def children(self):
        return {self._names[0]: self.up, self._names[1]: self.down}

    def forward(self, x, residual):
        return self.down.forward(self.up.forward(x, activation=self.activation), residual=residual)

    def forward_normed(self, hidden, norm, compute_dtype, ctx):
        # few rows: the whole chain in one kernel, cut along the hidden units
        if (hidden.shape[0] <= kernels.layer_kernel_rows(self.width) and ctx.batch.max_q_len == 1 and isinstance(norm, LayerNorm)
                and ctx.batch.max_total_len <= kernels.decode_layer_reach(hidden.shape[0])   # changes with the attention half
                and isinstance(self.up.weight, kernels.PackedMatrix) and isinstance(self.down.weight, kernels.PackedMatrix)
                and self.up.weight.dtype == torch.bfloat16 and kernels.decode_layer_supported(self.width, inner=self.inner)):
            return kernels.decode_mlp_half(hidden, norm.weight, norm.bias, norm.eps, self.up.weight, self.up.bias,
                                           self.down.weight, self.down.bias, activation=self.activation)
        # else kernel by kernel; the down product of few rows may come back with its sums pending, and
        # few rows go from kernel to kernel in the packed layout, which the products read faster
        rows = hidden.shape[0]
        few = kernels.PACKED_ROWS_FROM <= rows <= 64
        x, hidden = norm.forward_with_sums(hidden, compute_dtype, packed=few and self.up.accepts_packed_rows(rows, compute_dtype))
        packed_out = few and self.up.accepts_packed_rows(rows, compute_dtype) and self.down.accepts_packed_rows(rows, compute_dtype, pending=True)
        return self.down.forward_pending(self.up.forward(x, activation=self.activation, packed_out=packed_out), hidden)


class GatedMLP(FeedForward):
    """down(silu(gate x) * (up x)), no biases; the three matrices are stored [out, in] under their bare names. Gate and up run
    as one product over the two matrices laid behind each other, the activation and the multiplication as one kernel over its
    halves, and the residual sum (if a residual is given) inside the down product."""

    def __init__(self, width: int, inner: int, names=("gate", "up", "down")):
        self.width, self.inner = width, inner
        self._names = names
        self.gate_up = self.down = None
        self._down_product = BranchProduct()

    def tensor_specs(self):
        from ..weights.spec import MATRIX, TABLE, Normal, TensorSpec

        gate, up, down = self._names
        return {gate: TensorSpec((self.inner, self.width), TABLE, Normal(self.width ** -0.5)),
                up: TensorSpec((self.inner, self.width), TABLE, Normal(self.width ** -0.5)),
                down: TensorSpec((self.width, self.inner), MATRIX, Normal(self.inner ** -0.5))}

    def bind(self, tensors):
        gate, up, down = (tensors[name] for name in self._names)
        self.gate_up = kernels.pack_matrix(torch.cat([gate, up], dim=0).contiguous()) if gate.is_cuda else torch.cat([gate, up], dim=0)
        self.down = down

    def forward(self, x, residual):
        inner = kernels.silu_mul(kernels.linear(x, self.gate_up))
        return self._down_product(inner, self.down, residual)


class ClampedGatedMLP(FeedForward):
    """down(g * sigmoid(alpha g) * (u + shift)) with g = min(gate x, limit) and u = clamp(up x, -limit, limit) (``limit`` None:
    unclamped); with ``biases`` every product has one, stored under the matrix's name + ".b". Gate and up run as one product over the
    two matrices laid behind each other (biases inside), the gate unit as one kernel over its halves."""

    def __init__(self, width: int, inner: int, limit: float | None, alpha: float = 1.0, shift: float = 0.0, biases: bool = True,
                 names=("gate", "up", "down")):
        if limit is not None and not limit > 0:
            raise ValueError(f"the limit must be positive, not {limit}")
        self.width, self.inner, self.limit, self.alpha, self.shift, self.biases = width, inner, limit, float(alpha), float(shift), bool(biases)
        self._names = names
        self.gate_up = self.gate_up_bias = self.down = self.down_bias = None
        self._down_product = BranchProduct()
        self.sums_later = False   # True: a call without a residual may return kernels.BranchRows (the block that adds the branch takes its sums)

    def tensor_specs(self):
        from ..weights.spec import MATRIX, TABLE, VECTOR, Normal, TensorSpec

        gate, up, down = self._names
        specs = {gate: TensorSpec((self.inner, self.width), TABLE, Normal(self.width ** -0.5)),
                 up: TensorSpec((self.inner, self.width), TABLE, Normal(self.width ** -0.5)),
                 down: TensorSpec((self.width, self.inner), MATRIX, Normal(self.inner ** -0.5))}
        if self.biases:
            specs[gate + ".b"] = TensorSpec((self.inner,), VECTOR, Normal(0.1))
            specs[up + ".b"] = TensorSpec((self.inner,), VECTOR, Normal(0.1))
            specs[down + ".b"] = TensorSpec((self.width,), VECTOR, Normal(0.1))
        return specs

    def bind(self, tensors):
        gate, up, down = self._names
        both = torch.cat([tensors[gate], tensors[up]], dim=0).contiguous()
        self.gate_up = kernels.pack_matrix(both) if both.is_cuda else both
        self.down = tensors[down]
        if self.biases:
            self.gate_up_bias = torch.cat([tensors[gate + ".b"], tensors[up + ".b"]]).contiguous()
            self.down_bias = tensors[down + ".b"]

    def forward(self, x, residual):
        inner = kernels.gate_unit(kernels.linear(x, self.gate_up, self.gate_up_bias), self.limit, self.alpha, self.shift)
        if residual is None and self.sums_later:
            return self._down_product.later(inner, self.down, self.down_bias)
        return self._down_product(inner, self.down, residual, bias=self.down_bias)


register_part("feed_forward", "dense_mlp", DenseMLP)
register_part("feed_forward", "clamped_gated_mlp", ClampedGatedMLP)
register_part("feed_forward", "gated_mlp", GatedMLP)
