"""Norms. LayerNorm with gain and offset, its epsilon a parameter (the reference fixes 1e-5 in
code: engine/src/gpt2_gpu.cu:15; formula engine/src/layernorm.c:15-33)."""

from __future__ import annotations

from ..ops import kernels
from ..weights.spec import VECTOR, Normal, TensorSpec
from .base import Norm, register_part


class LayerNorm(Norm):
    takes_pending = True

    def __init__(self, width: int, eps: float):
        self.width, self.eps = width, eps
        self.weight = None
        self.bias = None

    def tensor_specs(self):
        return {
            "weight": TensorSpec((self.width,), VECTOR, Normal(0.05, mean=1.0)),
            "bias": TensorSpec((self.width,), VECTOR, Normal(0.02)),
        }

    def forward(self, x, out_dtype, row_index=None):
        return kernels.layernorm(x, self.weight, self.bias, self.eps, out_dtype=out_dtype, row_index=row_index)

    def forward_into(self, x, out):
        return kernels.layernorm(x, self.weight, self.bias, self.eps, out_dtype=out.dtype, out=out)

    def forward_with_sums(self, hidden, out_dtype, packed=False):
        return kernels.layernorm(hidden, self.weight, self.bias, self.eps, out_dtype=out_dtype, with_sums=True, packed_out=packed)


class RMSNorm(Norm):
    """x / sqrt(mean(x^2) + eps) * g, in 32-bit. ``one_plus``: the stored vector lies around zero and g = 1 + weight.
    ``tensor_name``: the vector's name behind the part's prefix ("" where the part's own name is the tensor's). ``out_scale``: a
    constant that multiplies the normed rows, folded into the 32-bit gain when the weights are bound (a model whose logits are scaled
    gives its final norm the scale: the head's product is linear)."""

    def __init__(self, width: int, eps: float, one_plus: bool = False, tensor_name: str = "weight", out_scale: float = 1.0):
        if not eps > 0:
            raise ValueError(f"eps must be positive, not {eps}")
        if out_scale != 1.0 and one_plus:
            raise ValueError("a scale is folded into a plain gain vector, not into one stored around zero")
        self.width, self.eps, self.one_plus, self.out_scale = width, float(eps), bool(one_plus), float(out_scale)
        self._tensor_name = tensor_name
        self.weight = None

    def tensor_specs(self):
        return {self._tensor_name: TensorSpec((self.width,), VECTOR, Normal(0.05, mean=0.0 if self.one_plus else 1.0))}

    def bind(self, tensors):
        self.weight = tensors[self._tensor_name]
        if self.out_scale != 1.0:
            self.weight = (self.weight.double() * self.out_scale).float()

    def forward(self, x, out_dtype, row_index=None):
        return kernels.rms_norm(x, self.weight, self.eps, one_plus=self.one_plus, out_dtype=out_dtype, row_index=row_index)

    def forward_sum(self, x, addend, alpha, out_dtype):
        """norm(alpha * x + addend) -> kernels.NormedRows: the rows in float32 and in ``out_dtype``, from one kernel (a layer
        that norms after its sums goes on with both)."""
        if out_dtype == x.dtype:
            stream = kernels.rms_norm(x, self.weight, self.eps, addend=addend, alpha=alpha, one_plus=self.one_plus)
            return kernels.NormedRows(stream, stream)
        return kernels.NormedRows(*kernels.rms_norm(x, self.weight, self.eps, addend=addend, alpha=alpha, one_plus=self.one_plus,
                                                    out_dtype=out_dtype, with_stream=True))

    def forward_added(self, stream, branch, then=None, out_dtype=None):
        """stream + norm(branch) in float32 alone: for a layer whose next branch has a norm of its own in front. ``branch`` as for
        ``forward_onto``. ``then``: that next norm (an RMSNorm with the same eps and kind of gain, rows the kernel norms twice in one
        launch) and the element type its products read: the result is kernels.ReadyRows(sum, then(sum), then), from the one kernel."""
        addend = None
        if branch.dim() == 3:
            branch, addend = branch[0], (branch[1:] if branch.shape[0] > 1 else None)
        if then is None:
            return kernels.rms_norm(branch, self.weight, self.eps, addend=addend, one_plus=self.one_plus, residual=stream)
        if (isinstance(then, RMSNorm) and then.eps == self.eps and then.one_plus == self.one_plus and then.width == self.width
                and self.width <= kernels.RMS_NORM_TWICE_WIDTH):
            total, rows = kernels.rms_norm(branch, self.weight, self.eps, addend=addend, one_plus=self.one_plus, residual=stream, out_dtype=out_dtype,
                                           with_stream=True, next_weight=then.weight)
        else:
            total = kernels.rms_norm(branch, self.weight, self.eps, addend=addend, one_plus=self.one_plus, residual=stream)
            rows = then.forward(total, out_dtype)
        return kernels.ReadyRows(total, rows, then)

    def forward_onto(self, stream, branch, out_dtype):
        """stream + norm(branch) -> kernels.NormedRows: the sum of a layer whose norm sits on its branch's output, in float32 and in
        ``out_dtype``, from one kernel. ``branch``: float32 rows, or the partial products [n, rows, width] of a product cut along K,
        which are added up on the way in."""
        addend = None
        if branch.dim() == 3:
            branch, addend = branch[0], (branch[1:] if branch.shape[0] > 1 else None)
        if out_dtype == stream.dtype:
            total = kernels.rms_norm(branch, self.weight, self.eps, addend=addend, one_plus=self.one_plus, residual=stream)
            return kernels.NormedRows(total, total)
        return kernels.NormedRows(*kernels.rms_norm(branch, self.weight, self.eps, addend=addend, one_plus=self.one_plus, residual=stream,
                                                    out_dtype=out_dtype, with_stream=True))


register_part("norm", "layernorm", LayerNorm)
register_part("norm", "rmsnorm", RMSNorm)
