"""A feed-forward of routed experts: many small feed-forwards of which a router picks a few for every row.

With h the layer's input and E = ``n_experts`` + ``n_identity`` router outputs: z = W_router h in 32-bit, scores s = softmax(z) over all E.
The choice goes by s + ``correction`` (a stored vector; the weights do not see it): the experts form ``n_groups`` equal groups of
neighbours, a group counts by the largest choice score in it, only experts of the best ``keep`` groups can be picked, and the ``top``
largest choice scores among those are. The picked experts' weights are their scores s over (their sum + ``floor``). Expert e is W_down,e
act(W_up,e h) with act the square of relu, no biases; the last ``n_identity`` router outputs are experts without tensors whose result is
h itself. The result is the weighted sum over the picked experts, plus (``shared_ff``) one more expert of the same form that every row
uses with weight 1.

All experts run as ONE up product over their matrices laid behind each other (the shared expert's last) and ONE down product over their
down matrices laid side by side: ``kernels.expert_unit`` between the two multiplies every hidden unit by its expert's weight for the
row, zero where the router did not pick it, so the down product's sum is the weighted sum over the picked experts; the share of the
experts that hand h on rides in as that product's residual operand. A row's result is a function of the row alone, nothing is planned
on the host, and a captured step replays it. The price is the arithmetic of the experts that were not picked: E / top times the needed
work in the two products, which few rows (decoding) do not notice, since they read every expert's matrices anyway."""

from __future__ import annotations

import torch

from ..ops import kernels
from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec
from .base import FeedForward, register_part
from .linear import BranchProduct, fuse_rows


class RoutedExperts(FeedForward):
    def __init__(self, width: int, n_experts: int, ff: int, top: int, *, n_identity: int = 0, n_groups: int = 1, keep: int = 1,
                 correction: bool = True, shared_ff: int | None = None, floor: float = 0.0):
        total = n_experts + n_identity
        if n_experts < 0 or n_identity < 0 or total < 1 or total > kernels.ROUTE_MAX_EXPERTS:
            raise ValueError(f"{n_experts} experts and {n_identity} that hand their input on: the router takes 1 to {kernels.ROUTE_MAX_EXPERTS} outputs")
        if n_groups < 1 or total % n_groups or not 1 <= keep <= n_groups:
            raise ValueError(f"{total} router outputs do not form {n_groups} equal groups of which {keep} are kept")
        if not 1 <= top <= keep * (total // n_groups):
            raise ValueError(f"{top} experts cannot be picked among {keep} groups of {total // n_groups}")
        self.width, self.n_experts, self.ff, self.top, self.n_identity = width, n_experts, ff, top, n_identity
        self.n_groups, self.keep, self.has_correction, self.shared_ff, self.floor = n_groups, keep, bool(correction), shared_ff or 0, float(floor)
        self.n_outputs = total
        self.router = self.correction = self.up = self.down = self._router_rows = None
        self.shared_units = 0   # the shared expert's hidden units and the zeros that fill the up matrix to whole blocks
        self._down_product = BranchProduct()
        self.sums_later = False   # True: a call without a residual may return kernels.BranchRows (the block that adds the branch takes its sums)

    def tensor_specs(self):
        specs = {"router": TensorSpec((self.n_outputs, self.width), TABLE, Normal(self.width ** -0.5))}
        if self.has_correction:
            specs["correction"] = TensorSpec((self.n_outputs,), VECTOR, Normal(0.05))
        names = [f"e{e}." for e in range(self.n_experts)]
        sizes = [self.ff] * self.n_experts
        if self.shared_ff:
            names.append("shared.")
            sizes.append(self.shared_ff)
        for name, size in zip(names, sizes):
            specs[name + "up"] = TensorSpec((size, self.width), TABLE, Normal(self.width ** -0.5))
            specs[name + "down"] = TensorSpec((self.width, size), TABLE, Normal(size ** -0.5))
        return specs

    def bind(self, tensors):
        names = [f"e{e}." for e in range(self.n_experts)] + (["shared."] if self.shared_ff else [])
        router = fuse_rows([tensors["router"]])
        self._router_rows = router
        self.router = kernels.pack_matrix(router) if router.is_cuda else router
        self.correction = tensors.get("correction")
        up = fuse_rows([tensors[name + "up"] for name in names]) if names else None
        if up is None:
            return
        self.shared_units = up.shape[0] - self.n_experts * self.ff
        down = torch.cat([tensors[name + "down"] for name in names], dim=1)
        spare = up.shape[0] - down.shape[1]
        if spare:   # the zero hidden units that fill the up matrix meet zero columns
            down = torch.cat([down, torch.zeros((down.shape[0], spare), dtype=down.dtype, device=down.device)], dim=1)
        down = down.contiguous()
        self.up, self.down = (kernels.pack_matrix(up), kernels.pack_matrix(down)) if up.is_cuda else (up, down)

    def rows_to_carry(self):
        """The router's matrix (and no bias), for a block that lets another product over the same input rows carry it along; ``forward`` is
        then given the router's sums as ``carried``."""
        return self._router_rows, None

    def forward(self, x, residual, carried=None):
        logits = carried if carried is not None else kernels.linear(x, self.router, out_dtype=torch.float32)
        weights = kernels.route(logits, self.n_outputs, self.top, correction=self.correction, n_groups=self.n_groups, keep=self.keep, floor=self.floor)
        if self.up is None:   # nothing but experts that hand their input on
            raise ValueError("a routed feed-forward needs at least one expert with matrices")
        if residual is None and self.sums_later:
            # the share of the experts that hand h on lies behind the down product's partial products and joins their sum
            spare = 1 if self.n_identity else 0
            hidden = kernels.linear(x, self.up)
            k_blocks = self._down_product.blocks(hidden, self.down)
            out = torch.empty((k_blocks + spare, hidden.shape[0], self.width), dtype=torch.float32, device=hidden.device)
            units, _ = kernels.expert_unit(hidden, weights, self.n_experts, self.ff, self.shared_units, h=x, n_identity=self.n_identity,
                                           carried_out=out[k_blocks] if spare else None)
            if k_blocks == 1:
                kernels.linear(units, self.down, out_dtype=torch.float32, out=out[0])
            else:
                kernels.linear_split(units, self.down, k_blocks, out=out)
            return kernels.BranchRows(out, None)
        units, carried = kernels.expert_unit(kernels.linear(x, self.up), weights, self.n_experts, self.ff, self.shared_units, h=x, n_identity=self.n_identity)
        if carried is not None and residual is not None:
            carried = kernels.add(carried, residual)
        return self._down_product(units, self.down, carried if carried is not None else residual)


register_part("feed_forward", "routed_experts", RoutedExperts)
