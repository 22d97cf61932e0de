"""Arrangements of norm, mixer and feed-forward in a layer. GPT-2's is pre-norm: a norm before
the mixer and one before the feed-forward, each branch added to the residual stream
(engine/src/transformer_block.c:49-71)."""

from __future__ import annotations

from .base import Block, FeedForward, LayerContext, Mixer, Norm, register_part


class PreNormBlock(Block):
    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm, feed_forward: FeedForward, compute_dtype,
                 names=("ln_1.", "attn.", "ln_2.", "mlp.")):
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.compute_dtype = compute_dtype
        self._names = names

    def children(self):
        return dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))

    def mixer_part(self):
        return self.mixer

    takes_pending = True

    def forward(self, hidden, ctx: LayerContext):
        hidden = self.mixer.forward_normed(hidden, self.norm_1, self.compute_dtype, ctx)
        return self.feed_forward.forward_normed(hidden, self.norm_2, self.compute_dtype, ctx)


class PostNormBlock(Block):
    """Norm after the sum: x <- norm_1(alpha * x + mixer(x)), then x <- norm_2(alpha * x + feed_forward(x)); the branches
    read x itself. ``alpha`` scales the stream in both sums. ``feed_forward`` None: the layer ends behind its mixer. The norms
    have ``forward_sum`` (RMSNorm), and mixer and feed-forward return their branch alone when given no residual."""

    takes_pending = True   # takes plain rows, pending rows or a norm's NormedRows, and returns NormedRows

    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm | None, feed_forward: FeedForward | None, alpha: float, compute_dtype,
                 names=("norm1", "mix.", "norm2", "mlp.")):
        if (norm_2 is None) != (feed_forward is None):
            raise ValueError("the second norm goes with the feed-forward")
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.alpha, self.compute_dtype = float(alpha), compute_dtype
        self._names = names

    def children(self):
        parts = dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))
        return {name: part for name, part in parts.items() if part is not None}

    def mixer_part(self):
        return self.mixer

    def forward(self, hidden, ctx: LayerContext):
        from ..ops import kernels

        if not isinstance(hidden, kernels.NormedRows):
            stream = kernels.settle(hidden)
            hidden = kernels.NormedRows(stream, stream if self.compute_dtype == stream.dtype else kernels.convert(stream, self.compute_dtype))
        hidden = self.norm_1.forward_sum(hidden.stream, self.mixer.forward(hidden.rows, None, ctx), self.alpha, self.compute_dtype)
        if self.feed_forward is None:
            return hidden
        return self.norm_2.forward_sum(hidden.stream, self.feed_forward.forward(hidden.rows, None), self.alpha, self.compute_dtype)


class BranchNormBlock(Block):
    """Norm on each branch's output: x <- x + norm_1(mixer(x)), then x <- x + norm_2(feed_forward(x)); the branches read the
    stream itself. ``feed_forward`` None: the layer ends behind its mixer. The norms have ``forward_onto`` (RMSNorm), and mixer and
    feed-forward return their branch alone when given no residual. The stream travels as kernels.NormedRows: in float32 and, the
    same numbers, in the compute type that the next branch's products read."""

    takes_pending = True

    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm | None, feed_forward: FeedForward | None, compute_dtype,
                 names=("norm1", "mix.", "norm2", "mlp.")):
        if (norm_2 is None) != (feed_forward is None):
            raise ValueError("the second norm goes with the feed-forward")
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.compute_dtype = compute_dtype
        self._names = names

    def children(self):
        parts = dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))
        return {name: part for name, part in parts.items() if part is not None}

    def mixer_part(self):
        return self.mixer

    def forward(self, hidden, ctx: LayerContext):
        from ..ops import kernels

        if not isinstance(hidden, kernels.NormedRows):
            stream = kernels.settle(hidden)
            hidden = kernels.NormedRows(stream, stream if self.compute_dtype == stream.dtype else kernels.convert(stream, self.compute_dtype))
        hidden = self.norm_1.forward_onto(hidden.stream, self.mixer.forward(hidden.rows, None, ctx), self.compute_dtype)
        if self.feed_forward is None:
            return hidden
        return self.norm_2.forward_onto(hidden.stream, self.feed_forward.forward(hidden.rows, None), self.compute_dtype)


class SandwichNormBlock(Block):
    """A norm in front of each branch and one on its output: x <- x + norm_1b(mixer(norm_1(x))), then x <- x + norm_2b(feed_forward(norm_2(x))).
    ``feed_forward`` None: the layer ends behind its mixer. The stream is float32 rows; the norms on the outputs have ``forward_added``
    (RMSNorm: stream + norm(branch) from one kernel, which also adds up the partial products of a branch whose last product was cut
    along K, and norms the sum once more for the branch that follows), and mixer and feed-forward return their branch alone when given
    no residual. ``hand_to(norm)``: the norm that reads this layer's output next (the following layer's ``norm_1``); the layer then
    returns kernels.ReadyRows, its stream and what that norm makes of it, and a layer that is handed such rows made by its own
    ``norm_1`` does not run it again. A layer is so two norm kernels for a branch's four norms."""

    takes_pending = True   # takes plain rows, pending rows or the ReadyRows of the layer before

    def __init__(self, norm_1: Norm, mixer: Mixer, norm_1b: Norm, norm_2: Norm | None, feed_forward: FeedForward | None, norm_2b: Norm | None,
                 compute_dtype, names=("norm1", "mix.", "norm1b", "norm2", "mlp.", "norm2b")):
        if not ((norm_2 is None) == (feed_forward is None) == (norm_2b is None)):
            raise ValueError("the second pair of norms goes with the feed-forward")
        self.norm_1, self.mixer, self.norm_1b, self.norm_2, self.feed_forward, self.norm_2b = norm_1, mixer, norm_1b, norm_2, feed_forward, norm_2b
        self.compute_dtype = compute_dtype
        self._names = names
        self._following = None

    def children(self):
        parts = dict(zip(self._names, (self.norm_1, self.mixer, self.norm_1b, self.norm_2, self.feed_forward, self.norm_2b)))
        return {name: part for name, part in parts.items() if part is not None}

    def mixer_part(self):
        return self.mixer

    def hand_to(self, norm: Norm | None):
        self._following = norm

    def _added(self, norm, stream, branch, then):
        if then is None or not hasattr(norm, "forward_added"):
            return norm.forward_added(stream, branch)
        return norm.forward_added(stream, branch, then=then, out_dtype=self.compute_dtype)

    def forward(self, hidden, ctx: LayerContext):
        from ..ops import kernels

        if isinstance(hidden, kernels.ReadyRows) and hidden.norm is self.norm_1:
            stream, rows = hidden.stream, hidden.rows
        else:
            stream = kernels.settle(hidden)
            rows = self.norm_1.forward(stream, self.compute_dtype)
        hidden = self._added(self.norm_1b, stream, self.mixer.forward(rows, None, ctx), self.norm_2 if self.feed_forward is not None else self._following)
        if self.feed_forward is None:
            return hidden
        return self._added(self.norm_2b, hidden.stream, self.feed_forward.forward(hidden.rows, None), self._following)


class ParallelBlock(Block):
    """One norm, both branches side by side on its output: with h = norm_1(x), x <- x + mult * (s1 * g1 * mixer(h) + s2 * g2 *
    feed_forward(h)). ``feed_forward`` None: the layer has its mixer alone. ``layer_scale``: s1, s2 are stored vectors (``ls1``,
    ``ls2``) that multiply a branch's result element by element (else 1). ``gated``: g1 = sigmoid(W1 h + b1), g2 = sigmoid(W2 h + b2) with
    stored matrices ``rg1``, ``rg2`` [width, width] and biases ``rg1.b``, ``rg2.b`` (else 1); both gates come from one product over the two
    matrices laid behind each other, in 32-bit: the mixer's own first product where it can carry them (``Mixer.carries_rows``). The sum is one kernel (``kernels.branch_join``: it also adds up the partial products of a
    branch whose last product was cut along K), which norms the sum for the layer that follows where that layer's first norm is known
    (``hand_to``): the layer then returns kernels.ReadyRows, and a layer that is handed rows made by its own ``norm_1`` does not run it."""

    takes_pending = True   # takes plain rows, pending rows or the ReadyRows of the layer before

    def __init__(self, norm_1: Norm, mixer: Mixer, feed_forward: FeedForward | None, width: int, compute_dtype, *, mult: float = 1.0,
                 layer_scale: bool = False, gated: bool = False, names=("norm1", "mix.", "mlp.")):
        self.norm_1, self.mixer, self.feed_forward = norm_1, mixer, feed_forward
        self.width, self.compute_dtype, self.mult, self.layer_scale, self.gated = width, compute_dtype, float(mult), bool(layer_scale), bool(gated)
        self._names = names
        self._following = None
        self._feed_forward_rides = False
        self.scale_1 = self.scale_2 = self.gates = self.gates_bias = None
        for part in (mixer, feed_forward):   # the sum's kernel takes a branch's bias and the partial products of its last product
            if part is not None and hasattr(part, "sums_later"):
                part.sums_later = True

    def children(self):
        parts = dict(zip(self._names, (self.norm_1, self.mixer, self.feed_forward)))
        return {name: part for name, part in parts.items() if part is not None}

    def mixer_part(self):
        return self.mixer

    def hand_to(self, norm: Norm | None):
        self._following = norm

    def _branches(self):
        return ("1", "2") if self.feed_forward is not None else ("1",)

    def tensor_specs(self):
        from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec

        specs = {}
        for n in self._branches():
            if self.layer_scale:
                specs["ls" + n] = TensorSpec((self.width,), VECTOR, Normal(0.2, mean=1.0))
            if self.gated:
                specs["rg" + n] = TensorSpec((self.width, self.width), TABLE, Normal(self.width ** -0.5))
                specs["rg" + n + ".b"] = TensorSpec((self.width,), VECTOR, Normal(0.5))
        return specs

    def bind(self, tensors):
        import torch

        from ..ops import kernels
        from .linear import fuse_rows

        if self.layer_scale:
            self.scale_1, self.scale_2 = tensors["ls1"], tensors.get("ls2")
        if self.gated:
            fused = fuse_rows([tensors["rg" + n] for n in self._branches()])
            self.gates_bias = torch.zeros((fused.shape[0],), dtype=torch.float32, device=fused.device)
            for index, n in enumerate(self._branches()):
                self.gates_bias[index * self.width : (index + 1) * self.width] = tensors["rg" + n + ".b"]
            if self.mixer.carries_rows:   # the gates ride along in the mixer's own first product (the mixer is bound after this part)
                self.mixer.carry_rows("gates", fused, self.gates_bias)
                self.gates = None
            else:
                self.gates = kernels.pack_matrix(fused) if fused.is_cuda else fused
        self._ride_feed_forward()

    def _ride_feed_forward(self):
        """A feed-forward whose first small product reads the layer's input rows (a router) sends it along in the mixer's too."""
        rider = getattr(self.feed_forward, "rows_to_carry", None)
        self._feed_forward_rides = False
        if rider is not None and self.mixer.carries_rows:
            rows = rider()
            if rows is not None:
                self.mixer.carry_rows("feed_forward", *rows)
                self._feed_forward_rides = True

    def bind_named(self, tensors: dict, prefix: str = "") -> None:
        # the feed-forward first, this part's own tensors next, the mixer last: both may hand rows to the mixer, which lays them behind its
        # own when it is bound
        if self.feed_forward is not None:
            self.feed_forward.bind_named(tensors, prefix + self._names[2])
        own = {name: tensors[prefix + name] for name in self.tensor_specs()}
        if own:
            self.bind(own)
        else:
            self._ride_feed_forward()
        self.norm_1.bind_named(tensors, prefix + self._names[0])
        self.mixer.bind_named(tensors, prefix + self._names[1])

    def forward(self, hidden, ctx: LayerContext):
        import torch

        from ..ops import kernels

        if isinstance(hidden, kernels.ReadyRows) and hidden.norm is self.norm_1:
            stream, rows = hidden.stream, hidden.rows
        else:
            stream = kernels.settle(hidden)
            rows = self.norm_1.forward(stream, self.compute_dtype)
        gates = kernels.linear(rows, self.gates, self.gates_bias, out_dtype=torch.float32) if self.gated and self.gates is not None else None
        first = self.mixer.forward(rows, None, ctx)
        carried = ctx.extra.pop("carried", {})
        if self.gated and self.gates is None:
            gates = carried["gates"]
        second = None
        if self.feed_forward is not None:
            second = self.feed_forward.forward(rows, None, carried=carried["feed_forward"]) if self._feed_forward_rides else self.feed_forward.forward(rows, None)
        following = self._following
        ahead = {}
        if following is not None and hasattr(following, "one_plus") and getattr(following, "out_scale", 1.0) == 1.0:
            ahead = dict(next_weight=following.weight, one_plus=following.one_plus, eps=following.eps, out_dtype=self.compute_dtype)
        joined = kernels.branch_join(stream, first, second, scale_a=self.scale_1, scale_b=self.scale_2, gates=gates, gate_a_at=0, gate_b_at=self.width,
                                     mult=self.mult, **ahead)
        return kernels.ReadyRows(joined[0], joined[1], following) if ahead else joined


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "branch_norm", BranchNormBlock)
