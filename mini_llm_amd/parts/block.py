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


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "branch_norm", BranchNormBlock)
