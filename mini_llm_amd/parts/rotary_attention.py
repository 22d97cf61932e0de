"""Softmax attention over the paged cache with rotated queries and keys and, optionally, rotated values.

With h the layer's input, H query heads, G key/value heads (query head j reads key/value head floor(j / (H / G))), ``dim`` elements to
a query or key and ``vdim`` to a value: q = W_q h, k = W_k h, v = W_v h (+ biases with ``biases``). ``rotary`` (pairing "half") turns the
first elements of every query and key by their position. ``value_rotary`` (any pairing, over the first ``value_rotary.dims`` elements of a
value, usually all): the value of position j is turned by j before it is kept, and every head's weighted sum at position i is turned
back by i, so that a value enters a sum turned by the distance j - i alone. score = scale q . k, causal, an ordinary softmax; W_o (+
bias) maps the heads laid behind each other back to the width.

``own_keys`` False: the layer has no key and value tensors and reads the pages another layer call keeps (the model's schedule names
it): that layer's keys after their rotation and its turned values, with queries of its own.

One product makes everything that reads h ([q | k | v], 32-bit sums, biases inside; ``carry_rows`` lays a block's own matrix behind them); ``kernels.map_rows`` (a head holding one map, no
norm) rotates and writes the pages; the framework's paged attention kernels do the rest, leaving the heads' sums in 32-bit where they
are turned back (``kernels.turn_heads``) before they are rounded for the output product. Heads of different key and value sizes are kept
in pages of the larger size (rounded to 16) with zeros behind."""

from __future__ import annotations

import torch

from ..ops import kernels
from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec
from .attention import MAX_HEAD_SIZE
from .base import KVNeed, LayerContext, Mixer, register_part
from .linear import BranchProduct, fuse_rows
from .positions import RotaryEncoding


class RotaryAttention(Mixer):
    graph_safe = True
    short_portion = kernels.DECODE_MAX_Q_LEN
    carries_rows = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: float, *, rotary: RotaryEncoding | None = None,
                 value_rotary: RotaryEncoding | None = None, biases: bool = True, own_keys: bool = True):
        if n_heads < 1 or n_kv_heads < 1 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} key/value heads")
        self.head_size = -(-max(dim, vdim) // 16) * 16
        if not 1 <= self.head_size <= MAX_HEAD_SIZE:
            raise ValueError(f"heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        if rotary is not None and (rotary.pairing != "half" or rotary.dims > dim or rotary.magnitude != 1.0):
            raise ValueError("this mixer rotates a head's first elements in the pairing of halves, at their own size")
        if value_rotary is not None and (value_rotary.dims > vdim or value_rotary.magnitude != 1.0):
            raise ValueError("values turn at their own size, over at most all their elements")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale, self.rotary, self.value_rotary = float(scale), rotary, value_rotary
        self.biases, self.own_keys = bool(biases), bool(own_keys)
        self.q_width, self.k_width, self.v_width, self.o_width = n_heads * dim, n_kv_heads * dim, n_kv_heads * vdim, n_heads * vdim
        self.w_in = self.b_in = self.o = self.o_bias = None
        self._out_product = BranchProduct()
        self.sums_later = False   # True: a call without a residual may return kernels.BranchRows (the block that adds the branch takes its sums)
        self._carried = {}        # name -> (matrix, bias) of rows that ride along in the input product
        self._carried_at = {}     # name -> (first column, columns) in the product's rows

    def carry_rows(self, name, matrix, bias=None):
        if matrix.dim() != 2 or matrix.shape[1] != self.width:
            raise ValueError(f"rows that ride along read the same {self.width} inputs")
        self._carried[name] = (matrix, bias)

    def _input_names(self):
        return ("q", "k", "v") if self.own_keys else ("q",)

    def tensor_specs(self):
        std = self.width ** -0.5
        widths = {"q": self.q_width, "k": self.k_width, "v": self.v_width}
        specs = {name: TensorSpec((widths[name], self.width), TABLE, Normal(std)) for name in self._input_names()}
        specs["o"] = TensorSpec((self.width, self.o_width), TABLE, Normal(self.o_width ** -0.5))
        if self.biases:
            for name in self._input_names():
                specs[name + ".b"] = TensorSpec((widths[name],), VECTOR, Normal(0.1))
            specs["o.b"] = TensorSpec((self.width,), VECTOR, Normal(0.1))
        return specs

    def bind(self, tensors):
        names = self._input_names()
        own = [tensors[name] for name in names]
        at = sum(t.shape[0] for t in own)
        self._carried_at = {}
        for rider, (matrix, _) in self._carried.items():
            self._carried_at[rider] = (at, matrix.shape[0])
            at += matrix.shape[0]
        fused = fuse_rows(own + [matrix.to(own[0].dtype) for matrix, _ in self._carried.values()])
        self.w_in = kernels.pack_matrix(fused) if fused.is_cuda else fused
        self.b_in = None
        if self.biases or any(bias is not None for _, bias in self._carried.values()):
            self.b_in = torch.zeros((fused.shape[0],), dtype=torch.float32, device=fused.device)
            at = 0
            for name in names:
                rows = tensors[name].shape[0]
                if self.biases:
                    self.b_in[at : at + rows] = tensors[name + ".b"]
                at += rows
            for rider, (_, bias) in self._carried.items():
                if bias is not None:
                    first, n = self._carried_at[rider]
                    self.b_in[first : first + n] = bias
        o = tensors["o"]
        self.o = kernels.pack_matrix(o.contiguous()) if o.is_cuda else o
        self.o_bias = tensors.get("o.b")

    def kv_need(self):
        return KVNeed(self.n_kv_heads, self.head_size, None)

    def forward(self, x, residual, ctx: LayerContext):
        """The branch alone (float32) when ``residual`` is None, else residual + branch."""
        batch = ctx.batch
        if ctx.write_cache != self.own_keys:
            raise ValueError("a layer with keys and values of its own writes its cache layer, and only such a layer does")
        fused = kernels.linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        if self._carried_at:
            ctx.extra["carried"] = {rider: fused[:, first : first + n] for rider, (first, n) in self._carried_at.items()}
        k_at = self.q_width if self.own_keys else None
        v_at = self.q_width + self.k_width if self.own_keys else None
        rotary, turn = self.rotary, self.value_rotary
        turn_dims = 0 if turn is None else turn.dims
        q = kernels.map_rows(fused, 0, k_at, v_at, None, None, 1.0, None if rotary is None else rotary.frequencies64(x.device),
                             0 if rotary is None else rotary.dims, batch.positions, ctx.group.slots, ctx.k_pages, ctx.v_pages, self.n_heads,
                             self.n_kv_heads, 1, self.dim, self.vdim, v_frequencies=turn.frequencies64(x.device) if turn_dims else None,
                             v_rot_dims=turn_dims, v_pairing="half" if turn is None else turn.pairing)
        reshape = turn_dims > 0 or self.head_size != self.vdim   # the heads' sums are turned back, or leave pages wider than the values
        mixed = kernels.paged_attention(
            q, ctx.k_pages, ctx.v_pages, batch.token_request, batch.positions, ctx.group.block_tables,
            self.n_heads, self.n_kv_heads, self.head_size, self.scale, max_q_len=batch.max_q_len, max_len=batch.max_total_len,
            q_starts=batch.q_starts, context_lens=batch.context_lens, first_row=getattr(batch, "first_row", 0), wide_out=reshape,
            **({"short_rows": batch.short_rows, "short_requests": batch.short_requests} if batch.short_portion <= kernels.DECODE_MAX_Q_LEN else {}),
        )
        if reshape:
            mixed = kernels.turn_heads(mixed, turn.frequencies64(x.device) if turn_dims else None, turn_dims, batch.positions, self.n_heads,
                                       self.head_size, self.vdim, sign=-1.0, pairing="half" if turn is None else turn.pairing, out_dtype=x.dtype)
        if residual is None and self.sums_later:
            return self._out_product.later(mixed, self.o, self.o_bias)
        return self._out_product(mixed, self.o, residual, bias=self.o_bias)


register_part("mixer", "rotary_attention", RotaryAttention)
