"""Differential attention over the paged cache: every head holds two attention maps over the same values, and the second is
subtracted from the first.

With h the layer's input, H query heads, G key/value heads (query head j reads key/value head floor(j / (H / G))), ``dim`` elements to
a query or key of one map and ``vdim`` to a value: q = W_q h + b_q is [H, 2, dim] (head by head, map 1 then map 2), k = W_k h + b_k
is [G, 2, dim], v = W_v h + b_v is [G, vdim]. Every query and key of every map is RMS-normed over its dim elements (one gain vector
of dim for all queries, one for all keys), then the rotation (``rotary``: pairing "half") turns its first elements by the position.
Each map is an ordinary causal softmax attention with score = scale q . k over the keys the mask lets through (``chunk``: only the
keys of the query's own chunk of so many positions, chunks counted from position 0; None: all keys up to the query). With a1, a2 the
two maps' results of a head and lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number a layer from four learned vectors: x = a1 -
lam a2, a head's result is x / rms(x) * (1 - diff), times sigmoid(W_g h) element by element, and W_o maps the heads laid behind each
other back to the width.

``own_keys`` False: the layer has no key and value tensors and reads the pages another layer call keeps (the model's schedule names
it), with queries, mask and everything else of its own.

One product makes everything that reads h ([q | k | v | g], 32-bit sums); ``kernels.map_rows`` norms, rotates and writes the pages;
the framework's paged attention kernels run the 2 H maps as heads of their own over 2 G key heads (a value head is stored under
each of its two maps, so that the kernels' grouping of heads serves unchanged) and leave their results in 32-bit, because a
difference of two maps that see nearly the same keys multiplies whatever rounding they carry; ``kernels.map_difference`` subtracts,
norms and gates. Heads of different key and value sizes are kept in pages of the larger size (rounded to 16) with zeros behind."""

from __future__ import annotations

import math

import torch

from ..ops import kernels
from ..weights.spec import TABLE, VECTOR, Normal, TensorSpec
from .attention import MAX_HEAD_SIZE
from .base import KVNeed, LayerContext, Mixer, register_part
from .linear import BranchProduct, fuse_rows
from .positions import RotaryEncoding

MAPS = 2


class DifferentialAttention(Mixer):
    graph_safe = True
    short_portion = kernels.DECODE_MAX_Q_LEN

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: float, diff: float, eps: float, *,
                 rotary: RotaryEncoding | None = None, chunk: int | None = None, own_keys: bool = True):
        if n_heads < 1 or n_kv_heads < 1 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {n_kv_heads} key/value heads")
        self.head_size = -(-max(dim, vdim) // 16) * 16
        if not 1 <= self.head_size <= MAX_HEAD_SIZE:
            raise ValueError(f"heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        if rotary is not None and (rotary.pairing != "half" or rotary.dims > dim or rotary.magnitude != 1.0):
            raise ValueError("this mixer rotates a map's first elements in the pairing of halves, at their own size")
        if chunk is not None and chunk < 1:
            raise ValueError(f"chunks of {chunk} positions")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale, self.diff, self.eps, self.rotary, self.chunk, self.own_keys = float(scale), float(diff), float(eps), rotary, chunk, bool(own_keys)
        self.q_width, self.k_width, self.v_width, self.g_width = n_heads * MAPS * dim, n_kv_heads * MAPS * dim, n_kv_heads * vdim, n_heads * vdim
        self.w_in = self.b_in = self.o = self.q_norm = self.k_norm = None
        self.lam = None   # the weight of the second map, known once the tensors are bound
        self._out_product = BranchProduct()

    def tensor_specs(self):
        std = self.width ** -0.5
        specs = {"q": TensorSpec((self.q_width, self.width), TABLE, Normal(std)),
                 "q.b": TensorSpec((self.q_width,), VECTOR, Normal(0.1)),
                 "q.norm": TensorSpec((self.dim,), VECTOR, Normal(0.1, mean=1.0)),
                 "g": TensorSpec((self.g_width, self.width), TABLE, Normal(std)),
                 "o": TensorSpec((self.width, self.g_width), TABLE, Normal(self.g_width ** -0.5))}
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = TensorSpec((self.dim,), VECTOR, Normal(0.1))
        if self.own_keys:
            specs["k"] = TensorSpec((self.k_width, self.width), TABLE, Normal(std))
            specs["k.b"] = TensorSpec((self.k_width,), VECTOR, Normal(0.1))
            specs["k.norm"] = TensorSpec((self.dim,), VECTOR, Normal(0.1, mean=1.0))
            specs["v"] = TensorSpec((self.v_width, self.width), TABLE, Normal(std))
            specs["v.b"] = TensorSpec((self.v_width,), VECTOR, Normal(0.1))
        return specs

    def bind(self, tensors):
        names = ("q", "k", "v", "g") if self.own_keys else ("q", "g")
        fused = fuse_rows([tensors[name] for name in names])
        self.w_in = kernels.pack_matrix(fused) if fused.is_cuda else fused
        self.b_in = torch.zeros((fused.shape[0],), dtype=torch.float32, device=fused.device)
        at = 0
        for name in names:
            rows = tensors[name].shape[0]
            if name + ".b" in tensors:
                self.b_in[at : at + rows] = tensors[name + ".b"]
            at += rows
        o = tensors["o"]
        self.o = kernels.pack_matrix(o.contiguous()) if o.is_cuda else o
        self.q_norm, self.k_norm = tensors["q.norm"], tensors.get("k.norm")
        dot = lambda a, b: float((tensors[a].double() * tensors[b].double()).sum())
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff

    def kv_need(self):
        # a chunk's pages stay: a layer that borrows them may look further back than the layer that keeps them
        return KVNeed(self.n_kv_heads * MAPS, self.head_size, None)

    def forward(self, x, residual, ctx: LayerContext):
        """The branch alone (float32) when ``residual`` is None, else residual + branch."""
        batch = ctx.batch
        if ctx.write_cache != self.own_keys:
            raise ValueError("a layer with keys and values of its own writes its cache layer, and only such a layer does")
        fused = kernels.linear(x, self.w_in, self.b_in, out_dtype=torch.float32)
        k_at = self.q_width if self.own_keys else None
        v_at = self.q_width + self.k_width if self.own_keys else None
        g_at = self.q_width + (self.k_width + self.v_width if self.own_keys else 0)
        rotary = self.rotary
        q = kernels.map_rows(fused, 0, k_at, v_at, self.q_norm, self.k_norm, self.eps, None if rotary is None else rotary.frequencies64(x.device),
                             0 if rotary is None else rotary.dims, batch.positions, ctx.group.slots, ctx.k_pages, ctx.v_pages, self.n_heads,
                             self.n_kv_heads, MAPS, self.dim, self.vdim)
        maps_out = kernels.paged_attention(
            q, ctx.k_pages, ctx.v_pages, batch.token_request, batch.positions, ctx.group.block_tables,
            self.n_heads * MAPS, self.n_kv_heads * MAPS, self.head_size, self.scale, chunk=self.chunk or 0,
            max_q_len=batch.max_q_len, max_len=batch.max_total_len, q_starts=batch.q_starts, context_lens=batch.context_lens,
            first_row=getattr(batch, "first_row", 0), wide_out=True,
            **({"short_rows": batch.short_rows, "short_requests": batch.short_requests} if batch.short_portion <= kernels.DECODE_MAX_Q_LEN else {}),
        )
        mixed = kernels.map_difference(maps_out, fused[:, g_at : g_at + self.g_width], self.lam, self.eps, self.n_heads, self.n_kv_heads, self.vdim,
                                       self.head_size, scale=1.0 - self.diff, out_dtype=x.dtype)
        return self._out_product(mixed, self.o, residual)


register_part("mixer", "differential_attention", DifferentialAttention)
