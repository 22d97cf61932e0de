"""The Dizizen architecture as a recipe of parts: a scaled token embedding; layers with ONE norm whose output both branches read, h =
norm1(x), x <- x + m (ls1 * sigmoid(rg1 h + b) * mixer(h) + ls2 * sigmoid(rg2 h + b) * ff(h)); attention with biases, rotated
queries and keys, values turned by their position and turned back behind the sum, which a later layer may borrow with its keys; per
layer a dense feed-forward with a clamped gate unit, routed experts, or none; a final RMS norm and a head of its own.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.ls{1,2}``, ``l<i>.rg{1,2}`` (+ ``.b``), ``l<i>.mix.{q,k,v,o}`` (+ ``.b``), ``l<i>.mlp.{gate,up,down}``
(+ ``.b``) or ``l<i>.mlp.{router,correction,e<j>.up,e<j>.down,shared.up,shared.down}``, ``final.norm``, ``head``."""

from __future__ import annotations

from ..config.dizizen import DenseMlpConfig, DizizenConfig, RoutedMlpConfig
from ..config.registry import register_architecture
from ..parts import LinearHead, TokenEmbedding, make_part
from .base import LayerCall, Model

QUICK_SIGMOID = 1.702   # the dense feed-forward's gate unit is g * sigmoid(1.702 g) * (u + 1)
UP_SHIFT = 1.0
WEIGHT_FLOOR = 1e-20    # joins the sum that the picked experts' scores are divided by


def _mixer(config: DizizenConfig, mixer):
    rotary = None if mixer.rot.dims == 0 else make_part("position_encoding", "rotary", dims=mixer.rot.dims, base=mixer.rot.base, pairing="half")
    # the values turn over all their elements, in the pairing of the keys, at the keys' base
    value_rotary = make_part("position_encoding", "rotary", dims=mixer.vdim, base=mixer.rot.base, pairing="half")
    return make_part("mixer", "rotary_attention", width=config.width, n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim,
                     scale=mixer.scale, rotary=rotary, value_rotary=value_rotary, biases=True, own_keys=mixer.kv_from is None)


def _feed_forward(config: DizizenConfig, mlp):
    if mlp is None:
        return None
    if isinstance(mlp, DenseMlpConfig):
        return make_part("feed_forward", "clamped_gated_mlp", width=config.width, inner=mlp.ff, limit=mlp.limit, alpha=QUICK_SIGMOID, shift=UP_SHIFT,
                         biases=True)
    if isinstance(mlp, RoutedMlpConfig):
        return make_part("feed_forward", "routed_experts", width=config.width, n_experts=mlp.experts, ff=mlp.expert_ff, top=mlp.top,
                         n_identity=mlp.identity, n_groups=mlp.groups, keep=mlp.keep, correction=True, shared_ff=mlp.shared_ff, floor=WEIGHT_FLOOR)
    raise TypeError(f"no feed-forward for {type(mlp).__name__}")


def build_dizizen(config: DizizenConfig, precision) -> Model:
    width, eps = config.width, config.norm_eps
    norm = lambda: make_part("norm", "rmsnorm", width=width, eps=eps, one_plus=True, tensor_name="")
    blocks, schedule = [], []
    for index, layer in enumerate(config.layers):
        blocks.append(make_part("block", "parallel", norm_1=norm(), mixer=_mixer(config, layer.mixer), feed_forward=_feed_forward(config, layer.mlp),
                                width=width, compute_dtype=precision.compute, mult=config.residual_mult, layer_scale=True, gated=True))
        borrowed = layer.mixer.kv_from
        schedule.append(LayerCall(block=index, cache=index if borrowed is None else borrowed, write_cache=borrowed is None))
    for block, following in zip(blocks, blocks[1:]):   # the schedule runs the layers in their order: a layer's sum is normed for the next
        block.hand_to(following.norm_1)
    return Model(
        config, precision,
        embedding=TokenEmbedding(config.vocab, width, scale=config.embedding_scale, tensor_name="", std=1.0 / max(config.embedding_scale, 1e-6)),
        position_encoding=None,
        blocks=blocks, schedule=schedule,
        final_norm=norm(),
        head=LinearHead(config.vocab, width, tensor_name=""),
        names={"embedding": "embed", "block": "l{i}.", "final_norm": "final.norm", "head": "head"},
    )


register_architecture("Dizizen", DizizenConfig, build_dizizen)
