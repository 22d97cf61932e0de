"""The Perezen architecture as a recipe of parts: a token embedding with learned positions added, layers with a norm in front of each
branch and one on its output (x <- x + norm1b(mixer(norm1(x))), x <- x + norm2b(ff(norm2(x)))), per layer the mixer its configuration
names (a matrix memory, or differential attention inside chunks of the sequence, which may read the keys and values an earlier layer
keeps), gated feed-forwards, a final RMS norm and a head of its own whose logits are multiplied by a constant.

Tensor names: ``embed``, ``pos``, ``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.<name>``,
``l<i>.mlp.{gate,up,down}``, ``final.norm``, ``head``."""

from __future__ import annotations

from ..config.perezen import DifferentialMixerConfig, MlstmMixerConfig, PerezenConfig
from ..config.registry import register_architecture
from ..parts import LinearHead, TokenEmbedding, make_part
from .base import LayerCall, Model


def _mixer(config: PerezenConfig, mixer):
    width, eps = config.width, config.norm_eps
    if isinstance(mixer, MlstmMixerConfig):
        return make_part("mixer", "matrix_memory", width=width, n_heads=mixer.heads, dim=mixer.dim, vdim=mixer.vdim, eps=eps, gate_cap=mixer.gate_cap)
    if isinstance(mixer, DifferentialMixerConfig):
        rot = mixer.rot
        rotary = None if rot is None or rot.dims == 0 else make_part("position_encoding", "rotary", dims=rot.dims, base=rot.base, pairing="half")
        return make_part("mixer", "differential_attention", width=width, n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, dim=mixer.dim,
                         vdim=mixer.vdim, scale=mixer.scale, diff=mixer.diff, eps=eps, rotary=rotary, chunk=mixer.chunk,
                         own_keys=mixer.kv_from is None)
    raise TypeError(f"no mixer for {type(mixer).__name__}")


def build_perezen(config: PerezenConfig, precision) -> Model:
    width, eps = config.width, config.norm_eps
    norm = lambda: make_part("norm", "rmsnorm", width=width, eps=eps, tensor_name="")
    blocks, schedule = [], []
    for index, layer in enumerate(config.layers):
        has_mlp = layer.ff is not None
        blocks.append(make_part(
            "block", "sandwich_norm", norm_1=norm(), mixer=_mixer(config, layer.mixer), norm_1b=norm(), norm_2=norm() if has_mlp else None,
            feed_forward=make_part("feed_forward", "gated_mlp", width=width, inner=layer.ff) if has_mlp else None,
            norm_2b=norm() if has_mlp else None, compute_dtype=precision.compute,
        ))
        borrowed = getattr(layer.mixer, "kv_from", None)
        schedule.append(LayerCall(block=index, cache=index if borrowed is None else borrowed, write_cache=borrowed is None))
    for block, following in zip(blocks, blocks[1:]):   # the schedule runs the layers in their order: a layer's last kernel norms for the next
        block.hand_to(following.norm_1)
    return Model(
        config, precision,
        embedding=TokenEmbedding(config.vocab, width, tensor_name="", std=1.0),
        position_encoding=make_part("position_encoding", "learned", n_positions=config.max_positions, width=width, tensor_name="", std=0.3),
        blocks=blocks, schedule=schedule,
        # logits = logit_scale * head . norm(x): the head's product is linear, so the constant rides in the final norm's 32-bit gain
        final_norm=make_part("norm", "rmsnorm", width=width, eps=eps, tensor_name="", out_scale=config.logit_scale),
        head=LinearHead(config.vocab, width, tensor_name=""),
        names={"embedding": "embed", "position_encoding": "pos", "block": "l{i}.", "final_norm": "final.norm", "head": "head"},
    )


register_architecture("Perezen", PerezenConfig, build_perezen)
