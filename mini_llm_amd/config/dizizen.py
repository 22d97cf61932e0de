"""Typed configuration of the Dizizen architecture: a list of layers that norm their input once and run mixer and feed-forward side by
side on it, each layer with its own sizes; attention with rotated queries, keys and values; dense feed-forwards with a clamped gate
unit, or routed experts.

config.json keys: ``architecture`` ("Dizizen"), ``vocab``, ``width``, ``embedding.scale``, ``norm.eps``, ``residual_mult`` and ``layers``, a
list of {``type``, ``mixer``, ``mlp``}. ``type`` is "attention": mixer = {heads, kv_heads, dim, vdim, scale, rot: {dims, base}, kv_from: index
of an earlier attention layer with keys and values of its own | absent}. ``mlp`` is null, {kind: "dense", ff, limit} or {kind: "moe",
expert: {ff}, router: {experts, top, identity | absent, groups: {count, keep} | absent}, shared: {ff} | absent}."""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ModelConfig, take_float, take_int
from .ketolix import MAX_HEAD_SIZE, _grouped_heads, _section
from .perezen import HalfRotaryConfig

MAX_ROUTER_OUTPUTS = 1024   # what the router kernel takes


@dataclass(frozen=True)
class RotatedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: HalfRotaryConfig
    kv_from: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "RotatedAttentionConfig":
        heads, kv_heads = _grouped_heads(raw, where)
        dim, vdim = take_int(raw, "dim"), take_int(raw, "vdim")
        if max(dim, vdim) > MAX_HEAD_SIZE:
            raise ConfigError(f"{where}heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        if vdim % 2:
            raise ConfigError(f"{where}values of {vdim} elements do not turn in pairs")
        kv_from = raw.get("kv_from")
        if kv_from is not None:
            kv_from = take_int(raw, "kv_from", minimum=0)
        return cls(heads, kv_heads, dim, vdim, take_float(raw, "scale"), HalfRotaryConfig.from_dict(_section(raw, "rot", where), where, dim), kv_from)

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "rot": self.rot.to_dict(), "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DenseMlpConfig":
        limit = take_float(raw, "limit")
        if not limit > 0:
            raise ConfigError(f"{where}mlp.limit must be positive, not {limit}")
        return cls(take_int(raw, "ff"), limit)

    def to_dict(self) -> dict:
        return {"ff": self.ff, "kind": "dense", "limit": self.limit}


@dataclass(frozen=True)
class RoutedMlpConfig:
    experts: int            # experts with matrices of their own
    identity: int           # router outputs behind them that hand the input on
    top: int
    groups: int
    keep: int
    expert_ff: int
    shared_ff: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "RoutedMlpConfig":
        router = _section(raw, "router", where)
        experts, identity = take_int(router, "experts"), take_int(router, "identity", 0, minimum=0)
        total = experts + identity
        if total > MAX_ROUTER_OUTPUTS:
            raise ConfigError(f"{where}{total} router outputs are more than the router kernel takes ({MAX_ROUTER_OUTPUTS})")
        groups_raw = _section(router, "groups", where, optional=True)
        groups, keep = (1, 1) if groups_raw is None else (take_int(groups_raw, "count"), take_int(groups_raw, "keep"))
        if total % groups or keep > groups:
            raise ConfigError(f"{where}{total} router outputs do not form {groups} equal groups of which {keep} are kept")
        top = take_int(router, "top")
        if top > keep * (total // groups):
            raise ConfigError(f"{where}{top} experts cannot be picked among {keep} groups of {total // groups}")
        shared = _section(raw, "shared", where, optional=True)
        return cls(experts, identity, top, groups, keep, take_int(_section(raw, "expert", where), "ff"), None if shared is None else take_int(shared, "ff"))

    def to_dict(self) -> dict:
        router = {"experts": self.experts, "groups": {"count": self.groups, "keep": self.keep}, "identity": self.identity, "top": self.top}
        out = {"expert": {"ff": self.expert_ff}, "kind": "moe", "router": router}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


MLPS = {"dense": DenseMlpConfig, "moe": RoutedMlpConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: RotatedAttentionConfig
    mlp: object   # DenseMlpConfig, RoutedMlpConfig or None: the layer has no feed-forward

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class DizizenConfig(ModelConfig):
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    residual_mult: float
    layers: tuple
    eos_token_id: int | None = None

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw: dict) -> "DizizenConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json has no list of 'layers'")
        layers = []
        for index, entry in enumerate(layers_raw):
            where = f"layer {index}: "
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}must be an object")
            kind = entry.get("type")
            if kind != "attention":
                raise ConfigError(f"{where}unknown type {kind!r}; known: attention")
            mixer = RotatedAttentionConfig.from_dict(_section(entry, "mixer", where), where)
            if mixer.kv_from is not None:
                source = layers[mixer.kv_from].mixer if mixer.kv_from < index else None
                if source is None or source.kv_from is not None:
                    raise ConfigError(f"{where}kv_from = {mixer.kv_from} does not name an earlier layer with keys and values of its own")
                if (source.kv_heads, source.dim, source.vdim, source.rot) != (mixer.kv_heads, mixer.dim, mixer.vdim, mixer.rot):
                    raise ConfigError(f"{where}the keys and values of layer {mixer.kv_from} have other heads, sizes or rotation")
            mlp_raw = _section(entry, "mlp", where, optional=True)
            mlp = None
            if mlp_raw is not None:
                mlp_kind = mlp_raw.get("kind", "dense")
                if mlp_kind not in MLPS:
                    raise ConfigError(f"{where}unknown mlp.kind {mlp_kind!r}; known: {', '.join(sorted(MLPS))}")
                mlp = MLPS[mlp_kind].from_dict(mlp_raw, where)
            layers.append(LayerConfig(kind, mixer, mlp))
        eps = take_float(_section(raw, "norm", ""), "eps")
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, not {eps}")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer or null, not {eos!r}")
        return cls(architecture=raw.get("architecture") or "Dizizen", vocab=take_int(raw, "vocab"), width=take_int(raw, "width"),
                   embedding_scale=take_float(_section(raw, "embedding", ""), "scale"), norm_eps=eps, residual_mult=take_float(raw, "residual_mult"),
                   layers=tuple(layers), eos_token_id=eos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale}, "layers": [layer.to_dict() for layer in self.layers],
               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out
