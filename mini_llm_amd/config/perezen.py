"""Typed configuration of the Perezen architecture: learned positions, a list of layers with a norm before and behind every branch,
each layer with its own kind of mixer and its own sizes.

config.json keys: ``architecture`` ("Perezen"), ``vocab``, ``width``, ``max_positions``, ``norm.eps``, ``logit_scale`` (absent: 1) and
``layers``, a list of {``type``, ``mixer``, ``mlp``}; ``mlp`` is {kind: "dense", ff} or null. By ``type``:

- "mlstm": mixer = {heads, dim, vdim, gate_cap | absent}.
- "attention" (differential: two maps a head): mixer = {heads, kv_heads, dim, vdim, scale, diff, mask: {size} | absent (chunks of so many
  positions), rot: {dims, base} | absent, kv_from: index of an earlier attention layer with keys and values of its own | absent}."""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ModelConfig, take_float, take_int
from .ketolix import MAX_HEAD_SIZE, MlstmMixerConfig, _grouped_heads, _section


@dataclass(frozen=True)
class HalfRotaryConfig:
    dims: int
    base: float

    @classmethod
    def from_dict(cls, raw: dict, where: str, dim: int) -> "HalfRotaryConfig":
        dims = take_int(raw, "dims", minimum=0)
        if dims % 2 or dims > dim:
            raise ConfigError(f"{where}rot.dims = {dims} must be even and at most the heads' {dim} elements")
        base = take_float(raw, "base")
        if not base > 0:
            raise ConfigError(f"{where}rot.base must be positive, not {base}")
        return cls(dims, base)

    def to_dict(self) -> dict:
        return {"base": self.base, "dims": self.dims}


@dataclass(frozen=True)
class DifferentialMixerConfig:
    heads: int
    kv_heads: int
    dim: int        # elements of a query or key of ONE map; a head has two maps
    vdim: int
    scale: float
    diff: float
    chunk: int | None            # mask.size: a query sees the keys of its own chunk of so many positions; None: all before it
    rot: HalfRotaryConfig | None
    kv_from: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DifferentialMixerConfig":
        heads, kv_heads = _grouped_heads(raw, where)
        dim, vdim = take_int(raw, "dim"), take_int(raw, "vdim")
        if max(dim, vdim) > MAX_HEAD_SIZE:
            raise ConfigError(f"{where}heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        mask = _section(raw, "mask", where, optional=True)
        rot = _section(raw, "rot", where, optional=True)
        kv_from = raw.get("kv_from")
        if kv_from is not None:
            kv_from = take_int(raw, "kv_from", minimum=0)
        return cls(heads, kv_heads, dim, vdim, take_float(raw, "scale"), take_float(raw, "diff"), None if mask is None else take_int(mask, "size"),
                   None if rot is None else HalfRotaryConfig.from_dict(rot, where, dim), kv_from)

    def to_dict(self) -> dict:
        out = {"diff": self.diff, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


MIXERS = {"mlstm": MlstmMixerConfig, "attention": DifferentialMixerConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: object
    ff: int | None   # the feed-forward's inner size; None: the layer has none

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"}, "type": self.type}


@dataclass(frozen=True)
class PerezenConfig(ModelConfig):
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    logit_scale: float
    layers: tuple
    eos_token_id: int | None = None

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw: dict) -> "PerezenConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json has no list of 'layers'")
        layers = []
        for index, entry in enumerate(layers_raw):
            where = f"layer {index}: "
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}must be an object")
            kind = entry.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}unknown type {kind!r}; known: {', '.join(sorted(MIXERS))}")
            mixer = MIXERS[kind].from_dict(_section(entry, "mixer", where), where)
            if kind == "attention" and mixer.kv_from is not None:
                source = layers[mixer.kv_from].mixer if mixer.kv_from < index else None
                if not isinstance(source, DifferentialMixerConfig) or source.kv_from is not None:
                    raise ConfigError(f"{where}kv_from = {mixer.kv_from} does not name an earlier attention layer with keys and values of its own")
                if (source.kv_heads, source.dim, source.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim):
                    raise ConfigError(f"{where}the keys and values of layer {mixer.kv_from} have other heads or sizes")
            mlp = _section(entry, "mlp", where, optional=True)
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}unknown mlp.kind {mlp.get('kind')!r}; known: dense")
                ff = take_int(mlp, "ff")
            layers.append(LayerConfig(kind, mixer, ff))
        eps = take_float(_section(raw, "norm", ""), "eps")
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, not {eps}")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer or null, not {eos!r}")
        return cls(architecture=raw.get("architecture") or "Perezen", vocab=take_int(raw, "vocab"), width=take_int(raw, "width"),
                   max_positions=take_int(raw, "max_positions"), norm_eps=eps, logit_scale=take_float(raw, "logit_scale", 1.0), layers=tuple(layers),
                   eos_token_id=eos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers], "logit_scale": self.logit_scale,
               "max_positions": self.max_positions, "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out
