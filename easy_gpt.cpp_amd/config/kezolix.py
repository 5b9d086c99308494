"""Typed configuration of the Kezolix decoder, read from its config.json keys.

A Kezolix config.json names the design in `architecture` and gives `vocab`, `width`, `max_positions` (the rows of the
learned position table), `norm.eps`, `residual_mult` (the factor on what a layer's branches add to the stream) and
`layers`: a list with one entry per layer, each with `type` ('attention' or 'hgrn2'), `mixer` (attention: heads,
kv_heads, dim, vdim, scale, mask.size or no mask, and kv_from: the layer whose keys and values it reads instead of
making its own; hgrn2: heads, dim, vdim) and `mlp` (null for no feed-forward; kind 'dense' with ff; or kind 'moe' with
router.{experts, top, scale}, expert.ff and shared.ff or no shared expert).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .base import ConfigError, KeyReader


def _object(data: Mapping[str, Any], key: str, where: str, required: bool = True):
    v = data.get(key)
    if v is None:
        if required:
            raise ConfigError(f"{where}: required key '{key}' (an object) is missing")
        return None
    if not isinstance(v, Mapping):
        raise ConfigError(f"{where}: '{key}' must be an object{'' if required else ' or null'}")
    return v


@dataclass(frozen=True)
class LocalAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    block: int | None            # mask.size; None: every earlier key is visible
    kv_from: int | None          # the layer whose keys and values this one reads; None: its own

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "LocalAttentionConfig":
        r = KeyReader(data, where)
        heads, kv_heads = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
        if heads % kv_heads:
            raise ConfigError(f"{where}: 'heads' ({heads}) must be a multiple of 'kv_heads' ({kv_heads})")
        mask = _object(data, "mask", where, required=False)
        block = None if mask is None else KeyReader(mask, where + ".mask").integer("size", minimum=1)
        return cls(heads, kv_heads, r.integer("dim", minimum=1), r.integer("vdim", minimum=1), r.number("scale"), block,
                   r.integer("kv_from", None, minimum=0))


@dataclass(frozen=True)
class RecurrenceConfig:
    heads: int
    dim: int
    vdim: int

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "RecurrenceConfig":
        r = KeyReader(data, where)
        return cls(r.integer("heads", minimum=1), r.integer("dim", minimum=1), r.integer("vdim", minimum=1))


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                    # 'dense' or 'moe'
    ff: int                      # inner width (of one expert for 'moe')
    experts: int = 0
    top: int = 0
    scale: float = 1.0
    shared_ff: int | None = None

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "FeedForwardConfig":
        kind = KeyReader(data, where).string("kind", check=lambda v: v in ("dense", "moe"))
        if kind == "dense":
            return cls(kind, KeyReader(data, where).integer("ff", minimum=1))
        router = KeyReader(_object(data, "router", where), where + ".router")
        experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
        if top > experts:
            raise ConfigError(f"{where}.router: 'top' ({top}) is larger than 'experts' ({experts})")
        ff = KeyReader(_object(data, "expert", where), where + ".expert").integer("ff", minimum=1)
        shared = _object(data, "shared", where, required=False)
        shared_ff = None if shared is None else KeyReader(shared, where + ".shared").integer("ff", minimum=1)
        return cls(kind, ff, experts, top, router.number("scale", 1.0), shared_ff)


@dataclass(frozen=True)
class KezolixLayer:
    type: str                    # 'attention' or 'hgrn2'
    mixer: LocalAttentionConfig | RecurrenceConfig
    mlp: FeedForwardConfig | None


@dataclass(frozen=True)
class KezolixConfig:
    architecture: str
    vocab: int
    width: int
    max_positions: int
    eps: float
    residual_mult: float
    layers: tuple[KezolixLayer, ...]

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str = "config.json") -> "KezolixConfig":
        r = KeyReader(data, where)
        architecture = r.string("architecture")
        eps = KeyReader(_object(data, "norm", where), where + ".norm").number("eps", positive=True)
        raw = data.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError(f"{where}: required key 'layers' (a list of layers) is missing or empty")
        layers: list[KezolixLayer] = []
        for i, entry in enumerate(raw):
            at = f"{where}.layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at}: must be an object")
            kind = KeyReader(entry, at).string("type", check=lambda v: v in ("attention", "hgrn2"))
            mixer = _object(entry, "mixer", at)
            if kind == "attention":
                m = LocalAttentionConfig.from_dict(mixer, at + ".mixer")
                if m.kv_from is not None:
                    src = layers[m.kv_from].mixer if m.kv_from < i else None
                    if not isinstance(src, LocalAttentionConfig) or src.kv_from is not None:
                        raise ConfigError(f"{at}.mixer: 'kv_from' ({m.kv_from}) must name an earlier attention layer with keys and values of its own")
                    if (src.kv_heads, src.dim, src.vdim) != (m.kv_heads, m.dim, m.vdim):
                        raise ConfigError(f"{at}.mixer: kv_heads, dim and vdim must equal those of layer {m.kv_from}, whose keys and values it reads")
            else:
                m = RecurrenceConfig.from_dict(mixer, at + ".mixer")
            mlp = _object(entry, "mlp", at, required=False)
            layers.append(KezolixLayer(kind, m, None if mlp is None else FeedForwardConfig.from_dict(mlp, at + ".mlp")))
        return cls(architecture, r.integer("vocab", minimum=1), r.integer("width", minimum=1),
                   r.integer("max_positions", minimum=1), eps, r.number("residual_mult"), tuple(layers))
