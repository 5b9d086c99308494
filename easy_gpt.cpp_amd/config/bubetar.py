"""Typed configuration of the Bubetar decoder, read from its config.json keys.

A Bubetar config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, `logit_scale` (absent
or null: 1), `logit_softcap` (absent or null: no cap) and `layers`: a list with one entry per layer, each with `type`,
`mixer` and `mlp` (null for no feed-forward, or kind 'dense' with ff).  The mixers by type:

  latent_attention   heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot.{base, dims}
  parallel           left.{heads, kv_heads, dim, vdim, scale, rot.{base, dims}}, right.{heads, dim, vdim, decay[heads]},
                     left_scale, right_scale
  parallel_2         left.{heads, kv_heads, dim, vdim, scale, mask.size or no mask, rot.{base, dims, scaling.{factor,
                     low, high, original} or none}}, right.{heads, kv_heads, dim, vdim, conv}, left_scale, right_scale
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
class Rotation:
    base: float
    dims: int
    scaling: tuple[float, float, float, float] | None = None      # factor, low, high, original

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str, limit: int) -> "Rotation":
        r = KeyReader(data, where)
        dims = r.integer("dims", minimum=0)
        if dims % 2 or dims > limit:
            raise ConfigError(f"{where}: 'dims' ({dims}) must be even and at most {limit}")
        sc = _object(data, "scaling", where, required=False)
        scaling = None
        if sc is not None:
            s = KeyReader(sc, where + ".scaling")
            scaling = (s.number("factor", positive=True), s.number("low", positive=True), s.number("high", positive=True),
                       s.number("original", positive=True))
            if not scaling[2] > scaling[1]:
                raise ConfigError(f"{where}.scaling: 'high' ({scaling[2]}) must be larger than 'low' ({scaling[1]})")
        return cls(r.number("base", positive=True), dims, scaling)


def _heads(r: KeyReader, where: str, grouped: bool) -> tuple[int, int]:
    heads = r.integer("heads", minimum=1)
    kv_heads = r.integer("kv_heads", heads, minimum=1) if grouped else heads       # (absent: a key/value head per head)
    if heads % kv_heads:
        raise ConfigError(f"{where}: 'heads' ({heads}) must be a multiple of 'kv_heads' ({kv_heads})")
    return heads, kv_heads


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: Rotation

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "LatentAttentionConfig":
        r = KeyReader(data, where)
        rot_dim = r.integer("rot_dim", minimum=0)
        rot = Rotation.from_dict(_object(data, "rot", where), where + ".rot", rot_dim)
        return cls(r.integer("heads", minimum=1), r.integer("dim", minimum=1), rot_dim, r.integer("vdim", minimum=1),
                   r.integer("q_rank", minimum=1), r.integer("kv_rank", minimum=1), r.number("scale"), rot)


@dataclass(frozen=True)
class SoftmaxSideConfig:
    """The softmax attention of a pair: `window` None means every earlier key."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Rotation
    window: int | None = None

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "SoftmaxSideConfig":
        r = KeyReader(data, where)
        heads, kv_heads = _heads(r, where, grouped=True)
        dim = r.integer("dim", minimum=1)
        rot = Rotation.from_dict(_object(data, "rot", where), where + ".rot", dim)
        mask = _object(data, "mask", where, required=False)
        window = None if mask is None else KeyReader(mask, where + ".mask").integer("size", minimum=1)
        return cls(heads, kv_heads, dim, r.integer("vdim", minimum=1), r.number("scale"), rot, window)


@dataclass(frozen=True)
class ConstantDecayConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "ConstantDecayConfig":
        r = KeyReader(data, where)
        heads = r.integer("heads", minimum=1)
        raw = data.get("decay")
        if not isinstance(raw, list) or len(raw) != heads or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in raw):
            raise ConfigError(f"{where}: 'decay' must be a list of {heads} numbers, one per head")
        return cls(heads, r.integer("dim", minimum=1), r.integer("vdim", minimum=1), tuple(float(v) for v in raw))


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "DeltaRuleConfig":
        r = KeyReader(data, where)
        heads, kv_heads = _heads(r, where, grouped=True)
        return cls(heads, kv_heads, r.integer("dim", minimum=1), r.integer("vdim", minimum=1), r.integer("conv", minimum=1))


@dataclass(frozen=True)
class PairConfig:
    left: SoftmaxSideConfig
    right: ConstantDecayConfig | DeltaRuleConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class BubetarLayer:
    type: str                    # 'latent_attention', 'parallel' or 'parallel_2'
    mixer: LatentAttentionConfig | PairConfig
    ff: int | None               # the inner width of the feed-forward; None: the layer has none


LAYER_TYPES = ("latent_attention", "parallel", "parallel_2")


@dataclass(frozen=True)
class BubetarConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    logit_scale: float
    logit_softcap: float | None
    layers: tuple[BubetarLayer, ...]

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str = "config.json") -> "BubetarConfig":
        r = KeyReader(data, where)
        architecture = r.string("architecture")
        eps = KeyReader(_object(data, "norm", where), where + ".norm").number("eps", positive=True)
        raw = data.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError(f"{where}: required key 'layers' (a list of layers) is missing or empty")
        layers: list[BubetarLayer] = []
        for i, entry in enumerate(raw):
            at = f"{where}.layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at}: must be an object")
            kind = KeyReader(entry, at).string("type", check=lambda v: v in LAYER_TYPES)
            mixer = _object(entry, "mixer", at)
            if kind == "latent_attention":
                m = LatentAttentionConfig.from_dict(mixer, at + ".mixer")
            else:
                left = SoftmaxSideConfig.from_dict(_object(mixer, "left", at + ".mixer"), at + ".mixer.left")
                side = _object(mixer, "right", at + ".mixer")
                right = (ConstantDecayConfig if kind == "parallel" else DeltaRuleConfig).from_dict(side, at + ".mixer.right")
                mr = KeyReader(mixer, at + ".mixer")
                m = PairConfig(left, right, mr.number("left_scale"), mr.number("right_scale"))
                if kind == "parallel_2" and left.vdim != left.dim:
                    raise ConfigError(f"{at}.mixer.left: the values are the keys, so 'vdim' ({left.vdim}) must equal 'dim' ({left.dim})")
            mlp = _object(entry, "mlp", at, required=False)
            ff = None
            if mlp is not None:
                mk = KeyReader(mlp, at + ".mlp")
                mk.string("kind", check=lambda v: v == "dense")
                ff = mk.integer("ff", minimum=1)
            layers.append(BubetarLayer(kind, m, ff))
        cap = r.number("logit_softcap", None, positive=True)
        return cls(architecture, r.integer("vocab", minimum=1), r.integer("width", minimum=1), eps,
                   r.number("logit_scale", 1.0), cap, tuple(layers))
