"""Bubetar decoder: typed configuration -> ModelSpec.

Tensor names: `embed`, `l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`, `l<i>.norm2b`, `l<i>.mix.*`, `l<i>.mlp.{gate,up,down}`,
`final.norm`, `head`.  The mixers' tensors: latent attention `dq`, `dq.norm`, `uq`, `dkv`, `dkv.norm`, `uk`, `uv`, `o`; a
pair has `left.*` and `right.*`: the gated attention `q`, `k`, `v`, `q.norm`, `k.norm`, `g`, `o` beside the constant-decay
linear attention `q`, `k`, `v`, `g`, `norm`, `o`; or the window attention on its own keys `q`, `k`, `sink`, `o` beside the
gated delta rule `q`, `k`, `v` (each with `.conv`), `b`, `A_log`, `a1`, `a2`, `dt_bias`, `g1`, `g2`, `norm`, `o`.

A layer is the sandwich arrangement (a layer norm without bias before and behind each branch) with a factor of one and
no join over the depth; the feed-forward is the gated one with silu.
"""
from __future__ import annotations

from ..config.bubetar import BubetarConfig, BubetarLayer, Rotation
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

MAX_POSITION = 2**31 - 2        # the design names no longest sequence: positions are 32-bit integers
UNIT_EPS = 1e-6                 # under the root when queries and keys of the delta rule are made unit vectors


def _norm(prefix: str, name: str, eps: float) -> PartSpec:
    return PartSpec("layernorm", dict(eps=eps, name=name, bias_name=None), prefix=prefix)


def _rotation(rot: Rotation, kind: str) -> PartSpec:
    if rot.dims == 0:
        return PartSpec("none", {})
    scaling = None
    if rot.scaling is not None:
        factor, low, high, original = rot.scaling
        scaling = dict(rule="wavelength", factor=factor, low=low, high=high, original=original)
    return PartSpec(kind, dict(theta=rot.base, rotary_dim=rot.dims, scaling=scaling, exact_frequencies=True))


def _mixer_spec(layer: BubetarLayer, p: str, eps: float) -> PartSpec:
    m = layer.mixer
    if layer.type == "latent_attention":
        return PartSpec(
            "latent_attention",
            dict(n_heads=m.heads, plain_dim=m.dim, rotated_dim=m.rot_dim, value_dim=m.vdim, latent_dim=m.kv_rank,
                 query_latent_dim=m.q_rank, scale=m.scale, eps=eps, position=_rotation(m.rot, "rope_interleaved"),
                 names=dict(q="uq", q_down="dq", q_down_norm="dq.norm", down="dkv", down_norm="dkv.norm", up_k="uk", up_v="uv",
                            o="o")),
            prefix=p)
    left, right = m.left, m.right
    names = dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm", gate="g", sink="sink")
    if layer.type == "parallel":
        lspec = PartSpec(
            "normed_attention",
            dict(n_heads=left.heads, n_kv_heads=left.kv_heads, key_dim=left.dim, value_dim=left.vdim, scale=left.scale, eps=eps,
                 window=left.window, position=_rotation(left.rot, "rope_interleaved"), gated=True, names=names),
            prefix=p + "left.")
        rspec = PartSpec(
            "constant_decay_attention",
            dict(n_heads=right.heads, key_dim=right.dim, value_dim=right.vdim, decay=right.decay, eps=eps),
            prefix=p + "right.")
    else:
        lspec = PartSpec(
            "normed_attention",
            dict(n_heads=left.heads, n_kv_heads=left.kv_heads, key_dim=left.dim, value_dim=left.vdim, scale=left.scale, eps=eps,
                 window=left.window, position=_rotation(left.rot, "rope_half_split"), norm_weighted=False,
                 norm_after_rotation=True, values_are_keys=True, sink=True, names=names),
            prefix=p + "left.")
        rspec = PartSpec(
            "gated_delta_rule",
            dict(n_heads=right.heads, n_kv_heads=right.kv_heads, key_dim=right.dim, value_dim=right.vdim, taps=right.conv,
                 eps=eps, unit_eps=UNIT_EPS),
            prefix=p + "right.")
    # (the sum of the two sides is left to the norm behind the mixer, which every layer of this design has)
    return PartSpec("side_by_side", dict(left=lspec, right=rspec, eps=eps, join="weighted_sum",
                                         factors=(m.left_scale, m.right_scale), deferred=True), prefix=p)


def _layer_spec(layer: BubetarLayer, index: int, eps: float) -> LayerSpec:
    p = f"l{index}."
    mixer = _mixer_spec(layer, p + "mix.", eps)
    norms = {"mixer": _norm(p, "norm1", eps), "mixer_out": _norm(p, "norm1b", eps)}
    params = dict(residual_mult=1.0)
    if layer.ff is None:
        return LayerSpec(block="sandwich_mixer_only", mixer=mixer, feed_forward=None, norms=norms, block_params=params)
    ff = PartSpec("swiglu", dict(intermediate_size=layer.ff, names=("gate", "up", "down"), unrounded=True), prefix=p + "mlp.")
    norms["feed_forward"], norms["feed_forward_out"] = _norm(p, "norm2", eps), _norm(p, "norm2b", eps)
    return LayerSpec(block="sandwich", mixer=mixer, feed_forward=ff, norms=norms, block_params=params)


def bubetar_spec(cfg: BubetarConfig) -> ModelSpec:
    layers = tuple(_layer_spec(layer, i, cfg.eps) for i, layer in enumerate(cfg.layers))
    runs = tuple(RunSpec(layer=i, cache=i, state=None if layer.type == "latent_attention" else i)
                 for i, layer in enumerate(cfg.layers))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=MAX_POSITION,
        embedding=PartSpec("token_embedding_scaled", dict(scale=1.0, name="embed"), prefix=""),
        layers=layers,
        run_order=runs,
        final_norm=_norm("", "final.norm", cfg.eps),
        output_head=PartSpec("linear_head", dict(tied=False, name="head", softcap=cfg.logit_softcap, scale=cfg.logit_scale),
                             prefix=""),
    )


BUBETAR = register_architecture(
    Architecture(name="Bubetar", config_class=BubetarConfig, build_spec=bubetar_spec, model_types=("bubetar",)),
    replace=True,
)
