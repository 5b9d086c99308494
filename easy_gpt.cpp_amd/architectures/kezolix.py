"""Kezolix decoder: typed configuration -> ModelSpec.

Tensor names: `embed`, `pos`, `l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`, `l<i>.norm2b`, `l<i>.dwa`, `l<i>.mix.*`
(attention: `q`, `k`, `v`, `q.norm`, `k.norm`, `o`, without `k`, `v`, `k.norm` where the layer reads another's keys and
values; recurrence: `q`, `f`, `f.b`, `lower`, `v`, `norm`, `o`), `l<i>.mlp.*` (dense: `up`, `down`, `act`; experts:
`e<j>.{up,down}`, `router`, `correction`, `shared.{up,down,sg}`), `final.norm`, `head`.  A layer is the sandwich
arrangement (a layer norm without bias before and behind each branch, a constant factor on what a branch adds) with a
depth average behind it; its mixer is block-local attention or a recurrence with a bounded forget gate; its
feed-forward is dense with a normed polynomial, or a mixture of squared-relu experts with a gated shared expert.
"""
from __future__ import annotations

from ..config.kezolix import KezolixConfig, KezolixLayer
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

SLOPE_SPAN = 8.0        # head h of H penalises a key by 2^(-8 (h + 1) / H) per token of distance


def _norm(prefix: str, name: str, eps: float) -> PartSpec:
    return PartSpec("layernorm", dict(eps=eps, name=name, bias_name=None), prefix=prefix)


def _layer_spec(layer: KezolixLayer, index: int, total: int, cfg: KezolixConfig) -> LayerSpec:
    p, eps, m = f"l{index}.", cfg.eps, layer.mixer
    if layer.type == "attention":
        mixer = PartSpec("block_local_attention",
                         dict(n_heads=m.heads, n_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim, scale=m.scale, eps=eps,
                              block=m.block, slope_span=SLOPE_SPAN, shares_cache=m.kv_from is not None),
                         prefix=p + "mix.")
    else:
        mixer = PartSpec("bounded_gate_recurrence", dict(n_heads=m.heads, key_dim=m.dim, value_dim=m.vdim, eps=eps),
                         prefix=p + "mix.")
    norms = {"mixer": _norm(p, "norm1", eps), "mixer_out": _norm(p, "norm1b", eps)}
    join = PartSpec("depth_average", dict(index=index + 1, total=total, name="dwa"), prefix=p)
    params = dict(residual_mult=cfg.residual_mult)
    f = layer.mlp
    if f is None:
        return LayerSpec(block="sandwich_mixer_only", mixer=mixer, feed_forward=None, norms=norms, block_params=params,
                         stream_join=join)
    if f.kind == "dense":
        ff = PartSpec("activated", dict(intermediate_size=f.ff, activation="polynorm", eps=eps, names=("up", "down"), coef="act"),
                      prefix=p + "mlp.")
    else:
        shared = None
        if f.shared_ff is not None:
            shared = PartSpec("activated", dict(intermediate_size=f.shared_ff, activation="relu2", names=("up", "down"),
                                                row_gate="sg"), prefix=p + "mlp.shared.")
        ff = PartSpec("expert_mixture",
                      dict(n_experts=f.experts, top=f.top, intermediate_size=f.ff, shared=shared, router_bias=False,
                           routing="softmax_all", weight_scale=f.scale, expert="relu2"),
                      prefix=p + "mlp.")
    norms["feed_forward"], norms["feed_forward_out"] = _norm(p, "norm2", eps), _norm(p, "norm2b", eps)
    return LayerSpec(block="sandwich", mixer=mixer, feed_forward=ff, norms=norms, block_params=params, stream_join=join)


def kezolix_spec(cfg: KezolixConfig) -> ModelSpec:
    n = len(cfg.layers)
    layers = tuple(_layer_spec(layer, i, n + 1, cfg) for i, layer in enumerate(cfg.layers))
    runs = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "attention":
            src = layer.mixer.kv_from
            runs.append(RunSpec(layer=i, cache=i if src is None else src, writes_cache=src is None))
        else:
            runs.append(RunSpec(layer=i, state=i))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=cfg.max_positions,
        embedding=PartSpec("token_embedding_positions", dict(max_positions=cfg.max_positions, name="embed", position_name="pos"),
                           prefix=""),
        layers=layers,
        run_order=tuple(runs),
        final_norm=_norm("", "final.norm", cfg.eps),
        output_head=PartSpec("linear_head", dict(tied=False, name="head"), prefix=""),
    )


KEZOLIX = register_architecture(
    Architecture(name="Kezolix", config_class=KezolixConfig, build_spec=kezolix_spec, model_types=("kezolix",)),
    replace=True,
)
