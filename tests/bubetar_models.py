"""Small Bubetar configurations and weights for the tests: sizes that differ in every respect, weights drawn so that
activations are of order one, attention is peaked, sinks take a visible share of the softmax, the constant decays and
the delta rule's decays lie well inside (0, 1), the short convolutions weigh every tap, and beta lies between 0 and 1
(with weights of N(0, 0.02) a key that is wrongly seen, a lost state or a lost convolution input would hardly move the
logits).  The tensor names are written out here, not taken from the engine."""
from __future__ import annotations

import json
import os

import torch

from easy_gpt.cpp_amd.weights import write_safetensors


def rotation(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, dims=None):
    return "latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                                "scale": scale, "rot": rotation(base, rot_dim if dims is None else dims)}


def softmax_side(heads, kv_heads, dim, vdim, scale, rot, window=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if window:
        m["mask"] = {"size": window}
    return m


def pair(left, decay_side, left_scale, right_scale):
    return "parallel", {"left": left, "right": decay_side, "left_scale": left_scale, "right_scale": right_scale}


def pair_2(left, delta_side, left_scale, right_scale):
    return "parallel_2", {"left": left, "right": delta_side, "left_scale": left_scale, "right_scale": right_scale}


def constant_decay(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def delta_rule(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def layer(mixer, ff):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(vocab, width, eps, layers, logit_scale=None, logit_softcap=None):
    c = {"architecture": "Bubetar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if logit_scale is not None:
        c["logit_scale"] = logit_scale
    if logit_softcap is not None:
        c["logit_softcap"] = logit_softcap
    return c


# one layer of each kind and a second latent layer; rotation over part of a head; a window of 12; two value heads on
# each query/key head of the delta rule; a layer without a feed-forward
CONFIG_A = config(300, 64, 1e-6, [
    layer(pair(softmax_side(4, 2, 16, 24, 0.25, rotation(10000.0, 8)), constant_decay(2, 16, 24, (0.9, 0.97)), 0.7, 1.3), 96),
    layer(latent(3, 12, 8, 20, 24, 32, 0.2, 5000.0), 80),
    layer(pair_2(softmax_side(4, 2, 16, 16, 0.3, rotation(10000.0, 8, (4.0, 1.0, 4.0, 64)), 12), delta_rule(4, 2, 8, 12, 3), 1.2, 0.8), None),
    layer(latent(2, 8, 4, 8, 16, 24, 0.3, 200.0), 48),
], logit_scale=0.7, logit_softcap=12.0)
# multiples of nothing: a width of 100; one query head per key/value head; a window of one token (a token sees itself
# alone) and one wider than any request; convolutions of one tap (no carried inputs) and of five; no rotation at all in
# one attention; a latent layer with one head and one without a rotated part; factors of one; neither a factor nor a
# cap on the logits; a delta rule as the first layer and a pair without a mask in its window attention
CONFIG_B = config(257, 100, 1e-5, [
    layer(pair_2(softmax_side(3, 3, 12, 12, 0.35, rotation(777.0, 12), 1), delta_rule(3, 3, 10, 14, 1), 1.0, 1.0), 50),
    layer(latent(1, 20, 6, 12, 10, 18, 0.25, 1000.0, dims=4), None),
    layer(pair(softmax_side(5, 1, 8, 8, 0.4, rotation(10000.0, 0)), constant_decay(1, 36, 20, (0.8,)), 1.0, 1.0), 33),
    layer(pair_2(softmax_side(2, 1, 20, 20, 0.3, rotation(50.0, 6, (2.0, 1.0, 3.0, 20))), delta_rule(2, 1, 6, 70, 5), 0.5, 2.0), 64),
    layer(latent(4, 6, 0, 10, 12, 14, 0.45, 10000.0), 40),
    layer(pair_2(softmax_side(2, 2, 14, 14, 0.3, rotation(30000.0, 10), 700), delta_rule(1, 1, 36, 8, 2), 0.9, 1.1), None),
])
# multiples of 16, so that the matrix-core attention runs: heads of 64 and 32, windows of 44 (no multiple of a page or
# of a chunk of keys) and of 64 (a page's and a chunk's edge), latents of 64 + 32 and 48 + 16, states of 64 x 80 and
# 160 x 64
CONFIG_C = config(411, 128, 1e-6, [
    layer(latent(4, 32, 32, 48, 64, 64, 0.12, 300000.0, dims=16), 192),
    layer(pair_2(softmax_side(8, 2, 64, 64, 0.1, rotation(500000.0, 32, (6.0, 1.0, 3.0, 256)), 44), delta_rule(4, 2, 64, 80, 5), 0.65, 1.15), 160),
    layer(pair(softmax_side(4, 4, 32, 64, 0.18, rotation(10000.0, 32)), constant_decay(2, 64, 48, (0.6, 0.995)), 1.2, 0.9), 64),
    layer(pair_2(softmax_side(4, 1, 32, 32, 0.15, rotation(10000.0, 16), 64), delta_rule(1, 1, 160, 64, 2), 1.0, 0.7), 96),
    layer(latent(2, 64, 16, 32, 32, 48, 0.11, 1000.0), None),
], logit_scale=0.4, logit_softcap=20.0)
# recurrent pairs alone, each kind twice with sizes of its own; then a model of latent attention alone (no state:
# every step may replay from a graph)
CONFIG_D = config(199, 96, 1e-5, [
    layer(pair(softmax_side(6, 3, 16, 16, 0.3, rotation(10000.0, 16)), constant_decay(3, 8, 40, (0.5, 0.9, 0.998)), 0.8, 1.0), 80),
    layer(pair_2(softmax_side(2, 2, 48, 48, 0.15, rotation(10000.0, 24, (16.0, 1.0, 2.0, 128)), 33), delta_rule(6, 3, 16, 8, 4), 1.0, 1.0), 64),
    layer(pair(softmax_side(2, 1, 24, 8, 0.2, rotation(300.0, 2)), constant_decay(4, 16, 16, (0.7, 0.8, 0.9, 0.95)), 1.1, 0.6), None),
], logit_softcap=30.0)
CONFIG_F = config(150, 72, 1e-5, [
    layer(latent(2, 8, 8, 8, 12, 16, 0.3, 10000.0), 40),
    layer(latent(3, 24, 4, 40, 20, 12, 0.2, 64.0, dims=2), None),
    layer(latent(6, 4, 12, 4, 8, 40, 0.35, 2e6), 56),
], logit_scale=2.0)
CONFIGS = {"A": (CONFIG_A, 5), "B": (CONFIG_B, 6), "C": (CONFIG_C, 7), "D": (CONFIG_D, 8), "F": (CONFIG_F, 10)}
# how peaked the attention is drawn (a factor on the queries' norm weights).  Configuration B is six layers deep, has a
# latent layer with a single head and a width of 100, whose products are rounded to bfloat16 before anything else reads
# them: with the sharpness of the others, bfloat16 rounding of one head's scores alone moves single rows by several per
# cent of the scale, which would hide what the test is for.
SHARPNESS = {"B": 1.5}


def draw_weights(cfg: dict, seed: int, sharp: float = 3.0, ranks=(5, 7)) -> dict[str, torch.Tensor]:
    """name -> float32 tensor whose values are bfloat16 numbers (so that both precisions load the same model).  ranks: the
    inner widths of the delta rule's two low-rank projections (no configuration key names them)."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]

    def matrix(out_f, in_f, gain=1.0):
        return torch.randn(out_f, in_f, generator=g) * (gain / in_f ** 0.5)

    def gains(n):
        return 1.0 + 0.2 * torch.randn(n, generator=g)

    w = {"embed": torch.randn(cfg["vocab"], width, generator=g), "final.norm": gains(width), "head": matrix(cfg["vocab"], width, 2.0)}
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{i}."
        w[p + "norm1"], w[p + "norm1b"] = gains(width), gains(width)
        m, q = entry["mixer"], p + "mix."
        if entry["type"] == "latent_attention":
            nh, dim, rot, vdim = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            w[q + "dq"], w[q + "dq.norm"] = matrix(m["q_rank"], width), gains(m["q_rank"]) * sharp
            w[q + "uq"] = matrix(nh * (dim + rot), m["q_rank"])
            w[q + "dkv"], w[q + "dkv.norm"] = matrix(m["kv_rank"] + rot, width), gains(m["kv_rank"])
            w[q + "uk"], w[q + "uv"] = matrix(nh * dim, m["kv_rank"]), matrix(nh * vdim, m["kv_rank"])
            w[q + "o"] = matrix(width, nh * vdim)
        else:
            left, right = m["left"], m["right"]
            hq, hk, dk, dv = left["heads"], left["kv_heads"], left["dim"], left["vdim"]
            a, b = q + "left.", q + "right."
            w[a + "q"], w[a + "k"] = matrix(hq * dk, width, 2.0), matrix(hk * dk, width, 2.0)
            w[a + "o"] = matrix(width, hq * dv)
            if entry["type"] == "parallel":
                w[a + "v"], w[a + "g"] = matrix(hk * dv, width), matrix(hq * dv, width, 2.0)
                w[a + "q.norm"], w[a + "k.norm"] = gains(dk) * sharp, gains(dk)
                hr, rk, rv = right["heads"], right["dim"], right["vdim"]
                w[b + "q"], w[b + "k"] = matrix(hr * rk, width, 2.0), matrix(hr * rk, width, 2.0)
                w[b + "v"], w[b + "g"] = matrix(hr * rv, width, 2.0), matrix(hr * rv, width, 2.0)
                w[b + "norm"], w[b + "o"] = gains(hr * rv), matrix(width, hr * rv)
            else:
                w[a + "sink"] = 1.5 * torch.randn(hq, generator=g)
                hr, hg, rk, rv, taps = right["heads"], right["kv_heads"], right["dim"], right["vdim"], right["conv"]
                for name, rows in (("q", hg * rk), ("k", hg * rk), ("v", hr * rv)):
                    w[b + name] = matrix(rows, width, 2.0)
                    w[b + name + ".conv"] = 0.6 * torch.randn(rows, taps, generator=g) + (0.5 if taps == 1 else 0.0)
                w[b + "b"] = matrix(hr, width, 2.0)
                w[b + "A_log"] = -0.5 + 0.7 * torch.randn(hr, generator=g)
                w[b + "a1"], w[b + "a2"] = matrix(ranks[0], width, 2.0), matrix(hr * rk, ranks[0], 2.0)
                w[b + "dt_bias"] = torch.randn(hr * rk, generator=g) - 1.0
                w[b + "g1"], w[b + "g2"] = matrix(ranks[1], width, 2.0), matrix(hr * rv, ranks[1], 2.0)
                w[b + "norm"], w[b + "o"] = gains(rv), matrix(width, hr * rv)
        if entry.get("mlp") is None:
            continue
        ff = entry["mlp"]["ff"]
        w[p + "norm2"], w[p + "norm2b"] = gains(width), gains(width)
        w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = matrix(ff, width, 2.0), matrix(ff, width), matrix(width, ff)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def write_model(model_dir: str, cfg: dict, seed: int, change=None, **kw) -> str:
    """Writes config.json and model.safetensors (bfloat16); `change(weights)` may edit the drawn tensors first."""
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    for name, (known, _) in CONFIGS.items():
        if known is cfg and "sharp" not in kw and name in SHARPNESS:
            kw["sharp"] = SHARPNESS[name]
    w = draw_weights(cfg, seed, **kw)
    if change is not None:
        change(w)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in w.items()})
    return model_dir
