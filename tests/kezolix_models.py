"""Small Kezolix configurations and weights for the tests: sizes that differ in every respect, weights drawn so that
activations are of order one, attention is peaked, the depth average mixes every earlier result with weights of either
sign, the forget gates lie between their lower bounds and one, and the router's correction changes who is chosen (with
weights of N(0, 0.02) a key that is wrongly seen, a lost state or a wrong choice would hardly move the logits).  A layer
norm stands behind every feed-forward, so the size of an expert's output does not matter, only its direction: where a
mixture has a shared expert the routed experts' outputs are small beside it, and where it has none the experts differ
little from each other, so that a choice between two nearly tied experts, which bfloat16 rounding of the router's input
may turn, stays below the bfloat16 tolerance while float32 (3e-5) sees every fault of the routing.  The tensor names
are written out here, not taken from the engine."""
from __future__ import annotations

import json
import os

import torch

from easy_gpt.cpp_amd.weights import write_safetensors


def attention(heads, kv_heads, dim, vdim, scale, block, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if block:
        m["mask"] = {"size": block}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention", m


def recurrence(heads, dim, vdim):
    return "hgrn2", {"heads": heads, "dim": dim, "vdim": vdim}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared_ff, scale=1.0):
    m = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff}
    return m


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(vocab, width, max_positions, eps, mult, layers):
    return {"architecture": "Kezolix", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps},
            "residual_mult": mult, "layers": layers}


# an attention layer whose keys and values a later layer reads with a block of its own; a layer without a feed-forward
CONFIG_A = config(300, 64, 512, 1e-6, 0.6, [
    layer(attention(4, 2, 16, 24, 0.25, 12), dense(96)),
    layer(recurrence(2, 16, 24), moe(6, 2, 48, 64, 1.5)),
    layer(attention(4, 2, 16, 24, 0.3, 30, kv_from=0), moe(4, 3, 40, 32, 0.5)),
    layer(recurrence(3, 10, 12), None),
])
# multiples of nothing: a width of 100, a recurrence first, one query head per key/value head, no blocks at all (every
# earlier key), blocks of one token (a token sees itself alone) and of 7, one expert per token without a shared
# expert, every expert chosen, a factor of one on the branches
CONFIG_B = config(257, 100, 400, 1e-5, 1.0, [
    layer(recurrence(3, 10, 12), moe(5, 1, 50, None, 2.0)),
    layer(attention(3, 3, 12, 20, 0.3, None), dense(50)),
    layer(attention(5, 1, 8, 8, 0.35, 1), None),
    layer(recurrence(1, 36, 70), moe(3, 3, 30, 20, 1.0)),
    layer(attention(2, 1, 20, 12, 0.2, 7), dense(33)),
])
# multiples of 16, so that the matrix-core attention runs: blocks of 100 (no multiple of a page or of a chunk of keys),
# of 40 on the first layer's keys, and of 64 (a page's and a chunk's edge); keys of 64 and 160 in the states
CONFIG_C = config(411, 128, 3000, 1e-6, 0.8, [
    layer(attention(8, 2, 64, 32, 0.11, 100), moe(8, 2, 64, 32, 2.0)),
    layer(recurrence(2, 64, 80), dense(192)),
    layer(attention(8, 2, 64, 32, 0.15, 40, kv_from=0), dense(64)),
    layer(recurrence(1, 160, 64), moe(16, 4, 32, 96, 1.0)),
    layer(attention(4, 4, 32, 64, 0.18, 64), moe(4, 1, 48, 16, 3.0)),
])
# attention alone (no state: every step may replay from a graph), the second layer on the first one's keys and values
CONFIG_D = config(199, 96, 700, 1e-5, 0.7, [
    layer(attention(6, 3, 16, 16, 0.3, 50), dense(80)),
    layer(attention(6, 3, 16, 16, 0.2, None, kv_from=0), moe(4, 2, 32, 48, 1.0)),
    layer(attention(2, 2, 48, 32, 0.15, 33), dense(64)),
])
# recurrences alone (no pages at all), the last one without a feed-forward
CONFIG_F = config(150, 72, 300, 1e-5, 0.9, [
    layer(recurrence(2, 8, 8), dense(40)),
    layer(recurrence(1, 24, 40), moe(3, 2, 24, 8, 1.0)),
    layer(recurrence(4, 16, 8), None),
])
# a deeper one: nine layers, two layers with keys of their own that are not the first ones, each read by two later
# layers with blocks of their own (one with no blocks), three query heads per key/value head, a recurrence between
CONFIG_G = config(321, 80, 500, 1e-5, 0.4, [
    layer(recurrence(2, 16, 16), dense(48)),
    layer(attention(6, 2, 16, 32, 0.2, 37), None),
    layer(attention(6, 2, 16, 32, 0.25, 9, kv_from=1), dense(40)),
    layer(attention(2, 2, 24, 16, 0.2, 64), moe(4, 2, 24, 16, 1.0)),
    layer(recurrence(2, 16, 16), None),
    layer(attention(6, 2, 16, 32, 0.3, None, kv_from=1), moe(5, 2, 16, None, 2.0)),
    layer(attention(2, 2, 24, 16, 0.3, 16, kv_from=3), dense(40)),
    layer(attention(2, 2, 24, 16, 0.15, 150, kv_from=3), None),
    layer(recurrence(5, 8, 16), dense(56)),
])
CONFIGS = {"A": (CONFIG_A, 5), "B": (CONFIG_B, 6), "C": (CONFIG_C, 7), "D": (CONFIG_D, 8), "F": (CONFIG_F, 10), "G": (CONFIG_G, 11)}


def draw_weights(cfg: dict, seed: int, sharp: float = 3.0) -> dict[str, torch.Tensor]:
    """name -> float32 tensor whose values are bfloat16 numbers (so that both precisions load the same model)."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]

    def matrix(out_f, in_f, gain=1.0):
        return torch.randn(out_f, in_f, generator=g) * (gain / in_f ** 0.5)

    def gains(n):
        return 1.0 + 0.2 * torch.randn(n, generator=g)

    w = {"embed": torch.randn(cfg["vocab"], width, generator=g), "pos": 0.5 * torch.randn(cfg["max_positions"], width, generator=g),
         "final.norm": gains(width), "head": matrix(cfg["vocab"], width, 2.0)}
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{i}."
        w[p + "norm1"], w[p + "norm1b"] = gains(width), gains(width)
        mix = torch.randn(i + 2, generator=g) * 0.6          # every earlier result with a weight of either sign
        mix[-1] += 1.0
        w[p + "dwa"] = mix
        m, q = entry["mixer"], p + "mix."
        if entry["type"] == "attention":
            hq, hk, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[q + "q"], w[q + "q.norm"] = matrix(hq * dk, width), gains(hq * dk) * sharp
            if m.get("kv_from") is None:
                w[q + "k"], w[q + "v"], w[q + "k.norm"] = matrix(hk * dk, width), matrix(hk * dv, width), gains(hk * dk)
            w[q + "o"] = matrix(width, hq * dv)
        else:
            hr, dk, dv = m["heads"], m["dim"], m["vdim"]
            w[q + "q"], w[q + "f"], w[q + "v"] = matrix(hr * dk, width, 2.0), matrix(hr * dk, width, 2.0), matrix(hr * dv, width)
            w[q + "f.b"] = 1.0 + torch.randn(hr * dk, generator=g)
            w[q + "lower"] = 0.9 * torch.rand(hr * dk, generator=g)
            w[q + "norm"], w[q + "o"] = gains(dv), matrix(width, hr * dv)
        mlp = entry.get("mlp")
        if mlp is None:
            continue
        w[p + "norm2"], w[p + "norm2b"] = gains(width), gains(width)
        q = p + "mlp."
        if mlp["kind"] == "dense":
            w[q + "up"], w[q + "down"] = matrix(mlp["ff"], width), matrix(width, mlp["ff"])
            w[q + "act"] = torch.tensor([0.6, -0.4, 0.3, 0.2]) + 0.2 * torch.randn(4, generator=g)
            continue
        ff, n = mlp["expert"]["ff"], mlp["router"]["experts"]
        shared = mlp.get("shared")
        common_up, common_down = matrix(ff, width, 2.0), matrix(width, ff)
        for e in range(n):
            w[f"{q}e{e}.up"] = matrix(ff, width) if shared else common_up + matrix(ff, width, 0.03)
            w[f"{q}e{e}.down"] = matrix(width, ff, 0.004) if shared else common_down + matrix(width, ff, 0.015)
        w[q + "router"] = matrix(n, width, 4.0)
        w[q + "correction"] = torch.where(torch.rand(n, generator=g) < 0.5, torch.zeros(n), torch.full((n,), 0.25))
        if shared:
            f2 = shared["ff"]
            w[q + "shared.up"], w[q + "shared.down"], w[q + "shared.sg"] = matrix(f2, width, 2.0), matrix(width, f2), matrix(1, width, 2.0)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def write_model(model_dir: str, cfg: dict, seed: int, change=None) -> str:
    """Writes config.json and model.safetensors (bfloat16); `change(weights)` may edit the drawn tensors first."""
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    w = draw_weights(cfg, seed)
    if change is not None:
        change(w)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in w.items()})
    return model_dir
