"""A plain, slow Kezolix decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.

It shares no code with the engine: it reads a model folder with its own few lines and knows the tensor names
itself.  Notation: x [T, W] is the residual stream of one sequence, positions count from 0, a linear weight is
[out, in] and applied as x W^T.

The design: x = embed[token] + pos[position].  A layer has layer norms (a weight, no bias) before and after each of
its two branches, x <- x + m LN1b(mixer(LN1(x))), x <- x + m LN2b(ff(LN2(x))), and what the next layer (or the output)
reads is a learned weighted sum of the embedding and of every layer's result so far.  The mixer is either a
grouped-query softmax attention without rotation (queries and keys RMS-normed over the whole projection, a penalty
per head that grows with the distance, keys visible only inside the query's own block of positions; such a layer may
read another layer's keys and values instead of making its own), or a gated linear recurrence with a matrix state per
head whose forget gate has a learned lower bound and also sets what is written.  The feed-forward is dense with a
normed polynomial as activation, or a mixture of experts (squared relu) with a gated shared expert.  A last layer
norm and the output matrix.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np
import torch

F64 = torch.float64


def read_safetensors(path: str) -> dict[str, torch.Tensor]:
    with open(path, "rb") as f:
        raw = f.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8 : 8 + hlen])
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        buf = raw[base + b : base + e]
        if info["dtype"] == "F32":
            a = torch.from_numpy(np.frombuffer(buf, dtype="<f4").copy())
        elif info["dtype"] == "BF16":
            u16 = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            a = torch.from_numpy(u16.view(np.float32).copy())
        else:
            raise ValueError(info["dtype"])
        out[name] = a.reshape(info["shape"]).to(F64)
    return out


def read_model(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


# ----------------------------------------------------------------------------- mechanisms
def layer_norm(x, weight, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def head_slopes(heads: int) -> torch.Tensor:
    """2^(-8 (h + 1) / heads) for head h."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=F64)


def block_visible(n_tokens: int, size: int | None) -> torch.Tensor:
    """[T, T] bool: query i sees key j <= i when both lie in the same block of `size` positions (None: every j <= i)."""
    i = torch.arange(n_tokens)[:, None]
    j = torch.arange(n_tokens)[None, :]
    seen = j <= i
    if size is not None:
        seen = seen & (i // size == j // size)
    return seen


def keys_and_values(h, w, p, m, eps):
    """What an attention layer leaves for itself and for the layers that read from it: keys after their norm
    [T, kv heads, dim] and values [T, kv heads, vdim]."""
    t = h.shape[0]
    k = rms_norm(h @ w[p + "k"].T, w[p + "k.norm"], eps)             # over the whole projection
    v = h @ w[p + "v"].T
    return k.view(t, m["kv_heads"], m["dim"]), v.view(t, m["kv_heads"], m["vdim"])


def sloped_block_attention(q, k, v, scale, size):
    """q [T, heads, dk], k [T, kv heads, dk], v [T, kv heads, dv] of one sequence -> [T, heads, dv]: softmax over the
    keys that `block_visible` allows of (q . k) * scale - slope_head * (i - j)."""
    t, nq, _ = q.shape
    nkv = k.shape[1]
    seen = block_visible(t, size)
    distance = (torch.arange(t)[:, None] - torch.arange(t)[None, :]).to(F64)
    slopes = head_slopes(nq)
    heads = []
    for head in range(nq):
        g = head // (nq // nkv)
        s = (q[:, head] @ k[:, g].T) * scale - slopes[head] * distance
        s = s.masked_fill(~seen, -math.inf)
        heads.append(torch.softmax(s, dim=-1) @ v[:, g])
    return torch.stack(heads, dim=1)


def block_attention(h, w, p, m, eps, k, v):
    """The attention mixer on the normed input h [T, W] with the keys and values it is given."""
    t = h.shape[0]
    q = rms_norm(h @ w[p + "q"].T, w[p + "q.norm"], eps).view(t, m["heads"], m["dim"])
    size = m["mask"]["size"] if m.get("mask") else None
    return sloped_block_attention(q, k, v, m["scale"], size).reshape(t, -1) @ w[p + "o"].T


def forget_gates(h, w, p):
    """[T, heads * dim]: lower + (1 - lower) * sigmoid(W_f h + b)."""
    low = w[p + "lower"]
    return low + (1.0 - low) * torch.sigmoid(h @ w[p + "f"].T + w[p + "f.b"])


def gated_state_scan(q, f, v, state=None):
    """Per head S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t.  q, f [T, heads, dk]; v [T, heads, dv].
    Returns o [T, heads, dv] and the last state [heads, dk, dv]."""
    t, nh, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(nh, dk, dv, dtype=F64) if state is None else state.clone()
    out = torch.zeros(t, nh, dv, dtype=F64)
    for i in range(t):
        s = f[i][:, :, None] * s + (1.0 - f[i])[:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", s, q[i])
    return out, s


def gated_recurrence(h, w, p, m, eps):
    """The recurrent mixer."""
    t = h.shape[0]
    nh, dk, dv = m["heads"], m["dim"], m["vdim"]
    z = h @ w[p + "q"].T
    q = (z * torch.sigmoid(z)).view(t, nh, dk)
    f = forget_gates(h, w, p).view(t, nh, dk)
    v = (h @ w[p + "v"].T).view(t, nh, dv)
    o, _ = gated_state_scan(q, f, v)
    o = rms_norm(o, w[p + "norm"], eps).reshape(t, nh * dv)          # per head, the weight shared by the heads
    return o @ w[p + "o"].T


def normed_polynomial(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with N(u) = u / sqrt(mean(u^2) + eps) over a token's values."""
    n = lambda u: u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)
    return coef[0] * n(z) + coef[1] * n(z * z) + coef[2] * n(z * z * z) + coef[3]


def dense_feed_forward(h, w, p, eps):
    return normed_polynomial(h @ w[p + "up"].T, w[p + "act"], eps) @ w[p + "down"].T


def squared_relu_expert(h, w, p):
    return (torch.relu(h @ w[p + "up"].T) ** 2) @ w[p + "down"].T


def route(h, w, p, router):
    """Chosen experts [T, top] and their weights: softmax over all experts; the choice goes by score + correction,
    the weights are the chosen scores over their sum, times the router's scale."""
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)
    idx = torch.argsort(-(s + w[p + "correction"]), dim=-1, stable=True)[:, : router["top"]]
    chosen = torch.gather(s, -1, idx)
    return idx, chosen / (chosen.sum(-1, keepdim=True) + 1e-20) * router["scale"]


def expert_mixture(h, w, p, mlp):
    idx, weight = route(h, w, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), weight[t]):
            out[t] += a * squared_relu_expert(h[t : t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared") is not None:
        out = out + squared_relu_expert(h, w, p + "shared.") * torch.sigmoid(h @ w[p + "shared.sg"].T)
    return out


def depth_average(results, weights):
    """sum_j weights[j] * results[j]."""
    return sum(a * x for a, x in zip(weights, results))


# ----------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, collect=None):
    """Logits [T, vocab] (float64) of one sequence; collect, if a list, gets what goes on after every layer."""
    eps = cfg["norm"]["eps"]
    mult = cfg["residual_mult"]
    t = len(tokens)
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] + w["pos"][:t]
    results = [x]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = layer_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            if m.get("kv_from") is not None:
                k, v = kept[m["kv_from"]]
            else:
                k, v = kept[i] = keys_and_values(h, w, p + "mix.", m, eps)
            y = block_attention(h, w, p + "mix.", m, eps, k, v)
        elif layer["type"] == "hgrn2":
            y = gated_recurrence(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + mult * layer_norm(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, w[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = dense_feed_forward(h, w, p + "mlp.", eps)
            elif mlp["kind"] == "moe":
                y = expert_mixture(h, w, p + "mlp.", mlp)
            else:
                raise ValueError(mlp["kind"])
            x = x + mult * layer_norm(y, w[p + "norm2b"], eps)
        results.append(x)
        x = depth_average(results, w[p + "dwa"])
        if collect is not None:
            collect.append(x.clone())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T
