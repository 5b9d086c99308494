"""A plain, slow Bubetar decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.

It shares no code with the engine: it reads a model folder with its own few lines and knows the tensor names
itself.  Notation: x [T, W] is the residual stream of one sequence, positions count from 0, a linear weight is
[out, in] and applied as x W^T.

The design: x = embed[token].  A layer has layer norms (a weight, no bias) before and after each of its two branches,
x <- x + LN1b(mixer(LN1(x))), x <- x + LN2b(ff(LN2(x))).  The mixer is one of three: softmax attention whose queries
come through a normed latent and whose keys and values are made from a second normed latent, with one rotated key
part that the heads share ('latent_attention'); grouped-query attention with normed queries and keys, rotation of
neighbouring pairs and an output gate beside a linear attention with a constant decay per head ('parallel'); or
grouped-query attention whose values are its unrotated keys, behind a sliding window with a sink, beside a gated delta
rule with short convolutions and a decay per key channel ('parallel_2').  The two sides of a pair are added with a
constant factor each.  The feed-forward is a gated one with silu.  A last layer norm, the output matrix, a factor and a
tanh cap.
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


# ----------------------------------------------------------------------------- small pieces
def layer_norm(x, weight, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def rotation_frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` {factor, low, high, original} the long wavelengths are
    stretched: f stays where 2 pi / f < original / high, becomes f / factor where 2 pi / f > original / low, and in
    between is (1 - s) f / factor + s f with s = (original / wavelength - low) / (high - low)."""
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, original = sc["factor"], sc["low"], sc["high"], sc["original"]
        out = f.clone()
        for i in range(dims // 2):
            wavelength = 2.0 * math.pi / f[i].item()
            if wavelength < original / high:
                continue
            if wavelength > original / low:
                out[i] = f[i] / factor
            else:
                s = (original / wavelength - low) / (high - low)
                out[i] = (1.0 - s) * f[i] / factor + s * f[i]
        f = out
    return f


def rotate(x, positions, rot: dict, layout: str):
    """x [T, heads, d]: the first rot['dims'] places of every head turn by position * f_i; 'interleaved' pairs the
    places (2i, 2i + 1), 'half' the places (i, i + dims / 2).  The rest passes."""
    dims = rot["dims"]
    if dims == 0:
        return x
    f = rotation_frequencies(rot)
    angle = positions.to(F64)[:, None] * f[None, :]             # [T, dims / 2]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    if layout == "interleaved":
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        half = dims // 2
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


def visible(n_tokens: int, window: int | None) -> torch.Tensor:
    """[T, T] bool: query i sees key j with 0 <= i - j (and i - j < window, if there is one)."""
    i = torch.arange(n_tokens)[:, None]
    j = torch.arange(n_tokens)[None, :]
    seen = j <= i
    if window is not None:
        seen = seen & (i - j < window)
    return seen


def softmax_attention(q, k, v, scale, window=None, sink=None):
    """q [T, heads, dk], k [T, kv heads, dk], v [T, kv heads, dv] -> [T, heads, dv].  Query head h reads key/value head
    h // (heads / kv heads).  With a sink [heads], exp(sink_h) joins the denominator (unscaled, no value)."""
    t, nq, _ = q.shape
    nkv = k.shape[1]
    seen = visible(t, window)
    heads = []
    for head in range(nq):
        g = head // (nq // nkv)
        s = (q[:, head] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        if sink is None:
            p = torch.softmax(s, dim=-1)
        else:
            top = torch.maximum(s.max(-1, keepdim=True).values, sink[head])
            e = torch.exp(s - top)
            p = e / (e.sum(-1, keepdim=True) + torch.exp(sink[head] - top))
        heads.append(p @ v[:, g])
    return torch.stack(heads, dim=1)


# ----------------------------------------------------------------------------- mixers
def latent_attention(h, w, p, m, eps):
    t = h.shape[0]
    nh, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = torch.arange(t)
    c_q = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (c_q @ w[p + "uq"].T).view(t, nh, dim + rot_dim)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = rotate(down[:, rank:].view(t, 1, rot_dim), positions, m["rot"], "interleaved")
    q_rot = rotate(q[..., dim:], positions, m["rot"], "interleaved")
    k_plain = (c @ w[p + "uk"].T).view(t, nh, dim)
    v = (c @ w[p + "uv"].T).view(t, nh, vdim)
    q_all = torch.cat([q[..., :dim], q_rot], dim=-1)
    k_all = torch.cat([k_plain, k_rot.expand(t, nh, rot_dim)], dim=-1)
    o = softmax_attention(q_all, k_all, v, m["scale"])
    return o.reshape(t, nh * vdim) @ w[p + "o"].T


def gated_normed_attention(h, w, p, m, eps):
    """The left side of 'parallel': queries and keys normed per head with a weight, rotation of neighbouring pairs,
    every earlier key, the heads' outputs times sigmoid(W_g h)."""
    t = h.shape[0]
    nh, g, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(t)
    q = rms_norm((h @ w[p + "q"].T).view(t, nh, dim), w[p + "q.norm"], eps)
    k = rms_norm((h @ w[p + "k"].T).view(t, g, dim), w[p + "k.norm"], eps)
    v = (h @ w[p + "v"].T).view(t, g, vdim)
    q, k = rotate(q, positions, m["rot"], "interleaved"), rotate(k, positions, m["rot"], "interleaved")
    o = softmax_attention(q, k, v, m["scale"]).reshape(t, nh * vdim)
    return (o * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def constant_decay_scan(q, k, v, decay, state=None):
    """Per head S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k [T, heads, dk]; v [T, heads, dv]."""
    t, nh, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(nh, dk, dv, dtype=F64) if state is None else state.clone()
    d = torch.as_tensor(decay, dtype=F64)[:, None, None]
    out = torch.zeros(t, nh, dv, dtype=F64)
    for i in range(t):
        s = d * s + k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", s, q[i])
    return out, s


def lightning_attention(h, w, p, m, eps):
    """The right side of 'parallel'."""
    t = h.shape[0]
    nh, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).view(t, nh, dim)
    k = silu(h @ w[p + "k"].T).view(t, nh, dim)
    v = silu(h @ w[p + "v"].T).view(t, nh, vdim)
    o, _ = constant_decay_scan(q, k, v, m["decay"])
    o = rms_norm(o.reshape(t, nh * vdim), w[p + "norm"], eps)            # all heads together
    return (o * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def key_valued_window_attention(h, w, p, m, eps):
    """The left side of 'parallel_2': the values are the keys as projected; rotation of the halves with stretched
    frequencies; queries and keys divided by their root mean square after the rotation; a window and a sink."""
    t = h.shape[0]
    nh, g, dim = m["heads"], m["kv_heads"], m["dim"]
    positions = torch.arange(t)
    q = (h @ w[p + "q"].T).view(t, nh, dim)
    k = (h @ w[p + "k"].T).view(t, g, dim)
    v = k.clone()
    q = rms_norm(rotate(q, positions, m["rot"], "half"), None, eps)
    k = rms_norm(rotate(k, positions, m["rot"], "half"), None, eps)
    window = m["mask"]["size"] if m.get("mask") else None
    o = softmax_attention(q, k, v, m["scale"], window, w[p + "sink"])
    return o.reshape(t, nh * dim) @ w[p + "o"].T


def short_convolution(x, taps_weight, before=None):
    """x [T, C], taps_weight [C, taps] (the last column is the current token's), zeros before the start (or the
    rows `before` [taps - 1, C]) -> [T, C]."""
    t, c = x.shape
    taps = taps_weight.shape[1]
    pad = torch.zeros(taps - 1, c, dtype=F64) if before is None else before
    z = torch.cat([pad, x], dim=0)
    out = torch.zeros(t, c, dtype=F64)
    for j in range(taps):
        out += z[j : j + t] * taps_weight[:, j]
    return out


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule_scan(q, k, v, beta, g, state=None):
    """Per head S <- g * S (rows of S are key channels); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    q, k, g [T, heads, dk]; v [T, heads, dv]; beta [T, heads]."""
    t, nh, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(nh, dk, dv, dtype=F64) if state is None else state.clone()
    out = torch.zeros(t, nh, dv, dtype=F64)
    for i in range(t):
        s = g[i][:, :, None] * s
        u = beta[i][:, None] * (v[i] - torch.einsum("hkv,hk->hv", s, k[i]))
        s = s + k[i][:, :, None] * u[:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", s, q[i])
    return out, s


def gated_delta_rule(h, w, p, m, eps):
    """The right side of 'parallel_2'."""
    t = h.shape[0]
    nh, g, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])).view(t, g, dim)
    k = silu(short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])).view(t, g, dim)
    v = silu(short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])).view(t, nh, vdim)
    q, k = unit(q) * dim ** -0.5, unit(k)
    group = nh // g
    q = q.repeat_interleave(group, dim=1)
    k = k.repeat_interleave(group, dim=1)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                 # [T, heads]
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    rate = torch.exp(w[p + "A_log"])[None, :, None]
    decay = torch.exp(-rate * torch.nn.functional.softplus(z).view(t, nh, dim))
    o, _ = delta_rule_scan(q, k, v, beta, decay)
    o = rms_norm(o, w[p + "norm"], eps)                                    # per head, the weight shared by the heads
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(t, nh, vdim)
    return (o * gate).reshape(t, nh * vdim) @ w[p + "o"].T


def gated_feed_forward(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def mixer(kind, h, w, p, m, eps):
    if kind == "latent_attention":
        return latent_attention(h, w, p, m, eps)
    if kind == "parallel":
        return (m["left_scale"] * gated_normed_attention(h, w, p + "left.", m["left"], eps)
                + m["right_scale"] * lightning_attention(h, w, p + "right.", m["right"], eps))
    if kind == "parallel_2":
        return (m["left_scale"] * key_valued_window_attention(h, w, p + "left.", m["left"], eps)
                + m["right_scale"] * gated_delta_rule(h, w, p + "right.", m["right"], eps))
    raise ValueError(kind)


# ----------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, collect=None):
    """Logits [T, vocab] (float64) of one sequence; collect, if a list, gets the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = mixer(layer["type"], layer_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
        x = x + layer_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(layer["mlp"]["kind"])
            y = gated_feed_forward(layer_norm(x, w[p + "norm2"], eps), w, p + "mlp.")
            x = x + layer_norm(y, w[p + "norm2b"], eps)
        if collect is not None:
            collect.append(x.clone())
    logits = layer_norm(x, w["final.norm"], eps) @ w["head"].T
    if cfg.get("logit_scale") is not None:
        logits = logits * cfg["logit_scale"]
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
