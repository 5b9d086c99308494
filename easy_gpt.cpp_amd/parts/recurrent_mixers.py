"""Mixers with a matrix state per head and request that stand beside an attention in one layer.

`ConstantDecayAttention`: linear attention whose state decays by one constant per head,
S_t = d_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q, k, v = silu of their projections and no other scale.  The heads'
outputs are RMS-normed together (one statistic over all heads, a weight per value), multiplied by sigmoid(W_g x) and
projected.

`GatedDeltaRule`: queries, keys and values pass a short causal convolution over time per channel (zeros before the
sequence's start) and silu; queries and keys are made unit vectors per head (x / sqrt(sum x^2 + unit_eps)), queries
also times key_dim^(-1/2).  With beta = sigmoid(W_b x) per head and the decay g = exp(-exp(A_h) softplus(W_a2 W_a1 x +
dt)) per head and key channel, a token does S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  A head's
output is divided by its root mean square, multiplied by a weight that the heads share and by sigmoid(W_g2 W_g1 x),
and projected.  Several value heads may share a query/key head.

Both keep their state in float32, one record per request (`state_need`), zero for a new request, and a step walks its
tokens in order, so a prompt may be cut anywhere.  The delta rule's record also holds the last taps - 1 inputs of the
convolutions.  Decays, gates, unit norms, the recurrence and the norms are float32; the input product stays unrounded
until they have used it.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import StateNeed, register_part
from .branch_mixers import _Branch
from .spec import ParamSpec


def _sizes_ok(key_dim: int, value_dim: int) -> None:
    if not (0 < int(key_dim) <= 1024 and 0 < int(value_dim) <= 4096):
        raise ValueError(f"key size {key_dim} / value size {value_dim} is not supported by the state scans (keys up to "
                         "1024, values up to 4096)")


class ConstantDecayAttention(_Branch):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, decay, eps: float,
                 names: dict | None = None):
        """decay: one number per head.  names: tensor names behind `prefix` of q, k, v, g, norm, o."""
        _sizes_ok(key_dim, value_dim)
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.key_dim, self.value_dim = int(n_heads), int(key_dim), int(value_dim)
        self.decay_values = tuple(float(d) for d in decay)
        if len(self.decay_values) != self.n_heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.n_heads} heads")
        self.eps = float(eps)
        self.names = dict(q="q", k="k", v="v", g="g", norm="norm", o="o")
        self.names.update(names or {})
        self.qk_width, self.v_width = self.n_heads * self.key_dim, self.n_heads * self.value_dim
        self.w_in = self.w_o = self.norm_weight = self.decay = None

    def state_need(self):
        return StateNeed((self.n_heads, self.key_dim, self.value_dim), torch.float32)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        return [
            ParamSpec(p + n["q"], (self.qk_width, h)), ParamSpec(p + n["k"], (self.qk_width, h)),
            ParamSpec(p + n["v"], (self.v_width, h)), ParamSpec(p + n["g"], (self.v_width, h)),
            ParamSpec(p + n["norm"], (self.v_width,), role="norm_scale"),
            ParamSpec(p + n["o"], (h, self.v_width)),
        ]

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        w = torch.cat([get(p + n[x]).to(dtype) for x in ("q", "k", "v", "g")], dim=0)       # one product reads x
        self.w_in = w.to(device).contiguous()
        self.norm_weight = self._to(get(p + n["norm"]), "compute", dtype, device)
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32).to(device)

    def branch(self, x, ctx, cache, state):
        k = kernels.backend()
        t = x.shape[0]
        qk, vw = self.qk_width, self.v_width
        proj = k.product(x, self.w_in, unrounded=True)                 # [q | k | v | g]
        o = k.decayed_state_scan(proj, x.dtype, 0, qk, 2 * qk, 1.0, None, state.data, state.slots, state.fresh_device,
                                 ctx.q_start, ctx.q_len, self.n_heads, self.key_dim, self.value_dim, q_silu=True,
                                 k_silu=True, v_silu=True, head_decay=self.decay)
        gated = torch.empty((t, vw), dtype=x.dtype, device=x.device)
        # all heads are normed together: one "head" as wide as all of them
        k.head_norm_gate(o, self.norm_weight, self.eps, proj, 2 * qk + vw, gated, 1, vw, gate_act="sigmoid")
        return k.product(gated, self.w_o, unrounded=True), None


class GatedDeltaRule(_Branch):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int, taps: int,
                 eps: float, unit_eps: float = 1e-6, decay_rank: int = 16, gate_rank: int = 16, names: dict | None = None):
        """n_heads value heads on n_kv_heads query/key heads; taps: the convolutions' length in tokens; decay_rank,
        gate_rank: the inner widths of the two low-rank projections (stored tensors decide; these are what random
        weights draw).  names: tensor names behind `prefix` of q, k, v (their convolutions are `<name>.conv`), beta,
        rate (the logarithm of each head's decay rate), decay_in, decay_out, decay_bias, gate_in, gate_out, norm, o."""
        _sizes_ok(key_dim, value_dim)
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads ({n_heads}) must be a multiple of n_kv_heads ({n_kv_heads})")
        if not 1 <= int(taps) <= 16:
            raise ValueError(f"a convolution of {taps} taps is not supported (1 to 16)")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.n_kv_heads = int(n_heads), int(n_kv_heads)
        self.key_dim, self.value_dim, self.taps = int(key_dim), int(value_dim), int(taps)
        self.eps, self.unit_eps = float(eps), float(unit_eps)
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        self.names = dict(q="q", k="k", v="v", conv=".conv", beta="b", rate="A_log", decay_in="a1", decay_out="a2",
                          decay_bias="dt_bias", gate_in="g1", gate_out="g2", norm="norm", o="o")
        self.names.update(names or {})
        self.qk_width, self.v_width = self.n_kv_heads * self.key_dim, self.n_heads * self.value_dim
        self.decay_width = self.n_heads * self.key_dim
        self.conv_width = 2 * self.qk_width + self.v_width
        self.matrix_floats = self.n_heads * self.key_dim * self.value_dim
        self.w_in = self.w_o = self.w_conv = self.w_decay = self.b_decay = self.rates = self.w_gate = self.norm_weight = None

    def state_need(self):
        # the matrices of all heads, then the convolutions' last taps - 1 inputs [taps - 1][q | k | v channels]
        return StateNeed((self.matrix_floats + (self.taps - 1) * self.conv_width,), torch.float32)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        c = n["conv"]
        return [
            ParamSpec(p + n["q"], (self.qk_width, h)), ParamSpec(p + n["q"] + c, (self.qk_width, self.taps)),
            ParamSpec(p + n["k"], (self.qk_width, h)), ParamSpec(p + n["k"] + c, (self.qk_width, self.taps)),
            ParamSpec(p + n["v"], (self.v_width, h)), ParamSpec(p + n["v"] + c, (self.v_width, self.taps)),
            ParamSpec(p + n["beta"], (self.n_heads, h)),
            ParamSpec(p + n["rate"], (self.n_heads,), role="bias", dtype="float32"),
            ParamSpec(p + n["norm"], (self.value_dim,), role="norm_scale"),
            ParamSpec(p + n["decay_in"], (self.decay_rank, h), free_axes=(0,)),
            ParamSpec(p + n["decay_out"], (self.decay_width, self.decay_rank), free_axes=(1,)),
            ParamSpec(p + n["decay_bias"], (self.decay_width,), role="bias"),
            ParamSpec(p + n["gate_in"], (self.gate_rank, h), free_axes=(0,)),
            ParamSpec(p + n["gate_out"], (self.v_width, self.gate_rank), free_axes=(1,)),
            ParamSpec(p + n["o"], (h, self.v_width)),
        ]

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        c = n["conv"]
        d_in, d_out, g_in, g_out = (get(p + n[x]) for x in ("decay_in", "decay_out", "gate_in", "gate_out"))
        for low, high, a, b in ((d_in, d_out, "decay_in", "decay_out"), (g_in, g_out, "gate_in", "gate_out")):
            if low.shape[0] != high.shape[1]:
                raise ValueError(f"{p + n[a]} has {low.shape[0]} rows, {p + n[b]} {high.shape[1]} columns: the two "
                                 "projections must share their inner width")
        self.decay_rank, self.gate_rank = int(d_in.shape[0]), int(g_in.shape[0])
        rows = [get(p + n[x]).to(dtype) for x in ("q", "k", "v", "beta")] + [d_in.to(dtype), g_in.to(dtype)]
        self.w_in = torch.cat(rows, dim=0).to(device).contiguous()          # [q | k | v | beta | decay low | gate low]
        self.w_conv = torch.cat([get(p + n[x] + c).to(dtype) for x in ("q", "k", "v")], dim=0).to(device).contiguous()
        self.w_decay = self._to(d_out, "compute", dtype, device)
        self.b_decay = self._to(get(p + n["decay_bias"]), "compute", dtype, device)
        # the decay is exp(-rate_h softplus(z)): one rate per head, repeated over the head's key channels
        rate = torch.exp(get(p + n["rate"]).to(torch.float32))
        self.rates = rate.repeat_interleave(self.key_dim).to(device).contiguous()
        self.w_gate = self._to(g_out, "compute", dtype, device)
        self.norm_weight = self._to(get(p + n["norm"]), "compute", dtype, device)
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)

    def branch(self, x, ctx, cache, state):
        k = kernels.backend()
        t = x.shape[0]
        qk, vw, nh = self.qk_width, self.v_width, self.n_heads
        beta_off = self.conv_width
        low_off = beta_off + nh
        proj = k.product(x, self.w_in, unrounded=True)
        # exp(-rate softplus(z)) = sigmoid(-z)^rate
        decay = k.channel_decay(proj, low_off, self.decay_rank, self.w_decay, self.b_decay, 1.0, rates=self.rates, negate=True)
        gate = k.channel_decay(proj, low_off + self.decay_rank, self.gate_rank, self.w_gate, None, 1.0)     # sigmoid(W_g2 W_g1 x)
        ops = k.short_conv(proj, x.dtype, 0, self.w_conv, self.taps, 2 * self.n_kv_heads, self.key_dim, self.n_kv_heads,
                           self.key_dim ** -0.5, self.unit_eps, beta_off, nh, state.data, self.matrix_floats, state.slots,
                           state.fresh_device, ctx.q_start, ctx.q_len, ctx.max_q_len)
        o = k.delta_rule_scan(ops, 0, qk, 2 * qk, self.conv_width, decay, state.data, 0, state.slots, state.fresh_device,
                              ctx.q_start, ctx.q_len, nh, self.n_kv_heads, self.key_dim, self.value_dim)
        gated = torch.empty((t, vw), dtype=x.dtype, device=x.device)
        k.head_norm_gate(o, self.norm_weight, self.eps, gate[None], 0, gated, nh, self.value_dim, gate_act="factor")
        return k.product(gated, self.w_o, unrounded=True), None


register_part("mixer", "constant_decay_attention", ConstantDecayAttention)
register_part("mixer", "gated_delta_rule", GatedDeltaRule)
