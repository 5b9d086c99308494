"""A linear recurrence with a matrix state per head whose forget gate also decides what is written.

Per head and key channel the gate is f = l + (1 - l) * sigmoid(W_f x + b) with a learned lower bound l; the state
S [key size, value size] moves as S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, and the output is o_t = S_t^T q_t with
q = silu(W_q x): there is no key projection and no other scale.  A head's output is RMS-normed over the value size with
a weight that the heads share; the heads are concatenated and projected.  The state is float32, one record per
request (`state_need`), zero for a new request, and a step walks its tokens in order, so a prompt may be cut anywhere.
Gates, the recurrence and the norm are float32; the input product stays unrounded until they have used it.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Mixer, StateNeed, register_part
from .spec import ParamSpec


class BoundedGateRecurrence(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, eps: float,
                 names: dict | None = None):
        if not (0 < int(key_dim) <= 4096 and 0 < int(value_dim) <= 4096):
            raise ValueError(f"key size {key_dim} / value size {value_dim} is not supported by the state scan (1 to 4096)")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.key_dim, self.value_dim = int(n_heads), int(key_dim), int(value_dim)
        self.eps = float(eps)
        self.names = dict(q="q", f="f", f_bias="f.b", lower="lower", v="v", norm="norm", o="o")
        self.names.update(names or {})
        self.qk_width, self.v_width = self.n_heads * self.key_dim, self.n_heads * self.value_dim
        self.w_in = self.w_o = self.f_bias = self.lower = self.norm_weight = None

    def state_need(self):
        return StateNeed((self.n_heads, self.key_dim, self.value_dim), torch.float32)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        return [
            ParamSpec(p + n["q"], (self.qk_width, h)), ParamSpec(p + n["f"], (self.qk_width, h)),
            ParamSpec(p + n["f_bias"], (self.qk_width,), role="bias"), ParamSpec(p + n["lower"], (self.qk_width,), role="bias"),
            ParamSpec(p + n["v"], (self.v_width, h)), ParamSpec(p + n["norm"], (self.value_dim,), role="norm_scale"),
            ParamSpec(p + n["o"], (h, self.v_width)),
        ]

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        self.w_in = torch.cat([get(p + n[x]).to(dtype) for x in ("q", "f", "v")], dim=0).to(device).contiguous()
        self.f_bias = self._to(get(p + n["f_bias"]), "compute", dtype, device)
        self.lower = self._to(get(p + n["lower"]), "compute", dtype, device)
        self.norm_weight = self._to(get(p + n["norm"]), "compute", dtype, device)
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)

    def forward(self, x, ctx, cache, state):
        k = kernels.backend()
        t = x.shape[0]
        qk = self.qk_width
        proj = k.product(x, self.w_in, unrounded=True)                    # [q | f | v]
        gate = k.bounded_gate(proj, qk, qk, self.f_bias, self.lower)     # float32 [T, heads * key size]
        o = k.decayed_state_scan(proj, x.dtype, 0, 0, 2 * qk, 1.0, gate, state.data, state.slots, state.fresh_device,
                                 ctx.q_start, ctx.q_len, self.n_heads, self.key_dim, self.value_dim, q_silu=True,
                                 tied_keys=True)
        normed = torch.empty((t, self.v_width), dtype=x.dtype, device=x.device)
        k.head_norm_gate(o, self.norm_weight, self.eps, None, 0, normed, self.n_heads, self.value_dim)
        return k.product(normed, self.w_o, unrounded=True)


register_part("mixer", "bounded_gate_recurrence", BoundedGateRecurrence)
