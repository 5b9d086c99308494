"""Dense gated feed-forward (SwiGLU).

As the reference computes it (/root/reference/src/models/mlp.cpp:41-49, CUDA form
/root/reference/src/cuda/ops/mlp.cu:152-162): u = x Wup^T, g = x Wgate^T,
y = (u * g / (1 + exp(-g))) Wdown^T; the gate is the activated branch; no biases.
The reference infers the inner width from the tensors
(/root/reference/src/models/model_param_validation.cpp:167-194); here it is a parameter.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import FeedForward, PendingNorm, register_part
from .spec import ParamSpec


class SwiGLU(FeedForward):
    graph_safe = True
    takes_pending_norm = True

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 names: tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight"),
                 unrounded: bool = False):
        """names: the tensors of the gate, up and down matrices behind `prefix`.  unrounded: the output is always
        float32 partial sums (for an arrangement that adds it to another branch's before anything is rounded)."""
        if activation != "silu":
            raise ValueError(f"activation '{activation}' is not supported by the swiglu feed-forward")
        self.prefix = prefix
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = tuple(names)
        self.unrounded = bool(unrounded)
        self.w_gate_up = self.w_down = None

    def param_specs(self):
        p, h, i = self.prefix, self.hidden_size, self.intermediate_size
        gate, up, down = self.names
        return [ParamSpec(p + gate, (i, h)), ParamSpec(p + up, (i, h)), ParamSpec(p + down, (h, i))]

    def load(self, get, dtype, device):
        p = self.prefix
        gate, up, down = self.names
        w = torch.cat([get(p + gate).to(dtype), get(p + up).to(dtype)], dim=0)
        self.w_gate_up = w.to(device).contiguous()
        self.w_down = self._to(get(p + down), "compute", dtype, device)

    def forward(self, x, ctx=None):
        k = kernels.backend()
        # With few tokens: the norm folds into the first product's staging of x, and SwiGLU (with the rows'
        # 1/rms factor) into the second's.
        residual = None

        def down(act):
            out = k.product(act, self.w_down, unrounded=self.unrounded, residual=residual)     # else added to the residual stream by the next norm
            return None if out is residual else out

        if isinstance(x, PendingNorm):
            pending = x
            rms = x.rms()
            fused = None
            if rms is not None and self.intermediate_size % 8 == 0:
                fused = k.product_normed(x.h, x.delta, rms[0], self.w_gate_up)
            if fused is not None:
                gate_up, row_ss, h_new = fused
                x.applied(h_new)
                residual = pending.residual()
                out = k.product_swiglu(gate_up, row_ss, self.hidden_size, rms[1], self.w_down, residual=residual)
                if out is not None:
                    return None if out is residual else out
                # SwiGLU by itself; it applies the rows' pending 1/rms factor
                act = torch.empty((h_new.shape[0], self.intermediate_size), dtype=self.w_down.dtype, device=h_new.device)
                k.swiglu(gate_up, act, row_ss=row_ss, hidden=self.hidden_size, eps=rms[1])
                return down(act)
            x = x.materialize()
            residual = pending.residual()
        t = x.shape[0]
        act = k.gate_up_swiglu(x, self.w_gate_up)        # a few dozen tokens: product and activation in one kernel
        if act is not None:
            return down(act)
        gate_up = k.product(x, self.w_gate_up)           # act [T, 2I] or float32 partial sums [S, T, 2I]
        if gate_up.dim() == 3:
            out = k.product_swiglu(gate_up, None, self.hidden_size, 0.0, self.w_down, residual=residual)
            if out is not None:
                return None if out is residual else out
        act = torch.empty((t, self.intermediate_size), dtype=x.dtype, device=x.device)
        k.swiglu(gate_up, act)
        return down(act)


class ActivatedFeedForward(FeedForward):
    """A feed-forward without a gate product: y = W_down act(W_up x), no biases.

    activation 'relu2': the square of relu.  'polynorm': c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 with powers taken element
    by element, N(u) = u / sqrt(mean(u^2) + eps) over a token's inner values, and the four numbers c in the tensor
    `coef`.  row_gate: the name of a [1, H] tensor g; the token's output is multiplied by sigmoid(g . x), one number
    per token (its weights ride as one more row of the up matrix, and since the down product is linear the factor is
    applied to the activated inner values).  The up product stays unrounded (float32) until the activation has used it;
    the statistics and the activation are float32.  The output is float32 partial sums."""

    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "relu2", eps: float = 0.0,
                 names: tuple[str, str] = ("up", "down"), coef: str = "act", row_gate: str | None = None):
        if activation not in ("relu2", "polynorm"):
            raise ValueError(f"activation '{activation}' is not supported by this feed-forward (relu2, polynorm)")
        self.prefix, self.hidden_size, self.intermediate_size = prefix, int(hidden_size), int(intermediate_size)
        self.activation, self.eps = activation, float(eps)
        self.names, self.coef_name, self.row_gate = tuple(names), coef, row_gate
        self.w_up = self.w_down = self.coef = None

    def param_specs(self):
        p, h, i = self.prefix, self.hidden_size, self.intermediate_size
        up, down = self.names
        specs = [ParamSpec(p + up, (i, h)), ParamSpec(p + down, (h, i))]
        if self.activation == "polynorm":
            specs.append(ParamSpec(p + self.coef_name, (4,), role="norm_scale", dtype="float32"))
        if self.row_gate is not None:
            specs.append(ParamSpec(p + self.row_gate, (1, h), alt_shapes=((h,),)))
        return specs

    def load(self, get, dtype, device):
        p = self.prefix
        up, down = self.names
        rows = [get(p + up).to(dtype)]
        if self.row_gate is not None:
            rows.append(get(p + self.row_gate).to(dtype).reshape(1, self.hidden_size))
        self.w_up = torch.cat(rows, dim=0).to(device).contiguous()
        self.w_down = self._to(get(p + down), "compute", dtype, device)
        if self.activation == "polynorm":
            self.coef = get(p + self.coef_name).to(torch.float32).reshape(4).to(device).contiguous()

    def forward(self, x, ctx=None):
        k = kernels.backend()
        i = self.intermediate_size
        z = k.product(x, self.w_up, unrounded=True)
        act = torch.empty((x.shape[0], i), dtype=x.dtype, device=x.device)
        k.ff_activation(z, i, self.activation, act, coef=self.coef, eps=self.eps, gate_col=i if self.row_gate is not None else -1)
        out = k.product(act, self.w_down, unrounded=True)
        return out if out.dim() == 3 else out.float()[None]


register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "activated", ActivatedFeedForward)
