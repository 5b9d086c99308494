"""A mixture of experts as a layer's feed-forward.

Every token goes to the `top` experts with the largest router logits z = W_r x + b (float32), weighted by the softmax
over those logits alone; an expert is W_down (silu(W_gate x) * (W_up x)) without biases.  With `routing='softmax_all'`
the scores are s = softmax(z) over all experts, the `top` experts with the largest s + correction (a stored number per
expert that only steers the choice) are chosen, and they weigh s over the sum of the chosen scores, times
`weight_scale`.  With `expert='relu2'` an expert has no gate product: W_down relu(W_up x)^2.  An optional shared
feed-forward runs for every token and is added.  Routing, grouping of the rows by expert and the experts' products
all happen on the device, so a step with experts is launched like any other and replays from a graph.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import FeedForward, make_part, register_part
from .spec import ParamSpec, PartSpec


class ExpertMixture(FeedForward):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_experts: int, top: int, intermediate_size: int,
                 shared: PartSpec | None = None, router_bias: bool = True, names: dict | None = None,
                 routing: str = "softmax_top", weight_scale: float = 1.0, expert: str = "swiglu"):
        """names: `expert` (the prefix of expert i's tensors, with {i}), `gate`, `up`, `down`, `router`, `router_bias`,
        `correction` behind `prefix`.  shared: a feed-forward part that every token runs through as well.  routing:
        'softmax_top' or 'softmax_all' (with the tensor `correction`, float [experts]); expert: 'swiglu' or 'relu2'."""
        if routing not in ("softmax_top", "softmax_all"):
            raise ValueError(f"routing '{routing}' is not supported (softmax_top, softmax_all)")
        if expert not in ("swiglu", "relu2"):
            raise ValueError(f"expert '{expert}' is not supported (swiglu, relu2)")
        self.routing, self.weight_scale, self.expert = routing, float(weight_scale), expert
        if not 0 < int(top) <= int(n_experts):
            raise ValueError(f"top ({top}) must be between 1 and the number of experts ({n_experts})")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_experts, self.top, self.intermediate_size = int(n_experts), int(top), int(intermediate_size)
        self.has_router_bias = bool(router_bias)
        self.names = dict(expert="e{i}.", gate="gate", up="up", down="down", router="router", router_bias="router.b",
                          correction="correction")
        self.correction = None
        self.names.update(names or {})
        self.shared = make_part("feed_forward", shared, hidden_size=hidden_size) if shared is not None else None
        if self.shared is not None and not self.shared.graph_safe:
            self.graph_safe = False
        self.w_router = self.b_router = self.w_gate_up = self.w_down = None

    def _expert(self, i: int, which: str) -> str:
        return self.prefix + self.names["expert"].format(i=i) + self.names[which]

    def param_specs(self):
        h, f = self.hidden_size, self.intermediate_size
        specs = []
        for i in range(self.n_experts):
            if self.expert == "swiglu":
                specs.append(ParamSpec(self._expert(i, "gate"), (f, h)))
            specs += [ParamSpec(self._expert(i, "up"), (f, h)), ParamSpec(self._expert(i, "down"), (h, f))]
        specs.append(ParamSpec(self.prefix + self.names["router"], (self.n_experts, h)))
        if self.routing == "softmax_all":
            specs.append(ParamSpec(self.prefix + self.names["correction"], (self.n_experts,), role="bias", dtype="float32"))
        if self.has_router_bias:
            specs.append(ParamSpec(self.prefix + self.names["router_bias"], (self.n_experts,), role="bias"))
        if self.shared is not None:
            specs += self.shared.param_specs()
        return specs

    def load(self, get, dtype, device):
        e, h, f = self.n_experts, self.hidden_size, self.intermediate_size
        gated = self.expert == "swiglu"
        # an expert's gate rows, then its up rows; without a gate its up rows alone
        self.w_gate_up = torch.empty((e, 2 * f if gated else f, h), dtype=dtype, device=device)
        self.w_down = torch.empty((e, h, f), dtype=dtype, device=device)
        for i in range(e):
            if gated:
                self.w_gate_up[i, :f].copy_(get(self._expert(i, "gate")).to(dtype))
            self.w_gate_up[i, f if gated else 0 :].copy_(get(self._expert(i, "up")).to(dtype))
            self.w_down[i].copy_(get(self._expert(i, "down")).to(dtype))
        if self.routing == "softmax_all":
            self.correction = get(self.prefix + self.names["correction"]).to(torch.float32).to(device).contiguous()
        self.w_router = self._to(get(self.prefix + self.names["router"]), "compute", dtype, device)
        if self.has_router_bias:
            self.b_router = self._to(get(self.prefix + self.names["router_bias"]), "compute", dtype, device)
        if self.shared is not None:
            self.shared.load(get, dtype, device)

    def forward(self, x, ctx=None):
        if self.routing == "softmax_top" and self.expert == "swiglu":
            out = kernels.backend().expert_mixture(x, self.w_router, self.b_router, self.w_gate_up, self.w_down, self.top)[None]
        else:
            out = kernels.backend().expert_mixture(x, self.w_router, self.b_router, self.w_gate_up, self.w_down, self.top,
                                                   gated=self.expert == "swiglu", score_all=self.routing == "softmax_all",
                                                   correction=self.correction, weight_scale=self.weight_scale)[None]
        if self.shared is None:
            return out
        s = self.shared.forward(x, ctx)
        if s.dim() != 3:
            s = s.float()[None]
        return torch.cat([out, s], dim=0)          # float32 partial sums: whoever adds to the stream adds them up


register_part("feed_forward", "expert_mixture", ExpertMixture)
