"""Mixers that are one of several branches of a layer, and the mixer that joins two of them.

`DistanceBiasAttention`: grouped-query softmax attention without rotation.  Positions enter in two ways only: a
factor on the queries that grows with the logarithm of the position, and a learned bias per head that depends on the
distance between query and key through a table of buckets (one row per distance up close, rows that widen with the
logarithm of the distance further out, the last row from `bias_far` on).  Queries and keys are RMS-normed over the
whole projection (all heads at once), the projections have biases, and the concatenated heads are multiplied by
sigmoid(W_g x) before the output projection.

`GatedLinearAttention`: a matrix state S [key size, value size] per head and request,
S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, whose decay a_t = sigmoid(W_2 W_1 x + b)^(1/tau) is per key
channel; a head's output is RMS-normed with a weight that the heads share and multiplied by silu(W_g x).  The state is
float32, one record per request (`state_need`), and a step walks its tokens in order, so a prompt may be cut anywhere.

`SideBySide`: two mixers that read the same input; each output is RMS-normed over the model width with a weight of
its own, and the result is `factor` times their sum; or, without norms, the result is the sum of the two outputs with
a constant factor each.  A branch hands over its output product unrounded (float32 partial sums) with the bias that
the product still lacks, and the join adds, norms and sums in float32.
"""
from __future__ import annotations

import math

import torch

from .. import kernels
from .base import CacheNeed, Mixer, StateNeed, make_part, register_part
from .spec import ParamSpec, PartSpec


def distance_bucket(n: int, rows: int, far: int) -> int:
    """The table row of distance n >= 0: n itself below rows // 2; from there on rows that widen with the logarithm
    of the distance, the last row (rows - 1) at distance `far` and beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def distance_bias_table(rel: torch.Tensor, far: int) -> torch.Tensor:
    """rel [rows, heads] -> float32 [heads, far + 1]: the bias of every head at the distances 0..far (every larger
    distance has the bias of `far`)."""
    rows = rel.shape[0]
    if rows < 2 or far <= rows // 2:
        raise ValueError(f"a distance bias of {rows} rows needs bias_far ({far}) beyond {rows // 2} and at least 2 rows")
    index = torch.tensor([distance_bucket(n, rows, far) for n in range(far + 1)], dtype=torch.long)
    return rel.to(torch.float32)[index].t().contiguous()


class _Branch(Mixer):
    """A mixer that can hand over its output before the output bias: `branch` returns (product, bias or None)."""

    def branch(self, x, ctx, cache, state):
        raise NotImplementedError

    def forward(self, x, ctx, cache, state=None):
        out, bias = self.branch(x, ctx, cache, state)
        if bias is None:
            return out
        # alone in a layer: the bias joins the product here, in float32, as one more partial sum
        total = out.sum(0, dtype=torch.float32) if out.dim() == 3 else out.float()
        return (total + bias.float())[None]


class DistanceBiasAttention(_Branch):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int,
                 scale: float, eps: float, bias_far: int, bias_rows: int = 32, query_growth: tuple | None = None,
                 names: dict | None = None):
        """bias_far: the distance from which the bias table's last row applies; bias_rows: the table's rows (a stored
        table decides; this many are drawn for random weights); query_growth (coef, every): queries at position p
        are multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).  names: tensor names behind `prefix`."""
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads ({n_heads}) must be a multiple of n_kv_heads ({n_kv_heads})")
        widest = kernels.KernelBackend.max_window_attention_dim
        if not (0 < int(key_dim) <= widest and 0 < int(value_dim) <= widest):
            raise ValueError(f"key size {key_dim} / value size {value_dim} is not supported by the attention kernel (1 to {widest})")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.n_kv_heads = int(n_heads), int(n_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.eps = float(scale), float(eps)
        self.bias_far, self.bias_rows = int(bias_far), int(bias_rows)
        self.coef, self.every = (float(query_growth[0]), int(query_growth[1])) if query_growth else (0.0, 0)
        if query_growth and self.every < 1:
            raise ValueError(f"query_growth: 'every' ({self.every}) must be at least 1")
        self.names = dict(q="q", k="k", v="v", g="g", o="o", q_bias="q.b", k_bias="k.b", v_bias="v.b", o_bias="o.b",
                          q_norm="q.norm", k_norm="k.norm", rel="rel")
        self.names.update(names or {})
        self.q_width, self.k_width = self.n_heads * self.key_dim, self.n_kv_heads * self.key_dim
        self.v_width, self.out_width = self.n_kv_heads * self.value_dim, self.n_heads * self.value_dim
        self.w_in = self.b_in = self.w_o = self.b_o = self.q_weight = self.k_weight = self.dist_bias = None

    def cache_need(self):
        return CacheNeed.keys_and_values(self.n_kv_heads, self.key_dim, None, self.value_dim)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        return [
            ParamSpec(p + n["q"], (self.q_width, h)), ParamSpec(p + n["q_bias"], (self.q_width,), role="bias"),
            ParamSpec(p + n["k"], (self.k_width, h)), ParamSpec(p + n["k_bias"], (self.k_width,), role="bias"),
            ParamSpec(p + n["v"], (self.v_width, h)), ParamSpec(p + n["v_bias"], (self.v_width,), role="bias"),
            ParamSpec(p + n["q_norm"], (self.q_width,), role="norm_scale"),
            ParamSpec(p + n["k_norm"], (self.k_width,), role="norm_scale"),
            ParamSpec(p + n["rel"], (self.bias_rows, self.n_heads), role="bias", dtype="float32", free_axes=(0,)),
            ParamSpec(p + n["g"], (self.out_width, h)),
            ParamSpec(p + n["o"], (h, self.out_width)), ParamSpec(p + n["o_bias"], (h,), role="bias"),
        ]

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        w = torch.cat([get(p + n[x]).to(dtype) for x in ("q", "k", "v", "g")], dim=0)      # one product for all that reads x
        self.w_in = w.to(device).contiguous()
        self.b_in = torch.cat([get(p + n[x]).to(dtype) for x in ("q_bias", "k_bias", "v_bias")]).to(device).contiguous()
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)
        self.b_o = self._to(get(p + n["o_bias"]), "compute", dtype, device)
        self.q_weight = self._to(get(p + n["q_norm"]), "compute", dtype, device)
        self.k_weight = self._to(get(p + n["k_norm"]), "compute", dtype, device)
        self.dist_bias = distance_bias_table(get(p + n["rel"]), self.bias_far).to(device)

    def branch(self, x, ctx, cache, state=None):
        k = kernels.backend()
        t = x.shape[0]
        proj = k.product(x, self.w_in, unrounded=True)
        q = torch.empty((t, self.q_width), dtype=x.dtype, device=x.device)
        k.whole_norm_store(proj, self.b_in, q, self.q_weight, self.k_weight, self.eps, ctx.positions, self.coef, self.every,
                           cache.slots if cache.writes else None, cache.k, cache.v, self.n_heads, self.n_kv_heads,
                           self.key_dim, self.value_dim, cache.page_size)
        attn = torch.empty((t, self.out_width), dtype=x.dtype, device=x.device)
        k.window_attention(q, attn, cache.k, cache.v, cache.block_table, ctx.q_start, ctx.q_len, ctx.kv_len, self.n_heads,
                           self.n_kv_heads, self.key_dim, self.value_dim, cache.page_size, self.scale, 0, 0, None,
                           ctx.max_q_len, ctx.max_kv_len, dist_bias=self.dist_bias)
        gated = torch.empty_like(attn)
        k.sigmoid_gate(attn, 0, proj, self.q_width + self.k_width + self.v_width, gated)
        return k.product(gated, self.w_o, unrounded=True), self.b_o


class GatedLinearAttention(_Branch):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, tau: float, eps: float,
                 decay_rank: int = 16, names: dict | None = None):
        """tau: the decay is sigmoid(z)^(1 / tau); decay_rank: the inner width of the decay's two projections (stored
        tensors decide; this is what random weights draw).  names: tensor names behind `prefix`."""
        if not float(tau) > 0:
            raise ValueError(f"tau ({tau}) must be positive")
        if not (0 < int(key_dim) <= 4096 and 0 < int(value_dim) <= 4096):
            raise ValueError(f"key size {key_dim} / value size {value_dim} is not supported by the state scan (1 to 4096)")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.key_dim, self.value_dim = int(n_heads), int(key_dim), int(value_dim)
        self.tau, self.eps, self.decay_rank = float(tau), float(eps), int(decay_rank)
        self.names = dict(q="q", k="k", v="v", g="g", o="o", norm="norm", decay_in="a1", decay_out="a2", decay_bias="a2.b")
        self.names.update(names or {})
        self.qk_width, self.v_width = self.n_heads * self.key_dim, self.n_heads * self.value_dim
        self.w_in = self.w_o = self.w_decay = self.b_decay = self.norm_weight = None

    def state_need(self):
        return StateNeed((self.n_heads, self.key_dim, self.value_dim), torch.float32)

    def param_specs(self):
        p, h, n, r = self.prefix, self.hidden_size, self.names, self.decay_rank
        return [
            ParamSpec(p + n["q"], (self.qk_width, h)), ParamSpec(p + n["k"], (self.qk_width, h)),
            ParamSpec(p + n["v"], (self.v_width, h)), ParamSpec(p + n["g"], (self.v_width, h)),
            ParamSpec(p + n["o"], (h, self.v_width)),
            ParamSpec(p + n["norm"], (self.value_dim,), role="norm_scale"),
            ParamSpec(p + n["decay_in"], (r, h), free_axes=(0,)),
            ParamSpec(p + n["decay_out"], (self.qk_width, r), free_axes=(1,)),
            ParamSpec(p + n["decay_bias"], (self.qk_width,), role="bias"),
        ]

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        low, high = get(p + n["decay_in"]), get(p + n["decay_out"])
        if low.shape[0] != high.shape[1]:
            raise ValueError(f"{p + n['decay_in']} has {low.shape[0]} rows, {p + n['decay_out']} {high.shape[1]} columns: "
                             "the two projections of the decay must share their inner width")
        self.decay_rank = int(low.shape[0])
        w = torch.cat([get(p + n[x]).to(dtype) for x in ("q", "k", "v", "g")] + [low.to(dtype)], dim=0)
        self.w_in = w.to(device).contiguous()
        self.w_decay = self._to(high, "compute", dtype, device)
        self.b_decay = self._to(get(p + n["decay_bias"]), "compute", dtype, device)
        self.norm_weight = self._to(get(p + n["norm"]), "compute", dtype, device)
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)

    def branch(self, x, ctx, cache, state):
        k = kernels.backend()
        t = x.shape[0]
        qk, vw = self.qk_width, self.v_width
        proj = k.product(x, self.w_in, unrounded=True)             # [q | k | v | g | low-rank decay input]
        decay = k.channel_decay(proj, 2 * qk + 2 * vw, self.decay_rank, self.w_decay, self.b_decay, self.tau)
        o = k.decayed_state_scan(proj, x.dtype, 0, qk, 2 * qk, self.key_dim ** -0.5, decay, state.data, state.slots,
                                 state.fresh_device, ctx.q_start, ctx.q_len, self.n_heads, self.key_dim, self.value_dim)
        gated = torch.empty((t, vw), dtype=x.dtype, device=x.device)
        k.head_norm_gate(o, self.norm_weight, self.eps, proj, 2 * qk + vw, gated, self.n_heads, self.value_dim)
        return k.product(gated, self.w_o, unrounded=True), None


class SideBySide(Mixer):
    def __init__(self, prefix: str, hidden_size: int, left: PartSpec, right: PartSpec, eps: float, factor: float = 0.5,
                 names: dict | None = None, join: str = "normed_mean", factors: tuple | None = None, deferred: bool = False):
        """left, right: the two branches (mixers that offer `branch`).  join 'normed_mean': each output is RMS-normed
        over the width with a weight of its own (names: those weights behind `prefix`) and the result is `factor` times
        their sum; join 'weighted_sum': the result is factors[0] * left + factors[1] * right, no norms, no weights;
        with `deferred` it is handed on as a `kernels.ProductSum` for an arrangement whose next kernel adds it up (the
        sandwich arrangement's norm behind the mixer)."""
        if join not in ("normed_mean", "weighted_sum"):
            raise ValueError(f"unknown join '{join}' of two mixers side by side (normed_mean, weighted_sum)")
        if join == "weighted_sum" and (factors is None or len(factors) != 2):
            raise ValueError("the join 'weighted_sum' takes factors=(left, right)")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.eps, self.factor, self.join = float(eps), float(factor), join
        self.factors = (float(factors[0]), float(factors[1])) if join == "weighted_sum" else None
        self.deferred = bool(deferred) and join == "weighted_sum"
        self.branches = [make_part("mixer", left, hidden_size=hidden_size), make_part("mixer", right, hidden_size=hidden_size)]
        for b in self.branches:
            if not hasattr(b, "branch"):
                raise ValueError(f"{type(b).__name__} cannot be a branch of a side-by-side mixer")
        if sum(b.cache_need() is not None for b in self.branches) > 1 or sum(b.state_need() is not None for b in self.branches) > 1:
            raise ValueError("a side-by-side mixer takes at most one branch with a paged cache and one with a state")
        self.names = dict(left_out="left.out", right_out="right.out")
        self.names.update(names or {})
        self.graph_safe = all(b.graph_safe for b in self.branches)
        self.out_weights = None

    def cache_need(self):
        return next((b.cache_need() for b in self.branches if b.cache_need() is not None), None)

    def state_need(self):
        return next((b.state_need() for b in self.branches if b.state_need() is not None), None)

    def param_specs(self):
        h = self.hidden_size
        specs = [s for b in self.branches for s in b.param_specs()]
        if self.join == "weighted_sum":
            return specs
        return specs + [ParamSpec(self.prefix + self.names["left_out"], (h,), role="norm_scale"),
                        ParamSpec(self.prefix + self.names["right_out"], (h,), role="norm_scale")]

    def load(self, get, dtype, device):
        for b in self.branches:
            b.load(get, dtype, device)
        if self.join == "normed_mean":
            self.out_weights = [self._to(get(self.prefix + self.names[x]), "compute", dtype, device) for x in ("left_out", "right_out")]

    def forward(self, x, ctx, cache, state=None):
        outs = [b.branch(x, ctx, cache if b.cache_need() is not None else None, state if b.state_need() is not None else None)
                for b in self.branches]
        (a, bias_a), (b, bias_b) = outs
        if self.deferred and bias_a is None and bias_b is None:
            return kernels.ProductSum(a, self.factors[0], b, self.factors[1])
        if self.join == "weighted_sum":
            return kernels.backend().normed_pair_mean(a, b, bias_a, bias_b, None, None, self.eps, self.factors[0],
                                                      factor_b=self.factors[1], act_dtype=x.dtype)
        return kernels.backend().normed_pair_mean(a, b, bias_a, bias_b, self.out_weights[0], self.out_weights[1], self.eps,
                                                  self.factor)


register_part("mixer", "distance_bias_attention", DistanceBiasAttention)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "side_by_side", SideBySide)
