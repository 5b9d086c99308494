"""Grouped-query softmax attention without rotation whose positions enter through the mask and a penalty alone.

Queries and keys are RMS-normed over the whole projection (all heads at once, a weight per value), the score of key j
for a query at position p is (q . k) * scale - slope_h * (p - j) with slope_h = 2^(-span (h + 1) / heads) for head h,
and key j <= p is visible only if it lies in the query's own block of `block` positions, floor(j / block) ==
floor(p / block), counted from position 0 of the request wherever a step cuts it (block None: every j <= p).  Key
and value sizes may differ.  A layer with `shares_cache` has no key and value tensors of its own: it reads the pages
that another entry of the run order wrote (`RunSpec(cache=j, writes_cache=False)`) with its own queries.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import CacheNeed, Mixer, register_part
from .spec import ParamSpec


def head_slopes(n_heads: int, span: float) -> torch.Tensor:
    """float32 [heads]: 2^(-span (h + 1) / heads)."""
    h = torch.arange(1, n_heads + 1, dtype=torch.float64)
    return torch.pow(torch.tensor(2.0, dtype=torch.float64), -float(span) * h / n_heads).to(torch.float32)


class BlockLocalAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int,
                 scale: float, eps: float, block: int | None = None, slope_span: float | None = 8.0,
                 shares_cache: bool = False, names: dict | None = None):
        """block: keys are visible within the query's block of this many positions (None: all earlier keys);
        slope_span: the heads' penalties per token of distance are 2^(-slope_span (h + 1) / heads) (None: no penalty);
        shares_cache: the layer has queries only and reads another entry's keys and values; names: tensor names behind
        `prefix`."""
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads ({n_heads}) must be a multiple of n_kv_heads ({n_kv_heads})")
        widest = kernels.KernelBackend.max_window_attention_dim
        if not (0 < int(key_dim) <= widest and 0 < int(value_dim) <= widest):
            raise ValueError(f"key size {key_dim} / value size {value_dim} is not supported by the attention kernel (1 to {widest})")
        if block is not None and int(block) < 1:
            raise ValueError(f"block ({block}) must be at least 1")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.n_kv_heads = int(n_heads), int(n_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.eps = float(scale), float(eps)
        self.block = int(block) if block is not None else 0
        self.slope_span = None if slope_span is None else float(slope_span)
        self.shares_cache = bool(shares_cache)
        self.names = dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm")
        self.names.update(names or {})
        self.q_width, self.k_width = self.n_heads * self.key_dim, self.n_kv_heads * self.key_dim
        self.v_width, self.out_width = self.n_kv_heads * self.value_dim, self.n_heads * self.value_dim
        self.w_in = self.w_o = self.q_weight = self.k_weight = self.slopes = None

    def cache_need(self):
        return CacheNeed.keys_and_values(self.n_kv_heads, self.key_dim, None, self.value_dim)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        specs = [ParamSpec(p + n["q"], (self.q_width, h)), ParamSpec(p + n["q_norm"], (self.q_width,), role="norm_scale")]
        if not self.shares_cache:
            specs += [ParamSpec(p + n["k"], (self.k_width, h)), ParamSpec(p + n["v"], (self.v_width, h)),
                      ParamSpec(p + n["k_norm"], (self.k_width,), role="norm_scale")]
        return specs + [ParamSpec(p + n["o"], (h, self.out_width))]

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        which = ("q",) if self.shares_cache else ("q", "k", "v")
        self.w_in = torch.cat([get(p + n[x]).to(dtype) for x in which], dim=0).to(device).contiguous()     # one product reads x
        self.q_weight = self._to(get(p + n["q_norm"]), "compute", dtype, device)
        if not self.shares_cache:
            self.k_weight = self._to(get(p + n["k_norm"]), "compute", dtype, device)
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)
        if self.slope_span is not None:
            self.slopes = head_slopes(self.n_heads, self.slope_span).to(device)

    def forward(self, x, ctx, cache, state=None):
        if cache.writes == self.shares_cache:
            raise RuntimeError("a layer that shares another's cache must not write it, and a layer of its own must")
        k = kernels.backend()
        t = x.shape[0]
        proj = k.product(x, self.w_in, unrounded=True)
        q = torch.empty((t, self.q_width), dtype=x.dtype, device=x.device)
        if self.shares_cache:
            k.whole_norm_store(proj, None, q, self.q_weight, None, self.eps, ctx.positions, 0.0, 0, None, cache.k, cache.v,
                               self.n_heads, 0, self.key_dim, self.value_dim, cache.page_size)
        else:
            k.whole_norm_store(proj, None, q, self.q_weight, self.k_weight, self.eps, ctx.positions, 0.0, 0, cache.slots,
                               cache.k, cache.v, self.n_heads, self.n_kv_heads, self.key_dim, self.value_dim, cache.page_size)
        attn = torch.empty((t, self.out_width), dtype=x.dtype, device=x.device)
        k.window_attention(q, attn, cache.k, cache.v, cache.block_table, ctx.q_start, ctx.q_len, ctx.kv_len, self.n_heads,
                           self.n_kv_heads, self.key_dim, self.value_dim, cache.page_size, self.scale, 0, 0, None,
                           ctx.max_q_len, ctx.max_kv_len, block=self.block, slopes=self.slopes)
        return k.product(attn, self.w_o, unrounded=True)


register_part("mixer", "block_local_attention", BlockLocalAttention)
