"""Attention mixers that treat single heads before the scores: norms per head, a window that keeps the first tokens,
latent keys and values, a sink in the softmax, an output gate.

Both mixers here run the same three steps through the backend: one product for everything that reads the mixer's
input, a preparation kernel that norms, rotates and stores into the cache pages, and `window_attention`, the
attention kernel with separate key and value sizes, window, kept first tokens and sink.

`NormedAttention`: grouped-query attention whose queries and keys are RMS-normed per head with a weight that the
heads share, whose values are divided by their root mean square before they are cached, and whose window keeps the
request's first tokens visible: position i sees j <= i if i - j < window or j < keep_first.

`LatentAttention`: every token leaves one latent vector c (RMS-normed, `latent_dim` wide) and one rotated key part
that all heads share; a head's unrotated key is W_uk c and its value W_uv c.  Only c and the rotated part are cached.
The scores are computed in the latent space: (q_plain . W_uk c) = ((W_uk^T q_plain) . c), so the query's unrotated
part is carried into the latent space once per token and head, the cache is read as one key/value head with keys
[c | rotated part] and values c, and the heads' outputs are carried back with W_uv afterwards.  The softmax's
denominator holds exp(sink_h) beside the keys' terms; the heads' outputs are multiplied by sigmoid(W_g x).
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import CacheNeed, Mixer, PagedTensor, PendingNorm, make_part, register_part
from .spec import ParamSpec, PartSpec


def _window(window) -> int | None:
    return int(window) if window else None


class _Projected:
    """What a mixer's first phase leaves for its second: the input product, the factor its rows may still lack (a norm
    that was folded into the product), and the stream that the output product may add itself into."""

    __slots__ = ("proj", "factor", "residual", "t", "dtype", "device")

    def __init__(self, proj, factor, residual, t, dtype, device):
        self.proj, self.factor, self.residual, self.t, self.dtype, self.device = proj, factor, residual, t, dtype, device


def _input_product(x, w, hidden_size) -> _Projected:
    """x w^T for a mixer's input: from a tensor, or from a pending norm, which is folded into the product where the
    backend has that kernel (the rows' 1/rms factor then goes on to the preparation kernel)."""
    k = kernels.backend()
    if isinstance(x, PendingNorm):
        rms = x.rms()
        fused = k.product_normed(x.h, x.delta, rms[0], w) if rms is not None else None
        if fused is not None:
            proj, row_ss, h_new = fused
            x.applied(h_new)
            return _Projected(proj, dict(row_ss=row_ss, hidden=hidden_size, norm_eps=rms[1]), x.residual(), h_new.shape[0],
                              w.dtype, h_new.device)
        pending, x = x, x.materialize()
        return _Projected(k.product(x, w, unrounded=True), {}, pending.residual(), x.shape[0], x.dtype, x.device)
    return _Projected(k.product(x, w, unrounded=True), {}, None, x.shape[0], x.dtype, x.device)


def _output_product(heads_out, w, residual):
    out = kernels.backend().product(heads_out, w, unrounded=True, residual=residual)
    return None if out is residual and residual is not None else out


class _TwoPhases(Mixer):
    """forward = finish(project(x)): `project` is all that reads the mixer's input (and, through a pending norm, the
    residual stream); `finish` is the rest, and may add the output into the stream."""

    takes_pending_norm = True

    def forward(self, x, ctx, cache, state=None):
        return self.finish(self.project(x, ctx), ctx, cache, state)


class NormedAttention(_TwoPhases):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int,
                 scale: float, eps: float, window: int | None = None, keep_first: int = 0, norm_queries_keys: bool = True,
                 norm_values: bool = False, norm_weighted: bool = True, norm_after_rotation: bool = False,
                 position: PartSpec | None = None, values_are_keys: bool = False, sink: bool = False, gated: bool = False,
                 names: dict | None = None):
        """norm_weighted False: queries and keys are divided by their root mean square and no more (no weight tensors);
        position: a rotary encoding of queries and keys (None: no rotation), applied behind the norm, or before it
        with norm_after_rotation; values_are_keys: there is no value projection, a value head is its key head as
        projected (before norm and rotation); sink: one number per head joins the softmax's denominator; gated: the
        heads' outputs are multiplied by sigmoid(W_g x).  names: tensor names behind `prefix` of q, k, v, o, the
        weights q_norm, k_norm, and sink, gate."""
        if n_heads % n_kv_heads:
            raise ValueError(f"n_heads ({n_heads}) must be a multiple of n_kv_heads ({n_kv_heads})")
        widest = kernels.KernelBackend.max_window_attention_dim
        if not (0 < int(key_dim) <= widest and 0 < int(value_dim) <= widest):
            raise ValueError(f"key size {key_dim} / value size {value_dim} is not supported by the attention kernel (1 to {widest})")
        if values_are_keys and int(value_dim) != int(key_dim):
            raise ValueError(f"values that are the keys have the keys' size: value_dim ({value_dim}) must be {key_dim}")
        if values_are_keys and norm_values:
            raise ValueError("values that are the keys as projected are not normed")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads, self.n_kv_heads = int(n_heads), int(n_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.eps = float(scale), float(eps)
        self.window = _window(window)
        self.keep_first = int(keep_first) if self.window else 0
        self.norm_queries_keys, self.norm_values = bool(norm_queries_keys), bool(norm_values)
        self.norm_weighted, self.norm_after_rotation = bool(norm_weighted), bool(norm_after_rotation)
        self.values_are_keys, self.has_sink, self.gated = bool(values_are_keys), bool(sink), bool(gated)
        self.position = None if position is None else make_part("position_encoding", position, head_dim=self.key_dim)
        self.names = dict(q="q_proj.weight", k="k_proj.weight", v="v_proj.weight", o="o_proj.weight",
                          q_norm="q_norm.weight", k_norm="k_norm.weight", sink="sink", gate="g_proj.weight")
        self.names.update(names or {})
        self.q_width, self.k_width = self.n_heads * self.key_dim, self.n_kv_heads * self.key_dim
        self.v_width = 0 if self.values_are_keys else self.n_kv_heads * self.value_dim
        self.out_width = self.n_heads * self.value_dim
        self.w_qkv = self.w_o = self.q_weight = self.k_weight = self.sink = None

    def cache_need(self):
        return CacheNeed.keys_and_values(self.n_kv_heads, self.key_dim, self.window, self.value_dim, self.keep_first)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        specs = [ParamSpec(p + n["q"], (self.q_width, h)), ParamSpec(p + n["k"], (self.k_width, h))]
        if not self.values_are_keys:
            specs.append(ParamSpec(p + n["v"], (self.v_width, h)))
        specs.append(ParamSpec(p + n["o"], (h, self.out_width)))
        if self.norm_queries_keys and self.norm_weighted:
            specs += [ParamSpec(p + n["q_norm"], (self.key_dim,), role="norm_scale"),
                      ParamSpec(p + n["k_norm"], (self.key_dim,), role="norm_scale")]
        if self.has_sink:
            specs.append(ParamSpec(p + n["sink"], (self.n_heads,), role="bias", dtype="float32"))
        if self.gated:
            specs.append(ParamSpec(p + n["gate"], (self.out_width, h)))
        if self.position is not None:
            specs += self.position.param_specs()
        return specs

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        which = ["q", "k"] + ([] if self.values_are_keys else ["v"]) + (["gate"] if self.gated else [])
        w = torch.cat([get(p + n[x]).to(dtype) for x in which], dim=0)      # one product serves all that reads x
        self.w_qkv = w.to(device).contiguous()
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)
        if self.norm_queries_keys and self.norm_weighted:
            self.q_weight = self._to(get(p + n["q_norm"]), "compute", dtype, device)
            self.k_weight = self._to(get(p + n["k_norm"]), "compute", dtype, device)
        if self.has_sink:
            self.sink = get(p + n["sink"]).to(torch.float32).to(device).contiguous()
        if self.position is not None:
            self.position.load(get, dtype, device)

    def project(self, x, ctx):
        return _input_product(x, self.w_qkv, self.hidden_size)

    def finish(self, p, ctx, cache, state=None):
        return _output_product(self._heads_out(p, ctx, cache), self.w_o, p.residual)

    def branch(self, x, ctx, cache, state=None):
        """Beside another mixer in one layer: the output product unrounded, no bias."""
        p = self.project(x, ctx)
        return kernels.backend().product(self._heads_out(p, ctx, cache), self.w_o, unrounded=True), None

    def _heads_out(self, p, ctx, cache):
        k = kernels.backend()
        t = p.t
        q = torch.empty((t, self.q_width), dtype=p.dtype, device=p.device)
        rotation = {}
        rotary = self.position.rotary(p.device) if self.position is not None else None
        if rotary is not None:
            rotation = dict(cos_sin=self.position.table(ctx), rotary_dim=rotary[1], pairing=self.position.pairing,
                            magnitude=getattr(self.position, "magnitude", 1.0))
        plain = self.norm_queries_keys and not self.norm_weighted
        if plain or self.norm_after_rotation or self.values_are_keys or self.gated:
            rotation.update(norm_plain=plain, norm_after_rotation=self.norm_after_rotation,
                            values_are_keys=self.values_are_keys, row_width=self.w_qkv.shape[0])
        k.head_norm_store(p.proj, q, self.q_weight, self.k_weight, self.eps, self.norm_values,
                          cache.slots if cache.writes else None, cache.k, cache.v, self.n_heads, self.n_kv_heads,
                          self.key_dim, self.value_dim, cache.page_size, **p.factor, **rotation)
        attn = torch.empty((t, self.out_width), dtype=p.dtype, device=p.device)
        k.window_attention(q, attn, cache.k, cache.v, cache.block_table, ctx.q_start, ctx.q_len, ctx.kv_len,
                           self.n_heads, self.n_kv_heads, self.key_dim, self.value_dim, cache.page_size, self.scale,
                           self.window or 0, self.keep_first, self.sink, ctx.max_q_len, ctx.max_kv_len)
        if not self.gated:
            return attn
        gated = torch.empty_like(attn)
        k.sigmoid_gate(attn, 0, p.proj, self.q_width + self.k_width + self.v_width, gated, **p.factor)
        return gated


class LatentAttention(_TwoPhases):
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, n_heads: int, plain_dim: int, rotated_dim: int, value_dim: int,
                 latent_dim: int, scale: float, eps: float, position: PartSpec, window: int | None = None,
                 keep_first: int = 0, sink: bool = False, gated: bool = False, query_latent_dim: int | None = None,
                 names: dict | None = None):
        """plain_dim / rotated_dim: a head's unrotated and rotated query/key places (a query head is laid out
        [plain | rotated]); latent_dim: the width of the cached latent.  query_latent_dim r: the queries come through a
        latent of their own, q = W_q rmsnorm(W_q_down x) with W_q [.., r] (None: q = W_q x).  names: tensor names behind
        `prefix` of q, q_down, q_down_norm, down (rows: latent, then the shared rotated key), down_norm, up_k, up_v, sink,
        gate, o."""
        widest = kernels.KernelBackend.max_window_attention_dim
        if not 0 < int(latent_dim) + int(rotated_dim) <= widest:
            raise ValueError(f"latent size {latent_dim} + rotated size {rotated_dim} is not supported by the attention "
                             f"kernel (at most {widest})")
        self.prefix, self.hidden_size = prefix, int(hidden_size)
        self.n_heads = int(n_heads)
        self.plain_dim, self.rotated_dim = int(plain_dim), int(rotated_dim)
        self.value_dim, self.latent_dim = int(value_dim), int(latent_dim)
        self.scale, self.eps = float(scale), float(eps)
        self.window = _window(window)
        self.keep_first = int(keep_first) if self.window else 0
        self.has_sink, self.gated = bool(sink), bool(gated)
        self.position = make_part("position_encoding", position, head_dim=max(self.rotated_dim, 2))
        self.query_latent_dim = int(query_latent_dim) if query_latent_dim else 0
        self.names = dict(q="q", q_down="q_down", q_down_norm="q_down_norm", down="down", down_norm="down_norm", up_k="up_k",
                          up_v="up_v", sink="sink", gate="gate", o="o")
        self.names.update(names or {})
        self.q_width = self.n_heads * (self.plain_dim + self.rotated_dim)
        self.down_width = self.latent_dim + self.rotated_dim
        self.out_width = self.n_heads * self.value_dim
        self.w_in = self.w_up_k = self.w_up_v = self.w_o = self.c_weight = self.sink = self.w_q = self.cq_weight = None
        # the first rows of the input product: the queries, or the latent they are made from
        self.lead_width = self.query_latent_dim or self.q_width

    def cache_need(self):
        # one key/value head: keys [latent | rotated part], values the latent, transposed within a page
        return CacheNeed((PagedTensor("k", (1, self.latent_dim + self.rotated_dim), 1),
                          PagedTensor("v", (1, self.latent_dim), 2)), self.window, self.keep_first)

    def param_specs(self):
        p, h, n = self.prefix, self.hidden_size, self.names
        if self.query_latent_dim:
            lead = [ParamSpec(p + n["q_down"], (self.query_latent_dim, h)),
                    ParamSpec(p + n["q_down_norm"], (self.query_latent_dim,), role="norm_scale"),
                    ParamSpec(p + n["q"], (self.q_width, self.query_latent_dim))]
        else:
            lead = [ParamSpec(p + n["q"], (self.q_width, h))]
        specs = lead + [
            ParamSpec(p + n["down"], (self.down_width, h)),
            ParamSpec(p + n["down_norm"], (self.latent_dim,), role="norm_scale"),
            ParamSpec(p + n["up_k"], (self.n_heads * self.plain_dim, self.latent_dim)),
            ParamSpec(p + n["up_v"], (self.out_width, self.latent_dim)),
            ParamSpec(p + n["o"], (h, self.out_width)),
        ]
        if self.has_sink:
            specs.append(ParamSpec(p + n["sink"], (self.n_heads,), role="bias", dtype="float32"))
        if self.gated:
            specs.append(ParamSpec(p + n["gate"], (self.out_width, h)))
        return specs + self.position.param_specs()

    def load(self, get, dtype, device):
        p, n = self.prefix, self.names
        rows = [get(p + n["q_down" if self.query_latent_dim else "q"]).to(dtype), get(p + n["down"]).to(dtype)]
        if self.query_latent_dim:
            self.w_q = self._to(get(p + n["q"]), "compute", dtype, device)
            self.cq_weight = self._to(get(p + n["q_down_norm"]), "compute", dtype, device)
        if self.gated:
            rows.append(get(p + n["gate"]).to(dtype))
        self.w_in = torch.cat(rows, dim=0).to(device).contiguous()          # one product for all that reads x
        self.w_up_k = self._to(get(p + n["up_k"]), "compute", dtype, device).view(self.n_heads, self.plain_dim, self.latent_dim)
        w_up_v = self._to(get(p + n["up_v"]), "compute", dtype, device).view(self.n_heads, self.value_dim, self.latent_dim)
        self.w_up_v = w_up_v.transpose(1, 2).contiguous()                    # [heads, latent, value]
        self.w_o = self._to(get(p + n["o"]), "compute", dtype, device)
        self.c_weight = self._to(get(p + n["down_norm"]), "compute", dtype, device)
        if self.has_sink:
            self.sink = get(p + n["sink"]).to(torch.float32).to(device).contiguous()
        self.position.load(get, dtype, device)

    def project(self, x, ctx):
        if self.query_latent_dim and isinstance(x, PendingNorm):
            # (the queries' latent is normed from the complete product: the input norm is not folded into it)
            pending, x = x, x.materialize()
            p = _input_product(x, self.w_in, self.hidden_size)
            p.residual = pending.residual()
            return p
        return _input_product(x, self.w_in, self.hidden_size)

    def finish(self, p, ctx, cache, state=None):
        k = kernels.backend()
        t, nh, rank, rot = p.t, self.n_heads, self.latent_dim, self.rotated_dim
        q_plain = torch.empty((t, nh, self.plain_dim), dtype=p.dtype, device=p.device)
        q_full = torch.empty((t, nh, rank + rot), dtype=p.dtype, device=p.device)
        rotary = self.position.rotary(p.device)
        cos_sin = self.position.table(ctx) if rotary is not None else None
        queries = {}
        if self.query_latent_dim:
            # the queries' latent, normed (one "head" as wide as the latent), then the queries themselves
            c_q = torch.empty((t, self.query_latent_dim), dtype=p.dtype, device=p.device)
            k.head_norm_gate(p.proj, self.cq_weight, self.eps, None, 0, c_q, 1, self.query_latent_dim,
                             x_width=self.w_in.shape[0], x_act=p.dtype)
            queries = dict(queries=k.product(c_q, self.w_q, unrounded=True), lead_width=self.lead_width)
        k.latent_prep(p.proj, q_plain, q_full, self.c_weight, self.eps, cos_sin, getattr(self.position, "magnitude", 1.0),
                      rotary[1] if rotary is not None else 0, cache.slots if cache.writes else None, cache.k, cache.v,
                      nh, self.plain_dim, rot, rank, cache.page_size, **p.factor, **queries)
        # the queries' unrotated parts carried into the latent space, head by head, into their places before the
        # rotated parts
        k.heads_product(q_plain.transpose(0, 1), self.w_up_k, out=q_full[:, :, :rank].transpose(0, 1))
        o_latent = torch.empty((t, nh * rank), dtype=p.dtype, device=p.device)
        k.window_attention(q_full.view(t, nh * (rank + rot)), o_latent, cache.k, cache.v, cache.block_table, ctx.q_start,
                           ctx.q_len, ctx.kv_len, nh, 1, rank + rot, rank, cache.page_size, self.scale, self.window or 0,
                           self.keep_first, self.sink, ctx.max_q_len, ctx.max_kv_len)
        # and the heads' outputs carried back: [heads, T, value]
        o = k.heads_product(o_latent.view(t, nh, rank).transpose(0, 1), self.w_up_v)
        if self.gated:
            heads_out = torch.empty((t, self.out_width), dtype=p.dtype, device=p.device)
            k.sigmoid_gate(o, nh, p.proj, self.lead_width + self.down_width, heads_out, **p.factor)
        else:
            heads_out = o.transpose(0, 1).reshape(t, self.out_width)
        return _output_product(heads_out, self.w_o, p.residual)


register_part("mixer", "normed_attention", NormedAttention)
register_part("mixer", "latent_attention", LatentAttention)
