"""The kernel backend: the one place from which parts reach device code.

`backend()` returns the object whose methods launch the hand-written HIP kernels
(`kernels.hip.HipKernels`).  There is no CPU implementation in the product: if
the compiled extension cannot be loaded on a machine with a GPU, `backend()`
raises.  `use_backend` lets a test put an object with the same methods in its
place (the tests' own slow emulation, to exercise the engine's bookkeeping on a
machine without a GPU).

Methods of a backend (T tokens, B requests, R rows, act = bfloat16 or float32):

  embed(token_ids i32[T], table act[V,H], out f32[T,H])
  add_rmsnorm(h f32[T,H], delta act[T,H]|None, weight act[H], eps, out act[T,H])
        h += delta in float32 (in place), out = h * rsqrt(mean(h^2) + eps) * weight
  rows_add_rmsnorm(h, delta|None, rows i32[R], weight, eps, out act[R,H])
        the same for rows `rows` only, h is not written
  linear(x act[T,K], w act[N,K], bias act[N]|None, out act|f32 [T,N])      out = x w^T + bias
  qkv_rope_store(qkv act[T,(nq+2nkv)*hd], bias|None, positions i32[T], inv_freq f32[rd/2]|None,
                 rotary_dim, slots i32[T]|None, k_cache, v_cache, nq, nkv, hd, page_size)
        adds bias, rotates the first rotary_dim features of every query and key head
        (pairs (i, i + rotary_dim/2), angle = position * inv_freq[i]) in place, and stores
        keys and values at `slots` (page * page_size + offset) of the caches, keys [P,nkv,page_size,hd],
        values [P,nkv,hd,page_size]
  paged_attention(qkv, out act[T,nq*hd], k_cache, v_cache, block_table i32[B,W], q_start i32[B],
                  q_len i32[B], kv_len i32[B], nq, nkv, hd, page_size, scale, window,
                  max_q_len, max_kv_len, combine=True, singles=True)
        query i of request b stands at position p = kv_len[b] - q_len[b] + i and reads keys
        j <= p (and j > p - window if window > 0) of that request through its block table
        (hints: singles=False says that no request brings exactly one token; combine=False lets the
        caller combine the parts of a split key range, which are then returned)
  swiglu(gate_up act[T,2I], out act[T,I])        out = silu(gate_up[:, :I]) * gate_up[:, I:]
  argmax(logits f32[R,V], out i32[R])            lowest index among equal maxima
  sample(logits f32[R,V], temperature f32[R], top_k i32[R], top_p f32[R], uniform f32[R], out i32[R])

  (head_norm_store, latent_prep and sigmoid_gate also take row_ss f32[S2,T], hidden, norm_eps: the product, float32
   partial sums, then still lacks each row's factor 1/sqrt(sum_s row_ss[s] / hidden + norm_eps), as `product_normed`
   leaves it)
  embed_rmsnorm(token_ids i32[T], table act[V,H], weight act[H], eps, out f32[T,H] | fixed point)
        out = table[id] / sqrt(mean(table[id]^2) + eps) * weight: an embedding with its norm, as the residual stream
  head_norm_store(proj act[T,W]|f32[S,T,W], q_out act[T,nq*dk], q_weight act[dk]|None, k_weight act[dk]|None, eps,
                  norm_values, slots i32[T]|None, k_cache, v_cache, nq, nkv, dk, dv, page_size)
        proj rows are [nq heads of dk | nkv heads of dk | nkv heads of dv]; query and key heads are divided by their
        root mean square and multiplied by the weight (None: they pass), value heads are divided by theirs if
        norm_values; queries to q_out, keys [P,nkv,page_size,dk] and values [P,nkv,dv,page_size] to `slots`
  latent_prep(proj, q_plain act[T,nq,dim], q_full act[T,nq,rank+rot], c_weight act[rank], eps, cos_sin f32[T,rd/2,2]|None,
              magnitude, rotary_dim, slots, k_cache, v_cache, nq, dim, rot, rank, page_size)
        proj rows are [nq heads of (dim | rot) | rank | rot | ...]; the heads' unrotated parts to q_plain, their rotated
        parts (pairs (2i, 2i+1) of the first rotary_dim places turned by the table's angles, cos and sin times
        magnitude) to q_full[..., rank:]; the latent, RMS-normed with c_weight, with the rotated shared key behind it
        as key [P,1,page_size,rank+rot], the latent alone as value [P,1,rank,page_size], at `slots`
  heads_product(x act[heads,T,K] (any strides), w act[heads,K,N]) -> act[heads,T,N]    one product per head
  sigmoid_gate(x act[T,N] | act[heads,T,N/heads], heads, gate act[T,W]|f32[S,T,W], gate_offset, out act[T,N])
        out = x * sigmoid(gate[:, gate_offset : gate_offset + N])
  window_attention(q act[T,nq*dk], out act[T,nq*dv], k_cache, v_cache, block_table, q_start, q_len, kv_len, nq, nkv,
                   dk, dv, page_size, scale, window, keep_first, sink f32[nq]|None, max_q_len, max_kv_len)
        as paged_attention with key size dk and value size dv; key j <= p is read if window == 0, p - j < window or
        j < keep_first; with a sink the softmax's denominator also holds exp(sink[head])

  window_attention(..., dist_bias f32[nq, far+1]|None): with a distance bias, key j of a query at position p gets
        dist_bias[head, min(p - j, far)] added to its scaled score (a learned bias by head and distance, tabulated per
        distance up to the one from which it no longer changes)

  embed_scaled(token_ids i32[T], table act[V,H], factor, out f32[T,H])          out = table[id] * factor
  add_layernorm(h f32[T,H], delta act[T,H]|f32[S,T,H]|None, rows i32[R]|None, weight act[H], bias act[H]|None, eps, out)
        h += delta; out = (h - mean) / sqrt(mean((h - mean)^2) + eps) * weight + bias; with rows only those, h untouched
  normed_pair_mean(a, b, bias_a|None, bias_b|None, weight_a, weight_b, eps, factor) -> f32[1,T,H]
        factor * (rmsnorm(a + bias_a) * weight_a + rmsnorm(b + bias_b) * weight_b); a, b products (act or partial sums)
  tanh_cap(x f32[...], cap, scale=1)           x = cap * tanh(scale * x / cap) in place (cap None: scale * x)
  post_norm_add(h f32[T,H], y, post_weight act[H], eps, mult, ...)     h += mult * LN(y) * post_weight, LN without bias; y a product
        (act [T, H] or float32 partial sums) or a ProductSum of two
  whole_norm_store(proj, bias act[W]|None, q_out act[T,nq*dk], q_weight act[nq*dk]|None, k_weight act[nkv*dk]|None, eps,
                   positions i32[T], coef, every, slots, k_cache, v_cache, nq, nkv, dk, dv, page_size)
        proj rows are [nq heads of dk | nkv heads of dk | nkv heads of dv | ...]; the bias is added, queries (all heads at
        once) and keys (likewise) are RMS-normed with a weight per value, queries multiplied by
        1 + coef * ln(floor((p + 1) / every) + 1) (every 0: not), queries to q_out, keys and values to the pages
  head_norm_gate(x f32[T,heads*dv]|f32[S,T,heads*dv], weight act[dv], eps, gate act[T,W]|f32[S,T,W], gate_offset, out act[T,heads*dv], heads, dv)
        out = per-head rmsnorm(x) * weight * silu(gate[:, gate_offset : gate_offset + heads*dv])
  channel_decay(low act[T,W]|f32[S,T,W], low_offset, rank, w act[C,rank], bias act[C]|None, tau) -> f32[T,C]
        sigmoid(low[:, low_offset : low_offset + rank] w^T + bias)^(1/tau), in float32
  decayed_state_scan(proj, act_dtype, q_offset, k_offset, v_offset, q_scale, decay f32[T,heads*dk], states f32[slots,heads,dk,dv],
                     slots i32[B], fresh bool[B]|None, q_start i32[B], q_len i32[B], heads, dk, dv) -> f32[S,T,heads*dv]
        per request and head, token by token: S = diag(decay_t) S + k_t v_t^T, o_t = S^T (q_t * q_scale); S is read from and
        written to states[slots[b]] (fresh[b]: it starts at zero); q, k, v are columns of the product rows; the output comes as
        partial sums over ranges of the key channels (the backend's choice of S), which the consumer adds
  (head_norm_store also takes row_width, cos_sin f32[T,rd/2,2] with rotary_dim and pairing 'half' | 'interleaved', norm_plain,
   norm_after_rotation, values_are_keys; latent_prep takes queries (the query heads as a product of their own) and lead_width;
   head_norm_gate takes gate_act 'silu' | 'sigmoid' | 'factor', x_width and x_act; normed_pair_mean without weights is
   factor * a + factor_b * b; channel_decay takes rates f32[C] and negate: sigmoid(-z)^rates = exp(-rates * softplus(z));
   decayed_state_scan takes k_silu, v_silu and head_decay f32[heads] in place of decay)
  short_conv(proj, act_dtype, col0, conv_w act[C,taps], taps, unit_heads, unit_dim, scaled_heads, scale, unit_eps, sig_offset,
             n_sig, states f32[slots,N], state_offset, slots i32[B], fresh bool[B]|None, q_start, q_len, max_q_len) -> f32[T,C+n_sig]
        columns col0.. of the product rows through C causal convolutions over time (the last tap is the current token's; the
        taps - 1 inputs before a step's first token come from states[slot, state_offset:] as [taps-1, C], zeros where fresh,
        and that record is brought up to date), SiLU, the first unit_heads heads of unit_dim made unit vectors
        (x / sqrt(sum x^2 + unit_eps), the first scaled_heads times scale); behind them sigmoid of n_sig further columns
  delta_rule_scan(ops f32[T,W], q_offset, k_offset, v_offset, beta_offset, decay f32[T,heads*dk], states f32[slots,N],
                  state_offset, slots, fresh, q_start, q_len, heads, kv_heads, dk, dv) -> f32[1,T,heads*dv]
        per request and value head, token by token: S = diag(decay_t) S; u = beta_t (v_t - S^T k_t); S += k_t u^T; o_t = S^T q_t;
        head h reads the queries and keys of head h // (heads // kv_heads); S [heads,dk,dv] lies at states[slot, state_offset:]
  expert_mixture(x act[T,H], router act[E,H], router_bias act[E]|None, w_gate_up act[E,2F,H], w_down act[E,H,F], top) -> f32[T,H]
        float32 logits x router^T + bias, the `top` largest (lowest index among equals), softmax over those; the weighted
        sum of down_e(silu(gate_e x) * (up_e x)) over the chosen experts e, added in the order of the choices

Beside these, a backend has fused variants that fold neighbouring operations into one kernel.  They are part of
the contract too (`KernelBackend` below): each returns None (False for the decode attention) where it does not
cover a case, and the caller then takes the unfused way.
"""
from __future__ import annotations

import contextlib

_backend = None


class ProductSum:
    """factor_a * a + factor_b * b of two products (each act [T, H] or float32 partial sums [S, T, H]) that nothing has
    added up yet: what two mixers side by side hand to an arrangement whose next kernel (`post_norm_add`) takes it as it
    is, so that the sum costs no kernel of its own."""

    __slots__ = ("a", "factor_a", "b", "factor_b")

    def __init__(self, a, factor_a, b, factor_b):
        self.a, self.factor_a, self.b, self.factor_b = a, float(factor_a), b, float(factor_b)


class KernelBackend:
    """What parts may call on a backend beyond the operations listed above, with the answers of a backend that
    fuses nothing.  `kernels.hip.HipKernels` overrides them where its kernels cover the shapes."""

    name = "abstract"
    max_head_dim = 256      # the widest attention head the kernels take: a part refuses more when it is built
    fused_rows = 0          # products whose x operand is computed while it is staged take at most this many rows
    max_window_attention_dim = 1024     # the widest key or value that window_attention takes

    def pinned_stream(self):
        """Context manager within which every launch goes to the stream that is current on entry."""
        return contextlib.nullcontext()

    def residual_dtype(self, n_tokens, act_dtype):
        """The type of a step's residual stream: float32, or int64 (64-bit fixed point in units of 2^-32) where the
        backend's products can add themselves into the stream (`residual=`)."""
        import torch

        return torch.float32

    def residual_add(self, h, delta) -> None:
        """h += delta in place, for a residual stream of either kind: delta act [T, H] or float32 partial sums
        [S, T, H].  For norms other than the built-in one (whose kernel adds and normalises in one pass): plain
        tensor arithmetic, so that such a norm need not know how the stream is kept."""
        import torch

        d = delta.sum(0, dtype=torch.float32) if delta.dim() == 3 else delta.float()
        if h.dtype == torch.int64:
            h += torch.round(d.double() * 4294967296.0).to(torch.int64)
        else:
            h += d

    def residual_values(self, h):
        """The residual stream as a float32 tensor [T, H] (a copy if it is kept in fixed point)."""
        import torch

        return (h.double() * (1.0 / 4294967296.0)).float() if h.dtype == torch.int64 else h

    def heads_product(self, x, w, out=None):
        """x[h] w[h] for every head h: x act [heads, T, K] (any strides), w act [heads, K, N] -> act [heads, T, N]
        (written into `out`, a view of those sizes whose rows are contiguous, if given).  The library's batched
        product (float32 operands are multiplied in float32)."""
        import torch

        return torch.bmm(x, w) if out is None else torch.bmm(x, w, out=out)

    def product(self, x, w, unrounded=False, residual=None):
        """x w^T as act [m, n], or as float32 partial sums [splits, m, n] for a consumer that adds them up; or, given
        a residual stream in fixed point that the backend can add the product into, that stream."""
        raise NotImplementedError

    def product_normed(self, h, delta, norm_weight, w):
        """((h + delta) * norm_weight) w^T without the rows' 1/rms factor: (float32 partial sums [S, T, N], row sums
        of squares [S2, T], h + delta as a new tensor), or None."""
        return None

    def product_swiglu(self, gate_up, row_ss, hidden, eps, w, residual=None):
        """swiglu(scale * sum of the partial sums gate_up) w^T as float32 partial sums (or added into `residual`,
        which is then returned), or None."""
        return None

    def product_attention(self, part_o, part_ml, w, residual=None):
        """(the combined parts of a split attention) w^T as float32 partial sums (or added into `residual`, which is
        then returned), or None."""
        return None

    def gate_up_swiglu(self, x, w):
        """silu(x Wgate^T) * (x Wup^T) as act [T, I] in one kernel, or None."""
        return None

    def attention_decode_fused(self, *args, **kwargs):
        """Bias, rotation, cache store and attention for single decoded tokens straight from the QKV product's partial
        sums; False if not covered (nothing was done), else what paged_attention returns."""
        return False

    def combine_attention(self, part_o, part_ml, out):
        """out act [T, nq*hd] from the parts of a split attention."""
        raise NotImplementedError

    def rope_table(self, positions, inv_freq):
        """float32 [T, half, 2]: (cos, sin) of every token's angles, for the kernels that rotate; or None."""
        return None


class KernelsUnavailable(RuntimeError):
    pass


def backend():
    global _backend
    if _backend is None:
        from .hip import HipKernels  # raises KernelsUnavailable with the reason

        _backend = HipKernels()
    return _backend


def use_backend(obj) -> None:
    """Install `obj` as the backend (None restores the default).  For tests."""
    global _backend
    _backend = obj


_tuning_dir = None
library_tuning = False      # whether the library's bfloat16 products are chosen by measurement (tune_library_products)


def tune_library_products(enable: bool = True) -> None:
    """Let the library's matrix products (the many-row bfloat16 products, torch.mm) be chosen by measurement: the
    first time a shape is multiplied outside a graph capture, torch's TunableOp times the library's candidates for
    it (about a second per shape with the limits set here) and keeps the fastest for the life of the process; the
    library's own first choice is up to a third slower on some shapes (the 2,048 x 9,728 x 896 product: 53 us
    against 40).  Process-wide, off unless asked for: a step with new shapes waits for the measurement, and which
    candidate wins may differ from run to run, and with it the last bits of a result."""
    global _tuning_dir, library_tuning
    import torch.cuda.tunable as tunable

    if enable and _tuning_dir is None:
        import os
        import tempfile

        _tuning_dir = tempfile.TemporaryDirectory(prefix="egpt_tuning_")      # TunableOp writes its picks to a file
        tunable.set_filename(os.path.join(_tuning_dir.name, "picks.csv"))
        tunable.set_max_tuning_duration(30)
        tunable.set_max_tuning_iterations(20)
    tunable.enable(bool(enable))
    tunable.tuning_enable(bool(enable))
    library_tuning = bool(enable)
