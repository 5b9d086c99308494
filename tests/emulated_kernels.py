"""A slow torch stand-in for the kernel backend, for tests on a machine without a GPU.

It lets the engine's bookkeeping (block tables, slots, ragged batches, page reuse,
the scheduler) be exercised on the CPU.  It is test equipment: the product never
installs it, and the GPU tests never use it.  Arithmetic is done in float64 and
rounded to the output tensor's dtype.
"""
from __future__ import annotations


import torch

from easy_gpt.cpp_amd.kernels import KernelBackend

F64 = torch.float64


def _whole(t):
    """A product operand: a tensor, or float32 partial sums [splits, rows, cols] to be added up."""
    return t.sum(0) if t is not None and t.dim() == 3 else t


class EmulatedKernels(KernelBackend):
    name = "emulated"

    def product(self, x, w, unrounded=False, residual=None):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype)
        self.linear(x, w, None, out)
        return out

    def embed(self, token_ids, table, out):
        out.copy_(table[token_ids.long()].to(out.dtype))

    def add_rmsnorm(self, h, delta, weight, eps, out):
        delta = _whole(delta)
        if delta is not None:
            h.add_(delta.to(h.dtype))
        x = h.to(F64)
        inv = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        out.copy_((x * inv * weight.to(F64)).to(out.dtype))

    def rows_add_rmsnorm(self, h, delta, rows, weight, eps, out):
        delta = _whole(delta)
        x = h[rows.long()].to(F64)
        if delta is not None:
            x = (h[rows.long()] + delta[rows.long()].to(h.dtype)).to(F64)
        inv = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        out.copy_((x * inv * weight.to(F64)).to(out.dtype))

    def linear(self, x, w, bias, out):
        y = x.to(F64) @ w.to(F64).T
        if bias is not None:
            y = y + bias.to(F64)
        out.copy_(y.to(out.dtype))

    def qkv_rope_store(self, qkv, bias, positions, inv_freq, rotary_dim, slots, k_cache, v_cache, nq, nkv, hd,
                       page_size, out=None, cos_sin=None):
        src = _whole(qkv)
        qkv = src if out is None else out
        t = qkv.shape[0]
        x = src.to(F64)
        if bias is not None:
            x = x + bias.to(F64)
        heads = x.view(t, nq + 2 * nkv, hd).clone()
        if rotary_dim:
            half = rotary_dim // 2
            ang = (positions.to(torch.float32)[:, None] * inv_freq[None, :]).to(F64)
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            rot = heads[:, : nq + nkv, :rotary_dim]
            x1, x2 = rot[..., :half].clone(), rot[..., half:].clone()
            heads[:, : nq + nkv, :half] = x1 * cos - x2 * sin
            heads[:, : nq + nkv, half:rotary_dim] = x1 * sin + x2 * cos
        qkv.copy_(heads.view(t, -1).to(qkv.dtype))
        if slots is not None:
            page = (slots // page_size).long()
            off = (slots % page_size).long()
            k_new = qkv.view(t, nq + 2 * nkv, hd)[:, nq : nq + nkv]
            v_new = qkv.view(t, nq + 2 * nkv, hd)[:, nq + nkv :]
            for i in range(t):
                k_cache[page[i], :, off[i], :] = k_new[i]
                v_cache[page[i], :, :, off[i]] = v_new[i]
        return qkv

    def paged_attention(self, qkv, out, k_cache, v_cache, block_table, q_start, q_len, kv_len, nq, nkv, hd,
                        page_size, scale, window, max_q_len, max_kv_len, combine=True, singles=True):
        group = nq // nkv
        q_all = qkv.view(qkv.shape[0], nq + 2 * nkv, hd)[:, :nq].to(F64)
        for b in range(q_start.shape[0]):
            s, n, kv = int(q_start[b]), int(q_len[b]), int(kv_len[b])
            for i in range(n):
                p = kv - n + i
                lo = max(0, p - window + 1) if window else 0
                js = torch.arange(lo, p + 1)
                pages = block_table[b, (js // page_size)].long()
                assert (pages >= 0).all(), "attention would read a page that was given back"
                offs = (js % page_size).long()
                for h in range(nq):
                    kh = h // group
                    keys = k_cache[pages, kh, offs, :].to(F64)
                    vals = v_cache[pages, kh, :, offs].to(F64)
                    sc = (keys @ q_all[s + i, h]) * scale
                    pr = torch.softmax(sc, dim=0)
                    out[s + i, h * hd : (h + 1) * hd] = (pr @ vals).to(out.dtype)

    def rope_table(self, positions, inv_freq):
        ang = (positions.to(torch.float32)[:, None] * inv_freq[None, :]).to(F64)
        return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.float32)

    def embed_rmsnorm(self, token_ids, table, weight, eps, out):
        x = table[token_ids.long()].to(F64)
        inv = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        out.copy_((x * inv * weight.to(F64)).to(out.dtype))

    @staticmethod
    def _store(k_cache, v_cache, slots, page_size, keys, values):
        page, off = (slots // page_size).long(), (slots % page_size).long()
        for i in range(keys.shape[0]):
            k_cache[page[i], :, off[i], :] = keys[i].to(k_cache.dtype)
            v_cache[page[i], :, :, off[i]] = values[i].to(v_cache.dtype)

    @staticmethod
    def _turn(a, cos_sin, magnitude, rotary_dim, pairing):
        """a [T, heads, d]: the first rotary_dim places turned by the table's angles."""
        a = a.clone()
        if rotary_dim:
            cs = cos_sin.to(F64) * magnitude
            co, si = cs[:, None, :, 0], cs[:, None, :, 1]
            if pairing == "interleaved":
                u, w = a[..., 0:rotary_dim:2].clone(), a[..., 1:rotary_dim:2].clone()
                a[..., 0:rotary_dim:2] = u * co - w * si
                a[..., 1:rotary_dim:2] = w * co + u * si
            else:
                half = rotary_dim // 2
                u, w = a[..., :half].clone(), a[..., half:rotary_dim].clone()
                a[..., :half] = u * co - w * si
                a[..., half:rotary_dim] = w * co + u * si
        return a

    def head_norm_store(self, proj, q_out, q_weight, k_weight, eps, norm_values, slots, k_cache, v_cache, nq, nkv, dk, dv,
                        page_size, row_width=None, cos_sin=None, rotary_dim=0, pairing="half", magnitude=1.0, norm_plain=False,
                        norm_after_rotation=False, values_are_keys=False):
        x = _whole(proj).to(F64)
        t = x.shape[0]
        unit = lambda a: a / torch.sqrt((a * a).mean(-1, keepdim=True) + eps)
        q = x[:, : nq * dk].view(t, nq, dk)
        k = x[:, nq * dk : (nq + nkv) * dk].view(t, nkv, dk)
        v = k.clone() if values_are_keys else x[:, (nq + nkv) * dk : (nq + nkv) * dk + nkv * dv].view(t, nkv, dv)
        turn = lambda a: self._turn(a, cos_sin, magnitude, rotary_dim, pairing)
        if norm_after_rotation:
            q, k = turn(q), turn(k)
        if q_weight is not None:
            q = unit(q) * q_weight.to(F64)
        elif norm_plain:
            q = unit(q)
        if k_weight is not None:
            k = unit(k) * k_weight.to(F64)
        elif norm_plain:
            k = unit(k)
        if not norm_after_rotation:
            q, k = turn(q), turn(k)
        if norm_values:
            v = unit(v)
        q_out.copy_(q.reshape(t, nq * dk).to(q_out.dtype))
        if slots is not None:
            self._store(k_cache, v_cache, slots, page_size, k, v)

    def latent_prep(self, proj, q_plain, q_full, c_weight, eps, cos_sin, magnitude, rotary_dim, slots, k_cache, v_cache,
                    nq, dim, rot, rank, page_size, queries=None, lead_width=None):
        x = _whole(proj).to(F64)
        t = x.shape[0]
        q = (x if queries is None else _whole(queries).to(F64))[:, : nq * (dim + rot)].view(t, nq, dim + rot)
        base = nq * (dim + rot) if queries is None else lead_width
        c, shared = x[:, base : base + rank], x[:, base + rank : base + rank + rot]
        c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * c_weight.to(F64)

        def turn(a):                                   # a [..., T, rot] with T second to last
            a = a.clone()
            if rotary_dim:
                cs = cos_sin.to(F64) * magnitude
                co, si = cs[:, :, 0], cs[:, :, 1]
                u, w = a[..., 0:rotary_dim:2].clone(), a[..., 1:rotary_dim:2].clone()
                a[..., 0:rotary_dim:2] = u * co - w * si
                a[..., 1:rotary_dim:2] = w * co + u * si
            return a

        q_plain.copy_(q[..., :dim].to(q_plain.dtype))
        q_full[..., rank:] = turn(q[..., dim:].transpose(0, 1)).transpose(0, 1).to(q_full.dtype)
        if slots is not None:
            keys = torch.cat([c, turn(shared)], dim=-1).view(t, 1, rank + rot)
            self._store(k_cache, v_cache, slots, page_size, keys, c.view(t, 1, rank))

    def heads_product(self, x, w, out=None):
        y = torch.bmm(x.to(F64), w.to(F64)).to(x.dtype)
        if out is None:
            return y
        out.copy_(y)
        return out

    def sigmoid_gate(self, x, heads, gate, gate_offset, out):
        t, n = out.shape
        g = _whole(gate)[:, gate_offset : gate_offset + n].to(F64)
        xx = x.to(F64)
        if heads:
            xx = xx.transpose(0, 1).reshape(t, n)
        out.copy_((xx * torch.sigmoid(g)).to(out.dtype))

    def window_attention(self, q, out, k_cache, v_cache, block_table, q_start, q_len, kv_len, nq, nkv, dk, dv, page_size,
                         scale, window, keep_first, sink, max_q_len, max_kv_len, dist_bias=None, block=0, slopes=None):
        group = nq // nkv
        q_all = q.view(q.shape[0], nq, dk).to(F64)
        for b in range(q_start.shape[0]):
            s, n, kv = int(q_start[b]), int(q_len[b]), int(kv_len[b])
            for i in range(n):
                p = kv - n + i
                lo = max(0, p - window + 1) if window else 0
                if block:
                    lo = max(lo, p // block * block)
                js = torch.cat([torch.arange(0, min(keep_first, lo)), torch.arange(lo, p + 1)])
                pages = block_table[b, (js // page_size)].long()
                assert (pages >= 0).all(), "attention would read a page that was given back"
                offs = (js % page_size).long()
                for h in range(nq):
                    kh = h // group
                    keys = k_cache[pages, kh, offs, :].to(F64)
                    vals = v_cache[pages, kh, :, offs].to(F64)
                    sc = (keys @ q_all[s + i, h]) * scale
                    if dist_bias is not None:
                        sc = sc + dist_bias[h, (p - js).clamp(max=dist_bias.shape[1] - 1)].to(F64)
                    if slopes is not None:
                        sc = sc - slopes[h].to(F64) * (p - js).to(F64)
                    m = sc.max() if sink is None else torch.maximum(sc.max(), sink[h].to(F64))
                    e = torch.exp(sc - m)
                    denom = e.sum() + (torch.exp(sink[h].to(F64) - m) if sink is not None else 0.0)
                    out[s + i, h * dv : (h + 1) * dv] = ((e / denom) @ vals).to(out.dtype)

    # ---- operations of designs with layer norms, side-by-side mixers, a decaying state and experts
    def embed_scaled(self, token_ids, table, factor, out):
        out.copy_((table[token_ids.long()].to(F64) * factor).to(out.dtype))

    def add_layernorm(self, h, delta, rows, weight, bias, eps, out):
        delta = _whole(delta)
        if rows is None:
            if delta is not None:
                h.add_(delta.to(h.dtype))
            x = h.to(F64)
        else:
            x = h[rows.long()].to(F64)
            if delta is not None:
                x = (h[rows.long()] + delta[rows.long()].to(h.dtype)).to(F64)
        mu = x.mean(-1, keepdim=True)
        y = (x - mu) / torch.sqrt(((x - mu) ** 2).mean(-1, keepdim=True) + eps) * weight.to(F64)
        out.copy_((y if bias is None else y + bias.to(F64)).to(out.dtype))

    def normed_pair_mean(self, a, b, bias_a, bias_b, weight_a, weight_b, eps, factor, factor_b=None, act_dtype=None):
        def normed(x, bias, w):
            x = _whole(x).to(F64)
            if bias is not None:
                x = x + bias.to(F64)
            if w is None:
                return x
            return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)

        fb = factor if factor_b is None else factor_b
        return (factor * normed(a, bias_a, weight_a) + fb * normed(b, bias_b, weight_b)).to(torch.float32)[None]

    def tanh_cap(self, x, cap, scale=1.0):
        y = x.to(F64) * scale
        x.copy_((y if cap is None else cap * torch.tanh(y / cap)).to(x.dtype))

    def whole_norm_store(self, proj, bias, q_out, q_weight, k_weight, eps, positions, coef, every, slots, k_cache, v_cache,
                         nq, nkv, dk, dv, page_size):
        x = _whole(proj).to(F64)
        t = x.shape[0]
        used = (nq + nkv) * dk + nkv * dv
        x = x[:, :used] + (bias.to(F64) if bias is not None else 0.0)
        unit = lambda a: a / torch.sqrt((a * a).mean(-1, keepdim=True) + eps)
        q, k, v = x[:, : nq * dk], x[:, nq * dk : (nq + nkv) * dk], x[:, (nq + nkv) * dk :]
        if q_weight is not None:
            q = unit(q) * q_weight.to(F64)
        if k_weight is not None:
            k = unit(k) * k_weight.to(F64)
        if every:
            q = q * (1.0 + coef * torch.log(((positions.long() + 1) // every + 1).to(F64)))[:, None]
        q_out.copy_(q.to(q_out.dtype))
        if slots is not None:
            self._store(k_cache, v_cache, slots, page_size, k.reshape(t, nkv, dk), v.reshape(t, nkv, dv))

    def head_norm_gate(self, x, weight, eps, gate, gate_offset, out, heads, dv, gate_act="silu", x_width=None, x_act=None):
        t = out.shape[0]
        xx = _whole(x).to(F64)[:, : heads * dv].reshape(t, heads, dv)
        xx = xx / torch.sqrt((xx * xx).mean(-1, keepdim=True) + eps) * weight.to(F64)
        if gate is None:
            out.copy_(xx.reshape(t, heads * dv).to(out.dtype))
            return
        g = _whole(gate)[:, gate_offset : gate_offset + heads * dv].to(F64)
        g = {"silu": g * torch.sigmoid(g), "sigmoid": torch.sigmoid(g), "factor": g}[gate_act]
        out.copy_((xx.reshape(t, heads * dv) * g).to(out.dtype))

    def channel_decay(self, low, low_offset, rank, w, bias, tau, rates=None, negate=False):
        z = _whole(low)[:, low_offset : low_offset + rank].to(F64) @ w.to(F64).T
        if bias is not None:
            z = z + bias.to(F64)
        if negate:
            z = -z
        return (torch.sigmoid(z) ** (1.0 / tau if rates is None else rates.to(F64))).to(torch.float32)

    def bounded_gate(self, z, z_offset, channels, bias, lower):
        v = _whole(z)[:, z_offset : z_offset + channels].to(F64)
        if bias is not None:
            v = v + bias.to(F64)
        low = lower.to(F64) if lower is not None else 0.0
        return (low + (1.0 - low) * torch.sigmoid(v)).to(torch.float32)

    def decayed_state_scan(self, proj, act_dtype, q_offset, k_offset, v_offset, q_scale, decay, states, slots, fresh, q_start,
                           q_len, heads, dk, dv, q_silu=False, tied_keys=False, k_silu=False, v_silu=False, head_decay=None):
        x = _whole(proj).to(F64)
        t = x.shape[0]
        if head_decay is not None:
            decay = head_decay.to(F64)[None, :, None].expand(t, heads, dk).reshape(t, heads * dk)
        out = torch.zeros((t, heads * dv), dtype=torch.float32)
        for b in range(q_start.shape[0]):
            s0, n, slot = int(q_start[b]), int(q_len[b]), int(slots[b])
            if n <= 0:
                continue
            st = torch.zeros((heads, dk, dv), dtype=F64) if fresh is not None and bool(fresh[b]) else states[slot].to(F64)
            for i in range(s0, s0 + n):
                q = x[i, q_offset : q_offset + heads * dk].view(heads, dk)
                q = (q * torch.sigmoid(q) if q_silu else q) * q_scale
                k = 1.0 - decay[i].to(F64).view(heads, dk) if tied_keys else x[i, k_offset : k_offset + heads * dk].view(heads, dk)
                v = x[i, v_offset : v_offset + heads * dv].view(heads, dv)
                if k_silu:
                    k = k * torch.sigmoid(k)
                if v_silu:
                    v = v * torch.sigmoid(v)
                st = decay[i].to(F64).view(heads, dk)[:, :, None] * st + k[:, :, None] * v[:, None, :]
                out[i] = torch.einsum("hkv,hk->hv", st, q).reshape(-1).to(torch.float32)
            states[slot] = st.to(states.dtype)
        return out

    def short_conv(self, proj, act_dtype, col0, conv_w, taps, unit_heads, unit_dim, scaled_heads, scale, unit_eps, sig_offset,
                   n_sig, states, state_offset, slots, fresh, q_start, q_len, max_q_len):
        x = _whole(proj).to(F64)
        t, c = x.shape[0], conv_w.shape[0]
        w = conv_w.to(F64)
        out = torch.zeros((t, c + n_sig), dtype=F64)
        for b in range(q_start.shape[0]):
            s0, n, slot = int(q_start[b]), int(q_len[b]), int(slots[b])
            if n <= 0:
                continue
            record = states[slot, state_offset : state_offset + (taps - 1) * c].view(taps - 1, c)
            before = torch.zeros((taps - 1, c), dtype=F64) if fresh is not None and bool(fresh[b]) else record.to(F64)
            z = torch.cat([before, x[s0 : s0 + n, col0 : col0 + c]], dim=0)
            y = sum(z[j : j + n] * w[:, j] for j in range(taps))
            y = y * torch.sigmoid(y)
            u = y[:, : unit_heads * unit_dim].reshape(n, unit_heads, unit_dim)
            u = u / torch.sqrt((u * u).sum(-1, keepdim=True) + unit_eps)
            u[:, :scaled_heads] = u[:, :scaled_heads] * scale
            y[:, : unit_heads * unit_dim] = u.reshape(n, -1)
            out[s0 : s0 + n, :c] = y
            out[s0 : s0 + n, c:] = torch.sigmoid(x[s0 : s0 + n, sig_offset : sig_offset + n_sig])
            if taps > 1:
                record.copy_(z[n:].to(states.dtype))
        return out.to(torch.float32)

    def delta_rule_scan(self, ops, q_offset, k_offset, v_offset, beta_offset, decay, states, state_offset, slots, fresh, q_start,
                        q_len, heads, kv_heads, dk, dv):
        x = ops.to(F64)
        t = x.shape[0]
        group = heads // kv_heads
        out = torch.zeros((t, heads * dv), dtype=torch.float32)
        for b in range(q_start.shape[0]):
            s0, n, slot = int(q_start[b]), int(q_len[b]), int(slots[b])
            if n <= 0:
                continue
            record = states[slot, state_offset : state_offset + heads * dk * dv].view(heads, dk, dv)
            st = torch.zeros((heads, dk, dv), dtype=F64) if fresh is not None and bool(fresh[b]) else record.to(F64)
            for i in range(s0, s0 + n):
                q = x[i, q_offset : q_offset + kv_heads * dk].view(kv_heads, dk).repeat_interleave(group, dim=0)
                k = x[i, k_offset : k_offset + kv_heads * dk].view(kv_heads, dk).repeat_interleave(group, dim=0)
                v = x[i, v_offset : v_offset + heads * dv].view(heads, dv)
                beta = x[i, beta_offset : beta_offset + heads]
                st = decay[i].to(F64).view(heads, dk)[:, :, None] * st
                u = beta[:, None] * (v - torch.einsum("hkv,hk->hv", st, k))
                st = st + k[:, :, None] * u[:, None, :]
                out[i] = torch.einsum("hkv,hk->hv", st, q).reshape(-1).to(torch.float32)
            record.copy_(st.to(states.dtype))
        return out[None]

    def expert_mixture(self, x, router, router_bias, w_gate_up, w_down, top, gated=True, score_all=False, correction=None,
                       weight_scale=1.0):
        xx = x.to(F64)
        z = xx @ router.to(F64).T
        if router_bias is not None:
            z = z + router_bias.to(F64)
        if score_all:
            sc = torch.softmax(z, dim=-1)
            pick = sc if correction is None else sc + correction.to(F64)
            idx = torch.argsort(-pick, dim=-1, stable=True)[:, :top]
            val = torch.gather(sc, -1, idx)
            wt = val / (val.sum(-1, keepdim=True) + 1e-20) * weight_scale
        else:
            val, idx = torch.topk(z, top, dim=-1)
            wt = torch.softmax(val, dim=-1)
        ff = w_gate_up.shape[1] // 2 if gated else w_gate_up.shape[1]
        out = torch.zeros(x.shape, dtype=F64)
        for t in range(x.shape[0]):
            for c in range(top):
                e = int(idx[t, c])
                gu = w_gate_up[e].to(F64) @ xx[t]
                if gated:
                    act = (gu[:ff] * torch.sigmoid(gu[:ff]) * gu[ff:]).to(x.dtype).to(F64)
                else:
                    act = (torch.relu(gu) ** 2).to(x.dtype).to(F64)
                out[t] += wt[t, c] * (w_down[e].to(F64) @ act)
        return out.to(torch.float32)

    def embed_positions(self, token_ids, positions, table, pos_table, out):
        out.copy_((table[token_ids.long()].to(F64) + pos_table[positions.long()].to(F64)).to(out.dtype))

    def post_norm_add(self, h, y, post_weight, eps, mult, history=None, n_history=0, mix=None, next_weight=None, h_out=None):
        def normed(x, w):
            mu = x.mean(-1, keepdim=True)
            return (x - mu) / torch.sqrt(((x - mu) ** 2).mean(-1, keepdim=True) + eps) * w.to(F64)

        from easy_gpt.cpp_amd.kernels import ProductSum

        if isinstance(y, ProductSum):
            y = y.factor_a * _whole(y.a).to(F64) + y.factor_b * _whole(y.b).to(F64)
        x = h.to(F64) + mult * normed(_whole(y).to(F64), post_weight)
        if history is not None:
            history[n_history].copy_(x.to(history.dtype))
            x = (mix.to(F64)[: n_history + 1, None, None] * history[: n_history + 1].to(F64)).sum(0)
        (h if h_out is None else h_out).copy_(x.to(h.dtype))
        if next_weight is None:
            return None
        return normed(x, next_weight).to(next_weight.dtype)

    def ff_activation(self, z, cols, mode, out, coef=None, eps=0.0, gate_col=-1):
        full = _whole(z).to(F64)
        v = full[:, :cols]
        if mode == "relu2":
            y = torch.relu(v) ** 2
        else:
            n = lambda u: u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps)
            c = coef.to(F64)
            y = c[0] * n(v) + c[1] * n(v * v) + c[2] * n(v * v * v) + c[3]
        if gate_col >= 0:
            y = y * torch.sigmoid(full[:, gate_col : gate_col + 1])
        out.copy_(y.to(out.dtype))

    def swiglu(self, gate_up, out):
        gate_up = _whole(gate_up)
        i = out.shape[1]
        g, u = gate_up[:, :i].to(F64), gate_up[:, i:].to(F64)
        out.copy_((u * g / (1.0 + torch.exp(-g))).to(out.dtype))

    def argmax(self, logits, out):
        out.copy_(torch.argmax(logits, dim=-1).to(out.dtype))

    def sample(self, logits, temperature, top_k, top_p, uniform, out):
        for r in range(logits.shape[0]):
            t = float(temperature[r])
            if t <= 0:
                out[r] = int(torch.argmax(logits[r]))
                continue
            p = torch.softmax(logits[r].to(F64) / t, dim=-1)
            k, tp = int(top_k[r]), float(top_p[r])
            if 0 < k < p.numel():
                kth = torch.topk(p, k).values[-1]
                p = torch.where(p >= kth, p, torch.zeros_like(p))
                p = p / p.sum()
            if 0.0 < tp < 1.0:
                ps, order = torch.sort(p, descending=True, stable=True)
                cum = torch.cumsum(ps, 0)
                cut = int((cum >= tp).nonzero()[0]) + 1
                keep = torch.zeros_like(p)
                keep[order[:cut]] = ps[:cut]
                p = keep / keep.sum()
            cdf = torch.cumsum(p, 0)
            idx = int(torch.searchsorted(cdf, torch.tensor(float(uniform[r]) * float(cdf[-1]), dtype=F64)))
            out[r] = min(idx, p.numel() - 1)
