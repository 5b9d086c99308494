"""The kernels and operands that the Bubetar design brought, each alone against the plain functions of
tests/plain_bubetar.py: the head preparation with rotation in either pairing, norms without weights before or behind
the rotation and values that are the keys; the latent preparation with queries from a product of their own; the norm of
heads taken from the first columns of wider rows, with a sigmoid gate and with a ready factor; the weighted sum of two
branches; the factor and cap on logits; decays from a step size and a rate per channel; the state scan with SiLU on keys
and values and one decay per head; the short convolutions with their carried inputs; and the delta rule's scan."""
import math

import pytest
import torch

import plain_bubetar as P
from test_gpu_head_kernels import close, rnd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
I32 = torch.int32


@pytest.fixture(scope="module")
def k():
    from easy_gpt.cpp_amd import kernels

    kernels.use_backend(None)
    return kernels.backend()


def product(x, dtype, splits):
    """A product as the kernels take it: whole in the activation type, or `splits` float32 partial sums; and its
    value as float64."""
    if not splits:
        given = x.to(dtype)
        return given.to(DEV), given.to(F64)
    g = torch.Generator().manual_seed(99)
    parts = torch.randn(splits, *x.shape, generator=g)
    parts[0] += x - parts.sum(0)
    return parts.to(DEV), parts.to(F64).sum(0) if splits > 1 else parts[0].to(F64)


def dev_ints(values):
    return torch.tensor(values, dtype=I32, device=DEV)


# ----------------------------------------------------------------------------- head preparation
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv, rot, pairing, mode, extra, splits", [
    (4, 2, 16, 24, 8, "interleaved", "weighted", 96, 2),        # norm with weights, then rotation of half a head; a gate behind
    (6, 2, 80, 80, 40, "half", "after", 0, 1),                  # rotation, then a norm without weights; values are the keys
    (3, 3, 12, 12, 12, "half", "after", 5, 0),
    (2, 1, 20, 20, 6, "half", "after", 0, 3),
    (5, 1, 8, 8, 0, "half", "weighted", 0, 0),                  # no rotation at all
    (2, 2, 70, 30, 70, "interleaved", "plain", 3, 1),           # a norm without weights before the rotation
])
def test_heads_are_normed_rotated_and_stored(k, dtype, nq, nkv, dk, dv, rot, pairing, mode, extra, splits):
    t, eps, page_size, mag = 9, 1e-5, 16, 1.0
    own_values = mode != "after"
    width = (nq + nkv) * dk + (nkv * dv if own_values else 0) + extra
    given, x = product(rnd(t, width, seed=1, scale=2.0), dtype, splits)
    positions = torch.tensor([0, 1, 2, 40, 41, 1000, 5, 6, 7], dtype=I32)
    table = {"base": 10000.0, "dims": rot}
    qw = (rnd(dk, seed=2, dtype=dtype) + 1) if mode == "weighted" else None
    kw = (rnd(dk, seed=3, dtype=dtype) + 1) if mode == "weighted" else None
    q = x[:, : nq * dk].view(t, nq, dk)
    key = x[:, nq * dk : (nq + nkv) * dk].view(t, nkv, dk)
    val = x[:, (nq + nkv) * dk : (nq + nkv) * dk + nkv * dv].view(t, nkv, dv) if own_values else key.clone()
    turn = lambda a: P.rotate(a, positions, table, "interleaved" if pairing == "interleaved" else "half")
    if mode == "after":
        q, key = P.rms_norm(turn(q), None, eps), P.rms_norm(turn(key), None, eps)
    else:
        q = turn(P.rms_norm(q, None if qw is None else qw.to(F64), eps))
        key = turn(P.rms_norm(key, None if kw is None else kw.to(F64), eps))
    slots = torch.tensor([3, 17, 18, 40, 41, 2, 63, 64, 80], dtype=I32)
    k_cache = torch.zeros((6, nkv, page_size, dk), dtype=dtype, device=DEV)
    v_cache = torch.zeros((6, nkv, dv, page_size), dtype=dtype, device=DEV)
    q_out = torch.empty((t, nq * dk), dtype=dtype, device=DEV)
    rotation = {}
    if rot:
        f = P.rotation_frequencies(table).to(torch.float32).to(DEV)
        rotation = dict(cos_sin=k.rope_table(positions.to(DEV), f), rotary_dim=rot, pairing=pairing, magnitude=mag)
    k.head_norm_store(given, q_out, None if qw is None else qw.to(DEV), None if kw is None else kw.to(DEV), eps, False, slots.to(DEV),
                      k_cache, v_cache, nq, nkv, dk, dv, page_size, row_width=width, norm_plain=mode != "weighted",
                      norm_after_rotation=mode == "after", values_are_keys=not own_values, **rotation)
    close(q_out, q.reshape(t, nq * dk), dtype, "queries")
    page, off = (slots // page_size).long(), (slots % page_size).long()
    close(k_cache[page.to(DEV), :, off.to(DEV), :], key, dtype, "keys in their pages")
    close(v_cache[page.to(DEV), :, :, off.to(DEV)], val, dtype, "values in their pages")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, dim, rot, rank, lead, dims, splits", [(3, 12, 8, 32, 24, 8, 2), (1, 20, 6, 18, 10, 4, 0), (4, 6, 0, 14, 12, 0, 1)])
def test_latent_preparation_takes_queries_from_a_product_of_their_own(k, dtype, nq, dim, rot, rank, lead, dims, splits):
    t, eps, page_size = 7, 1e-6, 16
    width = lead + rank + rot + 3
    given, x = product(rnd(t, width, seed=4), dtype, splits)
    q_given, qx = product(rnd(t, nq * (dim + rot), seed=5), dtype, splits)
    positions = torch.tensor([0, 1, 2, 3, 77, 78, 500], dtype=I32)
    table = {"base": 5000.0, "dims": dims}
    cw = rnd(rank, seed=6, dtype=dtype) + 1
    q = qx.view(t, nq, dim + rot)
    c = P.rms_norm(x[:, lead : lead + rank], cw.to(F64), eps)
    shared = P.rotate(x[:, lead + rank : lead + rank + rot].view(t, 1, rot), positions, table, "interleaved")[:, 0]
    q_rot = P.rotate(q[..., dim:], positions, table, "interleaved")
    slots = torch.tensor([5, 6, 7, 16, 31, 32, 47], dtype=I32)
    k_cache = torch.zeros((3, 1, page_size, rank + rot), dtype=dtype, device=DEV)
    v_cache = torch.zeros((3, 1, rank, page_size), dtype=dtype, device=DEV)
    q_plain = torch.empty((t, nq, dim), dtype=dtype, device=DEV)
    q_full = torch.zeros((t, nq, rank + rot), dtype=dtype, device=DEV)
    cos_sin = k.rope_table(positions.to(DEV), P.rotation_frequencies(table).to(torch.float32).to(DEV)) if dims else None
    k.latent_prep(given, q_plain, q_full, cw.to(DEV), eps, cos_sin, 1.0, dims, slots.to(DEV), k_cache, v_cache, nq, dim, rot, rank,
                  page_size, queries=q_given, lead_width=lead)
    close(q_plain, q[..., :dim], dtype, "unrotated query parts")
    if rot:
        close(q_full[..., rank:], q_rot, dtype, "rotated query parts")
    page, off = (slots // page_size).long().to(DEV), (slots % page_size).long().to(DEV)
    close(k_cache[page, 0, off, :], torch.cat([c, shared], dim=-1), dtype, "latent and rotated key")
    close(v_cache[page, 0, :, off], c, dtype, "latent as value")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dv, x_extra, x_splits, act", [(1, 48, 0, 3, "sigmoid"), (4, 12, 0, 1, "factor"), (1, 24, 40, 2, None),
                                                              (1, 10, 19, -1, None), (3, 70, 0, 0, "silu"), (1, 1300, 0, 1, "sigmoid"), (2, 2500, 7, 2, "factor"), (1, 257, 0, 0, None)])
def test_heads_are_normed_from_the_first_columns_of_a_row_and_gated(k, dtype, heads, dv, x_extra, x_splits, act):
    t, eps = 6, 1e-5
    width = heads * dv + x_extra
    x_raw = rnd(t, width, seed=7, scale=3.0)
    if x_splits < 0:                                            # one tensor of the activation type
        x_given, x = x_raw.to(dtype).to(DEV), x_raw.to(dtype).to(F64)
    elif x_splits == 0:
        x_given, x = x_raw.to(DEV), x_raw.to(F64)
    else:
        x_given, x = product(x_raw, torch.float32, x_splits)
    w = rnd(dv, seed=8, dtype=dtype) + 1
    want = P.rms_norm(x[:, : heads * dv].reshape(t, heads, dv), w.to(F64), eps).reshape(t, heads * dv)
    gate = None
    if act is not None:
        gate_given, g = product(rnd(t, heads * dv + 9, seed=9), dtype, 2)
        g = g[:, 4 : 4 + heads * dv]
        want = want * {"sigmoid": torch.sigmoid(g), "factor": g, "silu": g * torch.sigmoid(g)}[act]
        gate = gate_given
    out = torch.empty((t, heads * dv), dtype=dtype, device=DEV)
    k.head_norm_gate(x_given, w.to(DEV), eps, gate, 4, out, heads, dv, gate_act=act or "silu", x_width=width,
                     x_act=dtype if x_splits < 0 else None)
    close(out, want, dtype, f"normed heads, gate {act}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, sa, sb", [(64, 2, 0), (100, 0, 3), (1024, 1, 1)])
def test_two_branches_are_added_with_a_factor_each(k, dtype, hidden, sa, sb):
    t = 5
    a_given, a = product(rnd(t, hidden, seed=10, scale=2.0), dtype, sa)
    b_given, b = product(rnd(t, hidden, seed=11, scale=0.5), dtype, sb)
    out = k.normed_pair_mean(a_given, b_given, None, None, None, None, 1e-6, 0.6, factor_b=1.1, act_dtype=dtype)
    assert tuple(out.shape) == (1, t, hidden) and out.dtype == torch.float32
    close(out[0], 0.6 * a + 1.1 * b, torch.float32, "weighted sum of two branches")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, sa, sb", [(48, 3, 1), (256, 0, 2), (1000, 2, 0)])
def test_the_norm_behind_a_mixer_adds_up_two_sides_not_yet_joined(k, dtype, hidden, sa, sb):
    from easy_gpt.cpp_amd.kernels import ProductSum

    t, eps = 6, 1e-5
    h = rnd(t, hidden, seed=40, scale=2.0)
    a_given, a = product(rnd(t, hidden, seed=41, scale=2.0) + 0.3, dtype, sa)
    b_given, b = product(rnd(t, hidden, seed=42, scale=0.7), dtype, sb)
    post, nxt = rnd(hidden, seed=43, dtype=dtype) + 1, rnd(hidden, seed=44, dtype=dtype) + 1
    x = h.to(F64) + P.layer_norm(0.6 * a - 1.1 * b, post.to(F64), eps)
    h_dev = h.to(DEV).clone()
    got = k.post_norm_add(h_dev, ProductSum(a_given, 0.6, b_given, -1.1), post.to(DEV), eps, 1.0, next_weight=nxt.to(DEV))
    close(h_dev, x, torch.float32, "the stream")
    close(got, P.layer_norm(x, nxt.to(F64), eps), dtype, "the next norm")


def test_logits_take_a_factor_and_a_cap(k):
    x = rnd(7, 301, seed=12, scale=9.0)
    y = x.to(DEV).clone()
    k.tanh_cap(y, 11.0, scale=0.7)
    close(y, 11.0 * torch.tanh(0.7 * x.to(F64) / 11.0), torch.float32, "factor and cap")
    y = x.to(DEV).clone()
    k.tanh_cap(y, None, scale=-2.5)
    close(y, -2.5 * x.to(F64), torch.float32, "factor alone")
    y = x.to(DEV).clone()
    k.tanh_cap(y, 4.0)
    close(y, 4.0 * torch.tanh(x.to(F64) / 4.0), torch.float32, "cap alone")


# ----------------------------------------------------------------------------- decays and the constant-decay scan
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_decays_from_a_step_size_and_a_rate_per_channel(k, dtype):
    t, rank, heads, dk = 11, 5, 3, 14
    given, low = product(rnd(t, 40, seed=13, scale=2.0), dtype, 2)
    w, bias = rnd(heads * dk, rank, seed=14, dtype=dtype), rnd(heads * dk, seed=15, dtype=dtype)
    a_log = torch.tensor([-1.0, 0.3, 1.5])
    rates = torch.exp(a_log).repeat_interleave(dk)
    got = k.channel_decay(given, 7, rank, w.to(DEV), bias.to(DEV), 1.0, rates=rates.to(DEV), negate=True)
    z = low[:, 7 : 7 + rank] @ w.to(F64).T + bias.to(F64)
    want = torch.exp(-rates.to(F64) * torch.nn.functional.softplus(z))
    close(got, want, torch.float32, "exp(-rate softplus(z))")
    assert float(got.min()) >= 0.0 and float(got.max()) <= 1.0
    # without a rate and a sign it is the sigmoid
    close(k.channel_decay(given, 7, rank, w.to(DEV), None, 1.0), torch.sigmoid(low[:, 7 : 7 + rank] @ w.to(F64).T), torch.float32, "sigmoid")


def scan_setup(lengths, slots, n_slots):
    starts = [sum(lengths[:i]) for i in range(len(lengths))]
    return dev_ints(starts), dev_ints(lengths), dev_ints(slots), starts


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dk, dv", [(4, 24, 40), (2, 16, 24), (1, 36, 20), (3, 8, 130), (2, 64, 48)])
def test_the_scan_with_one_decay_per_head_and_silu_on_all_three(k, dtype, heads, dk, dv):
    """Three requests in a step: a portion behind a carried state, a single token, and a new prompt in a slot that held
    another's state."""
    lengths, slots = [37, 1, 50], [4, 0, 2]
    q_start, q_len, slot_t, starts = scan_setup(lengths, slots, 6)
    t = sum(lengths)
    width = 2 * heads * dk + heads * dv + 5
    given, x = product(rnd(t, width, seed=16), dtype, 2)
    decay = torch.tensor([0.5, 0.9, 0.97, 0.9995][:heads])
    states = rnd(6, heads, dk, dv, seed=17)
    fresh = torch.tensor([False, False, True])
    states_dev = states.to(DEV).clone()
    out = k.decayed_state_scan(given, dtype, 3, 3 + heads * dk, 3 + 2 * heads * dk, 1.0, None, states_dev, slot_t, fresh.to(DEV),
                               q_start, q_len, heads, dk, dv, q_silu=True, k_silu=True, v_silu=True, head_decay=decay.to(DEV))
    got = out.sum(0)
    for b, (s0, n, slot) in enumerate(zip(starts, lengths, slots)):
        rows = x[s0 : s0 + n]
        q = P.silu(rows[:, 3 : 3 + heads * dk]).view(n, heads, dk)
        key = P.silu(rows[:, 3 + heads * dk : 3 + 2 * heads * dk]).view(n, heads, dk)
        val = P.silu(rows[:, 3 + 2 * heads * dk : 3 + 2 * heads * dk + heads * dv]).view(n, heads, dv)
        o, last = P.constant_decay_scan(q, key, val, decay.tolist(), None if fresh[b] else states[slot].to(F64))
        close(got[s0 : s0 + n], o.reshape(n, heads * dv), torch.float32, f"outputs of request {b}")
        close(states_dev[slot], last, torch.float32, f"state of request {b}")
    for slot in (1, 3, 5):
        assert torch.equal(states_dev[slot].cpu(), states[slot])


# ----------------------------------------------------------------------------- short convolutions
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps, unit_heads, unit_dim, scaled, rest, n_sig", [(4, 6, 48, 3, 200, 5), (3, 4, 8, 2, 48, 4), (1, 6, 10, 3, 42, 3),
                                                                          (5, 2, 6, 1, 140, 2), (2, 2, 36, 1, 8, 1), (16, 1, 5, 1, 3, 0)])
def test_short_convolutions_with_carried_inputs_unit_heads_and_sigmoid_columns(k, dtype, taps, unit_heads, unit_dim, scaled, rest, n_sig):
    """A step of three requests (a portion behind carried inputs, a single token, a new prompt in a used slot), then a
    second step that goes on from what the first left: outputs and records against the plain convolution over the whole
    sequences."""
    c = unit_heads * unit_dim + rest
    col0, width = 2, 2 + c + n_sig + 3
    sig_off = col0 + c + 1
    offset, n_slots = 11, 5
    record = offset + (taps - 1) * c + 4
    w = rnd(c, taps, seed=18, scale=0.6, dtype=dtype)
    scale, unit_eps = unit_dim ** -0.5, 1e-6
    lengths1, slots, lengths2 = [9, 1, 14], [3, 0, 1], [2, 6, 1]
    seqs = [rnd(taps - 1 + l1 + l2, width, seed=20 + i, scale=1.5) for i, (l1, l2) in enumerate(zip(lengths1, lengths2))]
    fresh = [False, False, True]

    states = rnd(n_slots, record, seed=19)
    for i, slot in enumerate(slots):                          # what the records hold before the first step
        if not fresh[i]:
            states[slot, offset : offset + (taps - 1) * c] = seqs[i][: taps - 1, col0 : col0 + c].reshape(-1)
    states_dev = states.to(DEV).clone()

    def plain(i, lo, hi):
        """outputs for the rows lo..hi of sequence i (rows before taps - 1 are the carried inputs)."""
        x = given_values[i]
        before = torch.zeros(taps - 1, c, dtype=F64) if fresh[i] else x[: taps - 1, col0 : col0 + c]
        y = P.silu(P.short_convolution(x[taps - 1 :, col0 : col0 + c], w.to(F64), before))
        u = P.unit(y[:, : unit_heads * unit_dim].reshape(-1, unit_heads, unit_dim))
        u[:, :scaled] = u[:, :scaled] * scale
        y = torch.cat([u.reshape(y.shape[0], -1), y[:, unit_heads * unit_dim :], torch.sigmoid(x[taps - 1 :, sig_off : sig_off + n_sig])], dim=-1)
        return y[lo:hi]

    given_values = [s.to(F64) for s in seqs]
    done = [0, 0, 0]
    for step, lengths in enumerate((lengths1, lengths2)):
        q_start, q_len, slot_t, starts = scan_setup(lengths, slots, n_slots)
        rows = torch.cat([seqs[i][taps - 1 + done[i] : taps - 1 + done[i] + n] for i, n in enumerate(lengths)])
        given = rows.to(DEV)[None].contiguous()                # float32, one "partial sum": nothing is rounded
        fr = torch.tensor(fresh if step == 0 else [False] * 3).to(DEV)
        out = k.short_conv(given, dtype, col0, w.to(DEV), taps, unit_heads, unit_dim, scaled, scale, unit_eps, sig_off, n_sig,
                           states_dev, offset, slot_t, fr, q_start, q_len, max(lengths))
        assert tuple(out.shape) == (sum(lengths), c + n_sig)
        for i, (s0, n) in enumerate(zip(starts, lengths)):
            close(out[s0 : s0 + n], plain(i, done[i], done[i] + n), torch.float32, f"step {step} request {i}")
            done[i] += n
            kept = seqs[i][done[i] : done[i] + taps - 1, col0 : col0 + c]
            if fresh[i] and done[i] < taps - 1:               # fewer tokens yet than the record holds: zeros stand before them
                kept = torch.cat([torch.zeros(taps - 1 - done[i], c), seqs[i][taps - 1 : taps - 1 + done[i], col0 : col0 + c]])
            assert torch.equal(states_dev[slots[i], offset : offset + (taps - 1) * c].cpu().view(taps - 1, c), kept), (step, i)
    for slot in (2, 4):                                       # other requests' records and what else lies in a record
        assert torch.equal(states_dev[slot].cpu(), states[slot])
    assert torch.equal(states_dev[:, :offset].cpu(), states[:, :offset])
    assert torch.equal(states_dev[:, offset + (taps - 1) * c :].cpu(), states[:, offset + (taps - 1) * c :])


# ----------------------------------------------------------------------------- the delta rule
@pytest.mark.parametrize("heads, kv_heads, dk, dv", [(4, 4, 48, 80), (4, 2, 8, 12), (3, 3, 10, 14), (2, 1, 6, 70), (1, 1, 36, 8), (1, 1, 160, 64),
                                                     (6, 3, 16, 130), (2, 2, 300, 20), (1, 1, 600, 65)])
def test_the_delta_rule_scan(k, heads, kv_heads, dk, dv):
    """Three requests in a step (a portion behind a carried state, a single token, a new prompt in a used slot); then the
    first request's portion again in pieces of 1, 2 and the rest: the same bits."""
    lengths, slots = [45, 1, 38], [2, 4, 0]
    q_start, q_len, slot_t, starts = scan_setup(lengths, slots, 6)
    t = sum(lengths)
    qk, vw = kv_heads * dk, heads * dv
    offset, record = 7, 7 + heads * dk * dv + 5
    width = 2 * qk + vw + heads + 3
    q_off, k_off, v_off, b_off = 1, 1 + qk, 2 + 2 * qk, 3 + 2 * qk + vw
    ops = rnd(t, width, seed=30)
    ops[:, q_off : q_off + qk] = (P.unit(ops[:, q_off : q_off + qk].view(t, kv_heads, dk)) * dk ** -0.5).reshape(t, qk)
    ops[:, k_off : k_off + qk] = P.unit(ops[:, k_off : k_off + qk].view(t, kv_heads, dk)).reshape(t, qk)
    ops[:, b_off : b_off + heads] = torch.sigmoid(2 * ops[:, b_off : b_off + heads])
    decay = torch.sigmoid(2 + 2 * rnd(t, heads * dk, seed=31))
    states = rnd(6, record, seed=32, scale=0.5)
    fresh = torch.tensor([False, False, True])
    states_dev = states.to(DEV).clone()
    out = k.delta_rule_scan(ops.to(DEV), q_off, k_off, v_off, b_off, decay.to(DEV), states_dev, offset, slot_t, fresh.to(DEV), q_start,
                            q_len, heads, kv_heads, dk, dv)
    assert tuple(out.shape) == (1, t, vw)
    group = heads // kv_heads
    x = ops.to(F64)
    for b, (s0, n, slot) in enumerate(zip(starts, lengths, slots)):
        rows = x[s0 : s0 + n]
        q = rows[:, q_off : q_off + qk].view(n, kv_heads, dk).repeat_interleave(group, dim=1)
        key = rows[:, k_off : k_off + qk].view(n, kv_heads, dk).repeat_interleave(group, dim=1)
        val = rows[:, v_off : v_off + vw].view(n, heads, dv)
        before = None if fresh[b] else states[slot, offset : offset + heads * dk * dv].view(heads, dk, dv).to(F64)
        o, last = P.delta_rule_scan(q, key, val, rows[:, b_off : b_off + heads], decay[s0 : s0 + n].to(F64).view(n, heads, dk), before)
        close(out[0, s0 : s0 + n], o.reshape(n, vw), torch.float32, f"outputs of request {b}")
        close(states_dev[slot, offset : offset + heads * dk * dv].view(heads, dk, dv), last, torch.float32, f"state of request {b}")
    assert torch.equal(states_dev[[1, 3, 5]].cpu(), states[[1, 3, 5]])
    assert torch.equal(states_dev[:, :offset].cpu(), states[:, :offset]) and torch.equal(states_dev[:, -5:].cpu(), states[:, -5:])
    # the first request in pieces, from the same start
    again = states.to(DEV).clone()
    pieces, at = [], 0
    for n in (1, 2, lengths[0] - 3):
        o = k.delta_rule_scan(ops[at : at + n].to(DEV).contiguous(), q_off, k_off, v_off, b_off, decay[at : at + n].to(DEV).contiguous(), again,
                              offset, dev_ints([slots[0]]), torch.tensor([False]).to(DEV), dev_ints([0]), dev_ints([n]), heads, kv_heads, dk, dv)
        pieces.append(o[0])
        at += n
    assert torch.equal(torch.cat(pieces), out[0, : lengths[0]])
    assert torch.equal(again[slots[0]], states_dev[slots[0]])
