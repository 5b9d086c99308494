"""The kernels that the Kezolix design brought, each alone against the plain functions of tests/plain_kezolix.py:
the embedding with learned positions, the norm behind a branch with the depth average and the next norm, the forget
gate with its lower bound, the state scan whose write strength is one minus the forget gate, the normed polynomial and
the squared relu with a gate of one number per token, the router over all experts with a correction of the choice, and
the attention kernels with blocks of positions and a penalty per head and distance.  Where random inputs would hide a
fault (the keys at a block's two edges, the first block, a far key inside the block) the penalty alone decides: the
queries are zero, so a key's weight is a known function of its distance."""
import math

import pytest
import torch

import plain_kezolix as P
from test_gpu_head_kernels import close, paged, rnd

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


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


# ----------------------------------------------------------------------------- the stream
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [40, 256, 1000])
def test_embedding_with_learned_positions(k, dtype, hidden):
    table, pos = rnd(37, hidden, seed=1, dtype=dtype), rnd(50, hidden, seed=2, scale=0.5, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 17, 9], dtype=torch.int32)
    places = torch.tensor([0, 1, 49, 0, 23, 24], dtype=torch.int32)
    out = torch.empty((6, hidden), dtype=torch.float32, device=DEV)
    k.embed_positions(ids.to(DEV), places.to(DEV), table.to(DEV), pos.to(DEV), out)
    close(out, table.to(F64)[ids.long()] + pos.to(F64)[places.long()], torch.float32, "embedding + position")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, splits", [(48, 0), (100, 3), (256, 1), (2048, 0), (5000, 2)])
def test_the_norm_behind_a_branch_the_depth_average_and_the_next_norm(k, dtype, hidden, splits):
    t, eps, mult, n_before = 7, 1e-5, 0.7, 3
    h = rnd(t, hidden, seed=3, scale=2.0)
    y_given, y = product(rnd(t, hidden, seed=4, scale=3.0) + 0.5, dtype, splits)
    post, nxt = rnd(hidden, seed=5, dtype=dtype) + 1, rnd(hidden, seed=6, dtype=dtype) + 1
    x = h.to(F64) + mult * P.layer_norm(y, post.to(F64), eps)
    # without a history: the stream goes on as it is, with and without a norm for what follows
    h_dev = h.to(DEV).clone()
    assert k.post_norm_add(h_dev, y_given, post.to(DEV), eps, mult) is None
    close(h_dev, x, torch.float32, "the stream")
    h_dev = h.to(DEV).clone()
    got = k.post_norm_add(h_dev, y_given, post.to(DEV), eps, mult, next_weight=nxt.to(DEV))
    close(h_dev, x, torch.float32, "the stream")
    close(got, P.layer_norm(x, nxt.to(F64), eps), dtype, "the next norm")
    # with a history: the result is kept, what goes on is the weighted sum of all results so far
    history = rnd(n_before + 2, t, hidden, seed=7)
    mix = torch.tensor([0.4, -0.7, 0.2, 1.3])
    h_dev, hist_dev, onward = h.to(DEV).clone(), history.to(DEV).clone(), torch.empty((t, hidden), dtype=torch.float32, device=DEV)
    got = k.post_norm_add(h_dev, y_given, post.to(DEV), eps, mult, history=hist_dev, n_history=n_before, mix=mix.to(DEV),
                          next_weight=nxt.to(DEV), h_out=onward)
    results = [history[j].to(F64) for j in range(n_before)] + [x]
    avg = P.depth_average(results, mix.to(F64))
    close(hist_dev[n_before], x, torch.float32, "the kept result")
    assert torch.equal(hist_dev[:n_before].cpu(), history[:n_before]) and torch.equal(hist_dev[n_before + 1].cpu(), history[n_before + 1])
    close(onward, avg, torch.float32, "the depth average")
    close(got, P.layer_norm(avg, nxt.to(F64), eps), dtype, "the next norm of the average")
    assert torch.equal(h_dev.cpu(), h)


# ----------------------------------------------------------------------------- the recurrence
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("channels, offset, extra, splits", [(20, 0, 0, 0), (64, 24, 8, 2), (300, 7, 1, 1)])
def test_the_forget_gate_with_its_lower_bound(k, dtype, channels, offset, extra, splits):
    t = 9
    z_given, z = product(rnd(t, offset + channels + extra, seed=8, scale=3.0), dtype, splits)
    bias = rnd(channels, seed=9, dtype=dtype)
    lower = torch.rand(channels, generator=torch.Generator().manual_seed(10)).to(dtype)
    lower[0], lower[1] = 0.0, 1.0                                 # no bound at all; a channel that never forgets
    got = k.bounded_gate(z_given, offset, channels, bias.to(DEV), lower.to(DEV))
    low = lower.to(F64)
    want = low + (1 - low) * torch.sigmoid(z[:, offset : offset + channels] + bias.to(F64))
    close(got, want, torch.float32, "forget gates")
    assert float(got[:, 1].min()) == 1.0 and float((got.cpu() - lower.float()).min()) >= 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dk, dv", [(2, 16, 24), (3, 10, 12), (1, 160, 64), (2, 128, 128)])
def test_the_state_scan_writes_with_one_minus_the_forget_gate(k, dtype, heads, dk, dv):
    """Three requests in one step (a prompt's portion behind a carried state, a single token behind one, a new prompt in
    a slot that held another request's state), silu on the queries, keys that are one minus the gate."""
    lens, slots, fresh = [13, 1, 40], [2, 0, 3], [False, False, True]
    t = sum(lens)
    width = heads * dk + heads * dv + 5
    proj_given, proj = product(rnd(t, width, seed=11), dtype, 0)
    f = (0.05 + 0.95 * torch.rand(t, heads * dk, generator=torch.Generator().manual_seed(12))).float()
    f[:, 0] = 1.0
    states = rnd(4, heads, dk, dv, seed=13)
    st_dev = states.to(DEV).clone()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    starts = [0, lens[0], lens[0] + lens[1]]
    out = k.decayed_state_scan(proj_given, dtype, 5, 0, 5 + heads * dk, 1.0, f.to(DEV), st_dev, i32(slots), torch.tensor(fresh, device=DEV),
                               i32(starts), i32(lens), heads, dk, dv, q_silu=True, tied_keys=True)
    got = out.sum(0).cpu()
    for b, (s0, n, slot, new) in enumerate(zip(starts, lens, slots, fresh)):
        z = proj[s0 : s0 + n, 5 : 5 + heads * dk]
        q = (z * torch.sigmoid(z)).view(n, heads, dk)
        v = proj[s0 : s0 + n, 5 + heads * dk : 5 + heads * (dk + dv)].view(n, heads, dv)
        want, last = P.gated_state_scan(q, f[s0 : s0 + n].to(F64).view(n, heads, dk), v, None if new else states[slot].to(F64))
        close(got[s0 : s0 + n], want.reshape(n, heads * dv), torch.float32, f"request {b}")
        close(st_dev[slot], last, torch.float32, f"state of request {b}")
    assert torch.equal(st_dev[1].cpu(), states[1])               # a slot of no request of the step


# ----------------------------------------------------------------------------- feed-forward
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cols, extra, splits", [(50, 0, 0), (320, 0, 0), (320, 8, 0), (321, 1, 0), (96, 0, 3), (8192, 0, 0), (8192, 8, 0),
                                                 (8200, 0, 0), (9000, 1, 0), (4097, 0, 1), (320, 0, 1), (8192, 8, 1)])
def test_the_normed_polynomial(k, dtype, cols, extra, splits):
    """Rows that are kept in registers and rows too long for that; whole pieces of 16 bytes and rows that do not start
    on one; with and without a gate column behind the row."""
    t, eps = 5, 1e-5
    z_given, z = product(rnd(t, cols + extra, seed=14, scale=1.7), dtype, splits)
    coef = torch.tensor([0.6, -0.4, 0.3, 0.2])
    out = torch.empty((t, cols), dtype=dtype, device=DEV)
    k.ff_activation(z_given, cols, "polynorm", out, coef=coef.to(DEV), eps=eps)
    want = P.normed_polynomial(z[:, :cols], coef.to(F64), eps)
    close(out, want, dtype, "normed polynomial")
    if extra:
        k.ff_activation(z_given, cols, "polynorm", out, coef=coef.to(DEV), eps=eps, gate_col=cols + extra - 1)
        close(out, want * torch.sigmoid(z[:, -1:]), dtype, "with a gate")
    # each power is normed by itself: a row of one repeated value gives a + b + c + e whatever the value
    flat = torch.full((1, cols), 3.0).to(dtype).to(DEV)
    one = torch.empty((1, cols), dtype=dtype, device=DEV)
    k.ff_activation(flat, cols, "polynorm", one, coef=coef.to(DEV), eps=0.0)
    close(one, torch.full((1, cols), float(coef.sum()), dtype=F64), dtype, "a flat row")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cols, extra, splits", [(50, 1, 0), (64, 8, 0), (96, 0, 0), (2048, 8, 0), (300, 1, 2), (2048, 8, 1)])
def test_the_squared_relu_with_a_gate_of_one_number(k, dtype, cols, extra, splits):
    t = 6
    z_given, z = product(rnd(t, cols + extra, seed=15, scale=1.5), dtype, splits)
    out = torch.empty((t, cols), dtype=dtype, device=DEV)
    k.ff_activation(z_given, cols, "relu2", out)
    want = torch.relu(z[:, :cols]) ** 2
    close(out, want, dtype, "squared relu")
    if extra:
        k.ff_activation(z_given, cols, "relu2", out, gate_col=cols)
        close(out, want * torch.sigmoid(z[:, cols : cols + 1]), dtype, "with a gate")


@pytest.mark.parametrize("experts, top, hidden, ff, scale", [(6, 2, 64, 48, 1.5), (5, 1, 100, 50, 2.0), (3, 3, 100, 30, 1.0),
                                                             (16, 4, 128, 32, 1.0), (32, 4, 256, 64, 2.5)])
def test_the_router_over_all_experts(k, experts, top, hidden, ff, scale):
    """float32: softmax over all experts, the choice by score + correction, the weights by the scores alone, over
    their sum, times the scale; an expert is down(relu(up x)^2).  The correction is large enough to change who is
    chosen for most tokens."""
    t = 70
    x = rnd(t, hidden, seed=16)
    w = {"router": rnd(experts, hidden, seed=17, scale=2.0 / hidden ** 0.5),
         "correction": torch.where(torch.arange(experts) % 2 == 0, 0.3, 0.0)}
    for e in range(experts):
        w[f"e{e}.up"] = rnd(ff, hidden, seed=100 + e, scale=hidden ** -0.5)
        w[f"e{e}.down"] = rnd(hidden, ff, seed=200 + e, scale=ff ** -0.5)
    w64 = {n: v.to(F64) for n, v in w.items()}
    router = {"experts": experts, "top": top, "scale": scale}
    want = P.expert_mixture(x.to(F64), w64, "", {"router": router})
    plain_choice, _ = P.route(x.to(F64), w64, "", router)
    if top < experts:
        uncorrected, _ = P.route(x.to(F64), dict(w64, correction=torch.zeros(experts, dtype=F64)), "", router)
        assert (plain_choice.sort(-1).values != uncorrected.sort(-1).values).any(-1).float().mean() > 0.15
    up = torch.stack([w[f"e{e}.up"] for e in range(experts)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(experts)]).to(DEV)
    got = k.expert_mixture(x.to(DEV), w["router"].to(DEV), None, up, down, top, gated=False, score_all=True,
                           correction=w["correction"].to(DEV), weight_scale=scale)
    close(got, want, torch.float32, "mixture of squared-relu experts")


# ----------------------------------------------------------------------------- attention
def run_block_attention(k, q, k_cache, v_cache, table, kv_len, page_size, scale, block, slopes, dv):
    m, nq, dk = q.shape
    nkv = k_cache.shape[1]
    out = torch.empty((m, nq * dv), dtype=q.dtype, device=DEV)
    i32 = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
    k.window_attention(q.reshape(m, nq * dk).to(DEV).contiguous(), out, k_cache, v_cache, table, i32(0), i32(m), i32(kv_len),
                       nq, nkv, dk, dv, page_size, scale, 0, 0, None, m, kv_len, block=block, slopes=slopes)
    return out.view(m, nq, dv)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv, block", [(4, 2, 16, 24, 12), (3, 3, 12, 20, None), (5, 1, 8, 8, 1), (8, 2, 64, 32, 100),
                                                    (4, 4, 32, 64, 64), (16, 4, 128, 128, 256), (6, 3, 16, 16, 50), (2, 2, 48, 32, 33)])
@pytest.mark.parametrize("n, m", [(300, 300), (300, 1), (257, 2), (200, 37)])
def test_attention_within_blocks_with_slopes(k, dtype, nq, nkv, dk, dv, block, n, m):
    """The last m of n tokens ask (a whole prompt, a single token, a portion of two, a portion that starts inside a
    block), on the matrix-core kernel where its sizes fit and on the general one elsewhere."""
    from easy_gpt.cpp_amd.parts.local_attention import head_slopes

    q_all = rnd(n, nq, dk, seed=20, scale=1.5).to(dtype)
    keys, values = rnd(n, nkv, dk, seed=21).to(dtype), rnd(n, nkv, dv, seed=22).to(dtype)
    want = P.sloped_block_attention(q_all.to(F64), keys.to(F64), values.to(F64), 0.3, block)[n - m :]
    k_cache, v_cache, table = paged(keys, values, 16, dtype, seed=23)
    slopes = head_slopes(nq, 8.0).to(DEV)
    close(slopes, P.head_slopes(nq), torch.float32, "slopes")
    got = run_block_attention(k, q_all[n - m :], k_cache, v_cache, table, n, 16, 0.3, block or 0, slopes, dv)
    close(got, want, dtype, f"attention of the last {m} of {n}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block", [7, 64, 100, 1000])
@pytest.mark.parametrize("single", [False, True])
def test_zero_queries_weigh_a_block_by_distance_alone(k, dtype, block, single):
    """With queries of zero a key's weight is exp(-slope * distance) over the sum of these within the query's block,
    and key j carries the value j in its first feature and 1 at feature 1 + (j mod 15): the output names the keys that
    were seen and their weights, at a block's last position, at the next block's first, inside the first block and
    far inside a block."""
    nq, nkv, dk, dv, n = 4, 2, 16, 16, 2 * block + 3 if block < 1000 else 1500
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / nq) for h in range(nq)], dtype=F64)
    keys = rnd(n, nkv, dk, seed=24).to(dtype)
    values = torch.zeros(n, nkv, dv)
    values[:, :, 0] = torch.arange(n)[:, None].float() / 8.0       # (eighths: exact in bfloat16 up to 2,048 / 8)
    for j in range(n):
        values[j, :, 1 + j % 15] = 1.0
    values = values.to(dtype)
    k_cache, v_cache, table = paged(keys, values, 16, dtype, seed=25)
    asks = sorted({p for p in (0, 1, block - 1, block, block + 1, 2 * block - 1, 2 * block, n - 1) if p < n})
    for p in asks:
        first = p // block * block
        dist = (p - torch.arange(first, p + 1)).to(F64)
        wgt = torch.softmax(-slopes[:, None] * dist[None, :], dim=-1)                      # [heads, keys seen]
        want = torch.einsum("hj,jd->hd", wgt, values[first : p + 1, 0].to(F64))
        if single:
            q = torch.zeros(1, nq, dk, dtype=dtype)
            got = run_block_attention(k, q, k_cache, v_cache, table, p + 1, 16, 0.3, block, slopes.float().to(DEV), dv)[0]
        else:
            q = torch.zeros(p + 1, nq, dk, dtype=dtype)
            got = run_block_attention(k, q, k_cache, v_cache, table, p + 1, 16, 0.3, block, slopes.float().to(DEV), dv)[p]
        close(got, want, dtype, f"position {p} of blocks of {block}")
