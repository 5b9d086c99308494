"""Bubetar on the CPU: configuration and registry, the model's description (tensor names, cache groups, state records),
pins of the plain implementation's mechanisms (tests/plain_bubetar.py), and the engine's bookkeeping (pages, state slots
with their convolution inputs, ragged batches) with the tests' slow stand-in for the kernels against the plain
implementation."""
import copy
import math

import pytest
import torch

import bubetar_models as BM
import helpers as H
import plain_bubetar as P
from emulated_kernels import EmulatedKernels
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.config import BubetarConfig, ConfigError, resolve_architecture
from easy_gpt.cpp_amd.engine import Engine
from easy_gpt.cpp_amd.parts import build_model
from easy_gpt.cpp_amd.parts.position import stretch_by_wavelength
from easy_gpt.cpp_amd.weights import WeightsError

F64 = torch.float64


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    return {name: BM.write_model(str(tmp_path_factory.mktemp(f"bubetar_{name}")), cfg, seed) for name, (cfg, seed) in BM.CONFIGS.items()}


@pytest.fixture()
def emulated():
    kernels.use_backend(EmulatedKernels())
    yield
    kernels.use_backend(None)


def plain_rows(model_dir, reqs):
    cfg, w = P.read_model(model_dir)
    return {rid: P.forward(cfg, w, ids) for rid, ids in reqs.items()}


# ----------------------------------------------------------------------------- configuration and description
def test_the_design_is_found_by_its_name_and_every_size_is_read():
    assert resolve_architecture(BM.CONFIG_A).name == "Bubetar"
    cfg = BubetarConfig.from_dict(BM.CONFIG_A)
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.logit_scale, cfg.logit_softcap, len(cfg.layers)) == (300, 64, 1e-6, 0.7, 12.0, 4)
    pair = cfg.layers[0].mixer
    left, right = pair.left, pair.right
    assert cfg.layers[0].type == "parallel" and cfg.layers[0].ff == 96 and (pair.left_scale, pair.right_scale) == (0.7, 1.3)
    assert (left.heads, left.kv_heads, left.dim, left.vdim, left.scale, left.window, left.rot.base, left.rot.dims) == (4, 2, 16, 24, 0.25, None, 10000.0, 8)
    assert (right.heads, right.dim, right.vdim, right.decay) == (2, 16, 24, (0.9, 0.97))
    m = cfg.layers[1].mixer
    assert (m.heads, m.dim, m.rot_dim, m.vdim, m.q_rank, m.kv_rank, m.scale, m.rot.base, m.rot.dims) == (3, 12, 8, 20, 24, 32, 0.2, 5000.0, 8)
    pair = cfg.layers[2].mixer
    assert cfg.layers[2].ff is None and pair.left.window == 12 and pair.left.rot.scaling == (4.0, 1.0, 4.0, 64.0)
    assert (pair.right.heads, pair.right.kv_heads, pair.right.dim, pair.right.vdim, pair.right.conv) == (4, 2, 8, 12, 3)
    plain = BubetarConfig.from_dict(BM.CONFIG_B)
    assert plain.logit_scale == 1.0 and plain.logit_softcap is None and plain.layers[3].mixer.left.window is None


@pytest.mark.parametrize("edit, key", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18), "dims"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c["layers"][0]["mlp"].pop("ff"), "ff"),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "dims"),
    (lambda c: c["layers"][2]["mixer"]["left"].update(vdim=24), "vdim"),
    (lambda c: c["layers"][2]["mixer"]["left"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][2]["mixer"]["left"]["rot"]["scaling"].pop("original"), "original"),
    (lambda c: c["layers"][2]["mixer"]["left"]["rot"]["scaling"].update(high=0.5), "high"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"]["right"].pop("conv"), "conv"),
])
def test_a_wrong_configuration_is_refused_by_name(edit, key):
    cfg = copy.deepcopy(BM.CONFIG_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=key):
        BubetarConfig.from_dict(cfg)


def test_the_description_names_every_tensor_groups_the_caches_and_sizes_the_states():
    arch = resolve_architecture(BM.CONFIG_A)
    model = build_model(arch.build_spec(BubetarConfig.from_dict(BM.CONFIG_A)))
    declared = {s.name: tuple(s.shape) for s in model.param_specs()}
    drawn = BM.draw_weights(BM.CONFIG_A, 1, ranks=(16, 16))
    assert declared == {k: tuple(v.shape) for k, v in drawn.items()}
    assert declared["l1.mix.uq"] == (3 * 20, 24) and declared["l1.mix.dkv"] == (32 + 8, 64) and declared["l0.mix.right.norm"] == (48,)
    assert declared["l2.mix.right.q.conv"] == (16, 3) and declared["l2.mix.left.sink"] == (4,) and "l2.mix.left.v" not in declared
    assert "l2.norm2" not in declared and "l2.mlp.up" not in declared
    # latent layers keep one key/value head of latent + rotated part (two groups: their sizes differ); each pair's
    # attention its keys and values, the windowed one with its window
    needs = {g.cache_ids: (g.need.window, tuple((t.name, t.dims) for t in g.need.tensors)) for g in model.cache_groups}
    assert needs[(0,)] == (None, (("k", (2, 16)), ("v", (2, 24))))
    assert needs[(1,)] == (None, (("k", (1, 40)), ("v", (1, 32))))
    assert needs[(2,)] == (12, (("k", (2, 16)), ("v", (2, 16))))
    assert needs[(3,)] == (None, (("k", (1, 28)), ("v", (1, 24))))
    # a constant-decay state is its matrices; a delta rule's record also holds taps - 1 inputs of every convolution
    assert model.state_needs[0].shape == (2, 16, 24)
    assert model.state_needs[2].shape == (4 * 8 * 12 + 2 * (2 * 2 * 8 + 4 * 12),)
    assert set(model.state_needs) == {0, 2}
    assert model.graph_safe


def test_the_stored_tensors_decide_the_ranks_of_the_low_rank_projections(tmp_path, emulated):
    path = BM.write_model(str(tmp_path / "m"), BM.CONFIG_A, 3, ranks=(3, 11))
    eng = Engine.from_dir(path, dtype="float32", device="cpu", page_size=4, max_tokens=32, max_requests=1)
    rule = eng.model.layers[2].mixer.branches[1]
    assert (rule.decay_rank, rule.gate_rank) == (3, 11)
    reqs = H.make_requests(300, [19], seed=2)
    H.assert_rows_match(H.replay(eng, H.trace_portions(reqs)), plain_rows(path, reqs), 1e-5, "ranks of 3 and 11")

    def mismatch(w):
        w["l2.mix.right.a2"] = w["l2.mix.right.a2"][:, :2].contiguous()

    bad = BM.write_model(str(tmp_path / "bad"), BM.CONFIG_A, 3, change=mismatch, ranks=(3, 11))
    with pytest.raises(ValueError, match="inner width"):
        Engine.from_dir(bad, dtype="float32", device="cpu", page_size=4, max_tokens=32, max_requests=1)


def test_a_missing_tensor_is_named(tmp_path, emulated):
    def drop(w):
        del w["l2.mix.left.sink"]

    path = BM.write_model(str(tmp_path / "m"), BM.CONFIG_A, 3, change=drop)
    with pytest.raises(WeightsError) as e:
        Engine.from_dir(path, dtype="float32", device="cpu", page_size=4, max_tokens=32, max_requests=1)
    assert e.value.missing == ["l2.mix.left.sink"]


# ----------------------------------------------------------------------------- pins of the plain mechanisms
def test_frequencies_are_kept_stretched_or_mixed_by_their_wavelength():
    rot = BM.rotation(100.0, 8, (4.0, 1.0, 3.0, 30))
    plainf = torch.tensor([100.0 ** (-2.0 * i / 8) for i in range(4)], dtype=F64)
    f = P.rotation_frequencies(rot)
    wavelength = 2 * math.pi / plainf                   # 6.3, 19.9, 62.8, 198.7: kept below 10, divided beyond 30
    assert wavelength[0] < 10 < wavelength[1] < 30 < wavelength[2]
    assert f[0] == plainf[0] and f[2] == plainf[2] / 4 and f[3] == plainf[3] / 4
    s = (30 / wavelength[1] - 1.0) / (3.0 - 1.0)
    assert abs(f[1] - ((1 - s) * plainf[1] / 4 + s * plainf[1])) < 1e-15
    assert torch.allclose(stretch_by_wavelength(plainf, 4.0, 1.0, 3.0, 30), f, rtol=1e-14, atol=0)


def test_the_two_pairings_turn_their_places_by_the_positions_angle():
    rot = {"base": 1.0, "dims": 4}                      # base 1: every frequency is 1, the angle is the position
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0]]], dtype=F64).repeat(2, 1, 1)
    pos = torch.tensor([0, 1])
    c, s = math.cos(1.0), math.sin(1.0)
    inter = P.rotate(x, pos, rot, "interleaved")
    half = P.rotate(x, pos, rot, "half")
    assert torch.equal(inter[0], x[0]) and torch.equal(half[0], x[0])
    assert torch.allclose(inter[1, 0], torch.tensor([1 * c - 2 * s, 2 * c + 1 * s, 3 * c - 4 * s, 4 * c + 3 * s, 5.0], dtype=F64))
    assert torch.allclose(half[1, 0], torch.tensor([1 * c - 3 * s, 2 * c - 4 * s, 3 * c + 1 * s, 4 * c + 2 * s, 5.0], dtype=F64))


def test_a_sink_takes_its_share_of_the_softmax_and_a_window_ends_where_it_says():
    t, w = 7, 3
    q = torch.zeros(t, 1, 2, dtype=F64)
    k = torch.randn(t, 1, 2, dtype=F64)
    v = torch.eye(t, dtype=F64)[:, None, :]              # the value of token j is the j-th unit vector: outputs are weights
    out = P.softmax_attention(q, k, v, 1.0, w, torch.tensor([math.log(2.0)], dtype=F64))[:, 0]
    for i in range(t):
        seen = range(max(0, i - w + 1), i + 1)
        for j in range(t):
            assert abs(float(out[i, j]) - (1.0 / (len(seen) + 2.0) if j in seen else 0.0)) < 1e-12


def test_the_constant_decay_scan_has_its_closed_form_and_goes_on_from_a_carried_state():
    t = 9
    ones = torch.ones(t, 2, 1, dtype=F64)
    o, s = P.constant_decay_scan(ones, ones, ones, (0.5, 0.9))
    for h, d in enumerate((0.5, 0.9)):
        for i in range(t):
            assert abs(float(o[i, h, 0]) - sum(d ** n for n in range(i + 1))) < 1e-12
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(t, 2, 3, generator=g, dtype=F64) for _ in range(3))
    whole, last = P.constant_decay_scan(q, k, v, (0.5, 0.9))
    first, carried = P.constant_decay_scan(q[:4], k[:4], v[:4], (0.5, 0.9))
    second, end = P.constant_decay_scan(q[4:], k[4:], v[4:], (0.5, 0.9), carried)
    assert torch.allclose(torch.cat([first, second]), whole) and torch.allclose(end, last)


def test_the_delta_rule_overwrites_what_a_key_held():
    """Without decay and with beta 1, writing (k, v) and then (k, v') leaves v' alone under k; a key at right angles
    keeps what it held; with beta 1/2 half of the difference is written; the decay acts per key channel."""
    k1, k2 = torch.tensor([1.0, 0.0], dtype=F64), torch.tensor([0.0, 1.0], dtype=F64)
    va, vb, vc = (torch.tensor(x, dtype=F64) for x in ([1.0, 2.0, 3.0], [-1.0, 0.5, 4.0], [7.0, 7.0, 7.0]))
    keys = torch.stack([k1, k2, k1, k1])[:, None, :]
    vals = torch.stack([va, vb, vc, va])[:, None, :]
    ones = torch.ones(4, 1, 2, dtype=F64)
    beta = torch.tensor([[1.0], [1.0], [1.0], [0.5]], dtype=F64)
    o, s = P.delta_rule_scan(keys, keys, vals, beta, ones)
    assert torch.allclose(o[0, 0], va) and torch.allclose(o[1, 0], vb) and torch.allclose(o[2, 0], vc)
    assert torch.allclose(o[3, 0], vc + 0.5 * (va - vc))
    assert torch.allclose(s[0, 1], vb)                     # the second key's row was never touched again
    decay = ones.clone()
    decay[1:, 0, 0] = 0.5                                 # the first key channel halves with every token from the second on
    o, s = P.delta_rule_scan(keys[:2], keys[:2], vals[:2], beta[:2] * 0, decay[:2], state=torch.stack([va, vb])[None])
    assert torch.allclose(s[0, 0], va * 0.5) and torch.allclose(s[0, 1], vb)
    # carried across a cut
    g = torch.Generator().manual_seed(1)
    q, k = (P.unit(torch.randn(8, 2, 4, generator=g, dtype=F64)) for _ in range(2))
    v = torch.randn(8, 2, 3, generator=g, dtype=F64)
    b, d = torch.rand(8, 2, generator=g, dtype=F64), torch.rand(8, 2, 4, generator=g, dtype=F64)
    whole, last = P.delta_rule_scan(q, k, v, b, d)
    first, carried = P.delta_rule_scan(q[:3], k[:3], v[:3], b[:3], d[:3])
    second, end = P.delta_rule_scan(q[3:], k[3:], v[3:], b[3:], d[3:], carried)
    assert torch.allclose(torch.cat([first, second]), whole) and torch.allclose(end, last)


def test_a_short_convolution_reads_zeros_before_the_start_and_its_last_tap_is_the_current_token():
    x = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]], dtype=F64)
    taps = torch.tensor([[100.0, 10.0, 1.0], [0.0, 0.0, 2.0]], dtype=F64)
    y = P.short_convolution(x, taps)
    assert y[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0] and y[:, 1].tolist() == [20.0, 40.0, 60.0, 80.0]
    again = P.short_convolution(x[2:], taps, before=x[:2])
    assert torch.equal(again, y[2:])


def test_latent_keys_equal_a_product_with_the_latent_carried_into_the_query(models):
    """q_plain . (W_uk c) = (W_uk^T q_plain) . c: the identity by which only the latent and the rotated part are cached."""
    cfg, w = P.read_model(models["A"])
    m = cfg["layers"][1]["mixer"]
    g = torch.Generator().manual_seed(0)
    c = torch.randn(m["kv_rank"], generator=g, dtype=F64)
    q = torch.randn(m["heads"], m["dim"], generator=g, dtype=F64)
    up = w["l1.mix.uk"].view(m["heads"], m["dim"], m["kv_rank"])
    direct = torch.einsum("hd,hd->h", q, torch.einsum("hdr,r->hd", up, c))
    carried = torch.einsum("hr,r->h", torch.einsum("hd,hdr->hr", q, up), c)
    assert torch.allclose(direct, carried)


# ----------------------------------------------------------------------------- the engine's bookkeeping
@pytest.mark.parametrize("name", ["A", "B", "D", "F"])
def test_cuttings_agree_with_plain(models, emulated, name):
    cfg = BM.CONFIGS[name][0]
    reqs = H.make_requests(cfg["vocab"], [5, 41, 1, 23], seed=11)
    ref = plain_rows(models[name], reqs)
    for page_size, trace in [(4, H.trace_whole(reqs)), (16, H.trace_last_decoded(reqs, 9)), (3, H.trace_portions(reqs))]:
        eng = Engine.from_dir(models[name], dtype="float32", device="cpu", page_size=page_size, max_tokens=64, max_requests=2)
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(v) for v in reqs.values())
        H.assert_rows_match(rows, ref, 1e-5, f"{name} page {page_size}")
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_batches_with_pages_and_state_slots_used_again(models, emulated, name):
    cfg = BM.CONFIGS[name][0]
    reqs = H.make_requests(cfg["vocab"], [23, 9, 37, 30, 14, 26, 3, 19], seed=3)
    ref = plain_rows(models[name], reqs)
    trace = H.trace_mixed(reqs, seed=1, max_live=3, decode_tail=5)
    need = H.max_live_tokens(trace, round_to=4)
    eng = Engine.from_dir(models[name], dtype="float32", device="cpu", page_size=4, max_tokens=need, max_requests=3)
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, 1e-5, name)
    assert max(len(r["entries"]) for r in trace) == 3          # eight requests went through three state slots


def test_the_logits_take_their_factor_and_their_cap(models, emulated):
    """The same weights with and without factor and cap: cap * tanh(factor * plain / cap)."""
    cfg = copy.deepcopy(BM.CONFIG_A)
    del cfg["logit_scale"], cfg["logit_softcap"]
    reqs = H.make_requests(300, [12], seed=5)
    import json
    import os
    import shutil
    import tempfile

    d = tempfile.mkdtemp()
    try:
        shutil.copy(os.path.join(models["A"], "model.safetensors"), d)
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(cfg, f)
        bare = plain_rows(d, reqs)["r0"]
        full = plain_rows(models["A"], reqs)["r0"]
        assert torch.allclose(full, 12.0 * torch.tanh(0.7 * bare / 12.0))
        assert float((full - bare).abs().max()) > 0.1
        eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=4, max_tokens=16, max_requests=1)
        H.assert_rows_match(H.replay(eng, H.trace_whole(reqs)), {"r0": bare}, 1e-5, "no factor, no cap")
    finally:
        shutil.rmtree(d)
