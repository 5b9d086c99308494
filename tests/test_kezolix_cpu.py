"""Kezolix on the CPU: configuration and registry, the model's description (tensor names, which layer reads whose cache,
state records), pins of the plain implementation's mechanisms (tests/plain_kezolix.py), and the engine's bookkeeping
(pages, state slots, ragged batches, the depth's results) with the tests' slow stand-in for the kernels against the
plain implementation."""
import copy
import math

import pytest
import torch

import helpers as H
import kezolix_models as KM
import plain_kezolix as P
from emulated_kernels import EmulatedKernels
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.config import ConfigError, KezolixConfig, resolve_architecture
from easy_gpt.cpp_amd.engine import Engine
from easy_gpt.cpp_amd.parts import build_model
from easy_gpt.cpp_amd.parts.local_attention import head_slopes
from easy_gpt.cpp_amd.weights import WeightsError

F64 = torch.float64


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    return {name: KM.write_model(str(tmp_path_factory.mktemp(f"kezolix_{name}")), cfg, seed) for name, (cfg, seed) in KM.CONFIGS.items()}


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
    assert resolve_architecture(KM.CONFIG_B).name == "Kezolix"
    cfg = KezolixConfig.from_dict(KM.CONFIG_B)
    assert (cfg.vocab, cfg.width, cfg.max_positions, cfg.eps, cfg.residual_mult, len(cfg.layers)) == (257, 100, 400, 1e-5, 1.0, 5)
    r, m = cfg.layers[0].mixer, cfg.layers[0].mlp
    assert cfg.layers[0].type == "hgrn2" and (r.heads, r.dim, r.vdim) == (3, 10, 12)
    assert (m.kind, m.experts, m.top, m.ff, m.scale, m.shared_ff) == ("moe", 5, 1, 50, 2.0, None)
    a = cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.block, a.kv_from) == (3, 3, 12, 20, 0.3, None, None)
    assert cfg.layers[2].mixer.block == 1 and cfg.layers[2].mlp is None
    assert (cfg.layers[1].mlp.kind, cfg.layers[1].mlp.ff) == ("dense", 50)
    assert cfg.layers[3].mlp.shared_ff == 20
    assert KezolixConfig.from_dict(KM.CONFIG_A).layers[2].mixer.kv_from == 0


@pytest.mark.parametrize("edit, key", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "kind"),
    (lambda c: c["layers"][0]["mlp"].pop("ff"), "ff"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=16), "vdim"),
])
def test_a_wrong_configuration_is_refused_by_name(edit, key):
    cfg = copy.deepcopy(KM.CONFIG_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=key):
        KezolixConfig.from_dict(cfg)


def test_the_description_names_every_tensor_and_who_reads_whose_cache():
    arch = resolve_architecture(KM.CONFIG_A)
    spec = arch.build_spec(arch.config_class.from_dict(KM.CONFIG_A))
    model = build_model(spec)
    shapes = {s.name: tuple(s.shape) for s in model.param_specs()}
    drawn = KM.draw_weights(KM.CONFIG_A, 1)
    assert shapes == {k: tuple(v.shape) for k, v in drawn.items()}
    assert "l2.mix.k" not in shapes and "l2.mix.k.norm" not in shapes and shapes["l2.mix.q"] == (64, 64)
    assert shapes["l0.dwa"] == (2,) and shapes["l3.dwa"] == (5,) and shapes["l1.mlp.shared.sg"] == (1, 64)
    runs = spec.run_order
    assert [(r.layer, r.cache, r.writes_cache, r.state) for r in runs] == [(0, 0, True, None), (1, None, True, 1),
                                                                           (2, 0, False, None), (3, None, True, 3)]
    assert len(model.cache_groups) == 1 and model.cache_groups[0].cache_ids == (0,)
    assert sorted(model.state_needs) == [1, 3] and model.state_needs[3].shape == (3, 10, 12)
    assert spec.max_position == 512 and model.graph_safe


def test_a_missing_tensor_is_named(tmp_path, emulated):
    def drop(w):
        del w["l1.mix.lower"]

    path = KM.write_model(str(tmp_path / "m"), KM.CONFIG_A, 2, change=drop)
    with pytest.raises(WeightsError) as e:
        Engine.from_dir(path, dtype="float32", device="cpu", max_tokens=64)
    assert e.value.missing == ["l1.mix.lower"]


def test_a_request_cannot_outgrow_the_position_table(models, emulated):
    from easy_gpt.cpp_amd.engine import StepEntry

    eng = Engine.from_dir(models["B"], dtype="float32", device="cpu", page_size=16, max_tokens=512, max_requests=1)
    eng.add_request("a")
    eng.step([StepEntry("a", [1] * 400, [])])
    with pytest.raises(ValueError, match="400"):
        eng.step([StepEntry("a", [1], [0])])


# ----------------------------------------------------------------------------- pins of the plain mechanisms
def test_slopes_halve_every_eighth_of_the_heads():
    assert P.head_slopes(8).tolist() == pytest.approx([2.0 ** -(h + 1) for h in range(8)])
    assert P.head_slopes(1).tolist() == pytest.approx([2.0 ** -8])
    assert P.head_slopes(3).tolist() == pytest.approx([2.0 ** (-8 / 3), 2.0 ** (-16 / 3), 2.0 ** -8])
    for n in (1, 2, 5, 8, 14):
        assert head_slopes(n, 8.0).tolist() == pytest.approx(P.head_slopes(n).tolist(), rel=1e-6)


def test_blocks_are_counted_from_position_zero():
    seen = P.block_visible(10, 4)
    assert seen[3].tolist() == [True] * 4 + [False] * 6
    assert seen[4].tolist() == [False] * 4 + [True] + [False] * 5            # the first token of a block sees itself alone
    assert seen[9].tolist() == [False] * 8 + [True, True]
    assert P.block_visible(5, None)[4].all() and P.block_visible(5, 1).sum() == 5


def test_attention_with_queries_of_zero_weighs_keys_by_their_distance_alone():
    t, dv = 9, 3
    q = torch.zeros(t, 2, 4, dtype=F64)
    k = torch.randn(t, 1, 4, dtype=F64)
    v = torch.randn(t, 1, dv, dtype=F64)
    out = P.sloped_block_attention(q, k, v, 0.7, 5)
    slopes = P.head_slopes(2)
    for head in range(2):
        wts = torch.exp(-slopes[head] * torch.tensor([3.0, 2.0, 1.0, 0.0], dtype=F64))       # position 8 sees 5..8
        want = (wts[:, None] * v[5:9, 0]).sum(0) / wts.sum()
        assert torch.allclose(out[8, head], want, atol=1e-12)
    assert torch.allclose(out[5, 0], v[5, 0])


def test_the_state_scan_goes_on_from_a_carried_state_and_writes_what_it_does_not_keep():
    g = torch.Generator().manual_seed(0)
    q, f, v = torch.rand(7, 2, 3, generator=g, dtype=F64), torch.rand(7, 2, 3, generator=g, dtype=F64), torch.randn(7, 2, 4, generator=g, dtype=F64)
    whole, last = P.gated_state_scan(q, f, v)
    head, carried = P.gated_state_scan(q[:3], f[:3], v[:3])
    tail, last2 = P.gated_state_scan(q[3:], f[3:], v[3:], carried)
    assert torch.allclose(torch.cat([head, tail]), whole, atol=1e-14) and torch.allclose(last2, last, atol=1e-14)
    # a gate of one keeps the state and writes nothing; a gate of zero replaces it by the value
    ones, zeros = torch.ones(1, 1, 2, dtype=F64), torch.zeros(1, 1, 2, dtype=F64)
    s0 = torch.randn(1, 2, 3, dtype=F64)
    val = torch.randn(1, 1, 3, dtype=F64)
    assert torch.equal(P.gated_state_scan(ones, ones, val, s0)[1], s0)
    assert torch.equal(P.gated_state_scan(ones, zeros, val, s0)[1], val[0][:, None, :].expand(1, 2, 3))


def test_forget_gates_lie_between_their_lower_bound_and_one():
    w = {"m.f": torch.zeros(2, 3, dtype=F64), "m.f.b": torch.tensor([-50.0, 0.0], dtype=F64), "m.lower": torch.tensor([0.25, 0.5], dtype=F64)}
    f = P.forget_gates(torch.ones(1, 3, dtype=F64), w, "m.")
    assert f[0].tolist() == pytest.approx([0.25, 0.75])


def test_the_normed_polynomial_norms_each_power_by_itself():
    z = torch.tensor([[1.0, -2.0, 0.5, 3.0]], dtype=F64)
    out = P.normed_polynomial(z, torch.tensor([2.0, 0.0, 0.0, 0.5], dtype=F64), 0.0)
    assert torch.allclose(out, 2.0 * z / math.sqrt(float((z * z).mean())) + 0.5)
    out = P.normed_polynomial(z, torch.tensor([0.0, 0.0, 1.0, 0.0], dtype=F64), 0.0)
    assert float((out * out).mean()) == pytest.approx(1.0)
    assert torch.allclose(P.normed_polynomial(3.0 * z, torch.tensor([1.0, 1.0, 1.0, 0.0], dtype=F64), 0.0),
                          P.normed_polynomial(z, torch.tensor([1.0, 1.0, 1.0, 0.0], dtype=F64), 0.0))


def test_the_correction_steers_the_choice_and_not_the_weights():
    w = {"m.router": torch.eye(4, dtype=F64), "m.correction": torch.tensor([0.0, 0.0, 0.0, 0.9], dtype=F64)}
    h = torch.tensor([[1.0, 3.0, 2.0, -1.0]], dtype=F64)
    idx, weight = P.route(h, w, "m.", {"top": 2, "scale": 2.0})
    s = torch.softmax(h[0], 0)
    assert idx.tolist() == [[3, 1]]                       # expert 3 is chosen through its correction alone
    assert weight[0].tolist() == pytest.approx([2.0 * float(s[3] / (s[3] + s[1])), 2.0 * float(s[1] / (s[3] + s[1]))])
    w["m.correction"] = torch.zeros(4, dtype=F64)
    assert P.route(h, w, "m.", {"top": 2, "scale": 1.0})[0].tolist() == [[1, 2]]


def test_the_depth_average_reads_every_earlier_result(models):
    """The stream that leaves layer n is sum_j a[j] X_j over the embedding's output and the n + 1 results so far: a model
    cut after layer n gives the logits of that stream, and zeroing the weight of the embedding's output in the last
    layer's average changes the logits."""
    cfg, w = P.read_model(models["A"])
    tokens = H.make_requests(cfg["vocab"], [15], seed=2)["r0"]
    streams = []
    full = P.forward(cfg, w, tokens, streams)
    assert len(streams) == 4 and streams[0].shape == (15, 64)
    assert torch.equal(P.layer_norm(streams[-1], w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T, full)
    x0 = w["embed"][torch.tensor(tokens)] + w["pos"][:15]
    w2 = dict(w)
    w2["l3.dwa"] = w["l3.dwa"].clone()
    w2["l3.dwa"][0] = 0.0
    s2 = []
    P.forward(cfg, w2, tokens, s2)
    assert torch.allclose(streams[-1] - s2[-1], w["l3.dwa"][0] * x0, atol=1e-12)


# ----------------------------------------------------------------------------- the engine's bookkeeping
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "F", "G"])
def test_cuttings_agree_with_plain(models, emulated, name):
    cfg = KM.CONFIGS[name][0]
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
    cfg = KM.CONFIGS[name][0]
    reqs = H.make_requests(cfg["vocab"], [23, 9, 37, 30, 14, 26, 3, 19], seed=3)
    ref = plain_rows(models[name], reqs)
    trace = H.trace_mixed(reqs, seed=1, max_live=3, decode_tail=5)
    need = H.max_live_tokens(trace, round_to=4)
    eng = Engine.from_dir(models[name], dtype="float32", device="cpu", page_size=4, max_tokens=need, max_requests=3)
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, 1e-5, name)
    assert max(len(r["entries"]) for r in trace) == 3          # eight requests went through three state slots


def test_a_layer_without_a_depth_average_and_with_a_norm_of_another_eps(emulated):
    """The sandwich arrangement described by hand, without a stream join and with a second norm whose eps differs from
    the first one's (the fused kernel takes one eps; the arrangement then norms in a step of its own)."""
    from easy_gpt.cpp_amd.parts import LayerSpec, ModelSpec, PartSpec, RunSpec

    width, vocab, eps = 40, 50, 1e-5
    norm = lambda prefix, name, e=eps: PartSpec("layernorm", dict(eps=e, name=name, bias_name=None), prefix=prefix)
    spec = ModelSpec(
        hidden_size=width, vocab_size=vocab, max_position=64,
        embedding=PartSpec("token_embedding_positions", dict(max_positions=64, name="embed", position_name="pos")),
        layers=(LayerSpec("sandwich", PartSpec("bounded_gate_recurrence", dict(n_heads=2, key_dim=5, value_dim=9, eps=eps), prefix="a."),
                          PartSpec("activated", dict(intermediate_size=24, activation="polynorm", eps=eps), prefix="f."),
                          {"mixer": norm("a.", "n1"), "mixer_out": norm("a.", "n1b"), "feed_forward": norm("a.", "n2", 1e-2),
                           "feed_forward_out": norm("a.", "n2b")}, block_params=dict(residual_mult=0.5)),),
        run_order=(RunSpec(0, state=0),),
        final_norm=norm("", "fn"), output_head=PartSpec("linear_head", dict(tied=False, name="head")),
    )
    model = build_model(spec)
    g = torch.Generator().manual_seed(3)
    w = {}
    for ps in model.param_specs():
        t = torch.randn(ps.shape, generator=g) * (0.3 if len(ps.shape) > 1 else 0.5)
        if ps.role == "norm_scale":
            t = 1.0 + 0.2 * t
        if ps.name == "a.lower":
            t = t.abs().clamp(max=0.9)
        w[ps.name] = t.to(torch.bfloat16).to(torch.float32)
    model.load(lambda name: w[name], torch.float32, "cpu")
    eng = Engine(model, page_size=4, max_tokens=64, max_requests=2)
    tokens = H.make_requests(vocab, [21], seed=4)["r0"]
    w64 = {k: v.to(F64) for k, v in w.items()}
    x = w64["embed"][torch.tensor(tokens)] + w64["pos"][:21]
    y = P.gated_recurrence(P.layer_norm(x, w64["a.n1"], eps), w64, "a.", dict(heads=2, dim=5, vdim=9), eps)
    x = x + 0.5 * P.layer_norm(y, w64["a.n1b"], eps)
    z = P.normed_polynomial(P.layer_norm(x, w64["a.n2"], 1e-2) @ w64["f.up"].T, w64["f.act"], eps) @ w64["f.down"].T
    x = x + 0.5 * P.layer_norm(z, w64["a.n2b"], eps)
    want = P.layer_norm(x, w64["fn"], eps) @ w64["head"].T
    for trace in (H.trace_whole({"r0": tokens}), H.trace_portions({"r0": tokens})):
        H.assert_rows_match(H.replay(eng, trace), {"r0": want}, 1e-5, "sandwich alone")
