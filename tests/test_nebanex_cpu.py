"""Nebanex on the CPU: configuration and registry, the model's description (tensor names, cache groups, state records),
sizes that the stored tensors decide, pins of the plain implementation's mechanisms (tests/plain_nebanex.py), and the
engine's bookkeeping (pages, state slots, ragged batches) with the tests' slow stand-in for the kernels against the
plain implementation."""
import copy
import math

import pytest
import torch

import helpers as H
import nebanex_models as NM
import plain_nebanex as P
from emulated_kernels import EmulatedKernels
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.config import ConfigError, NebanexConfig, resolve_architecture
from easy_gpt.cpp_amd.engine import Engine
from easy_gpt.cpp_amd.parts import build_model
from easy_gpt.cpp_amd.parts.branch_mixers import distance_bias_table
from easy_gpt.cpp_amd.weights import WeightsError

F64 = torch.float64


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    return {name: NM.write_model(str(tmp_path_factory.mktemp(f"nebanex_{name}")), cfg, seed, rows, rank)
            for name, (cfg, seed, rows, rank) in NM.CONFIGS.items()}


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
    assert resolve_architecture(NM.CONFIG_B).name == "Nebanex"
    cfg = NebanexConfig.from_dict(NM.CONFIG_B)
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.embedding_scale, cfg.logit_softcap, len(cfg.layers)) == (257, 100, 1e-5, 1.0, None, 3)
    l, r, m = cfg.layers[0].left, cfg.layers[0].right, cfg.layers[0].mlp
    assert (l.heads, l.kv_heads, l.dim, l.vdim, l.scale, l.bias_max, l.growth_coef, l.growth_every) == (3, 3, 12, 20, 0.3, 9, 0.2, 1)
    assert (r.heads, r.dim, r.vdim, r.tau) == (3, 10, 12, 1.0)
    assert (m.experts, m.top, m.ff, m.shared_ff) == (5, 1, 50, None)
    assert cfg.layers[1].mlp is None and cfg.layers[1].left.growth_coef is None
    assert cfg.layers[2].mlp.shared_ff == 20
    assert NebanexConfig.from_dict(NM.CONFIG_A).logit_softcap == 8.0


@pytest.mark.parametrize("edit, key", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.pop("embedding"), "embedding"),
    (lambda c: c["layers"][0]["mixer"]["left"].pop("bias_max"), "bias_max"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=2), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["q_temp"].update(every=0), "every"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][0]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][0].update(type="serial"), "serial"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][2]["mlp"]["shared"].pop("ff"), "ff"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
])
def test_a_wrong_configuration_is_refused_by_name(edit, key):
    cfg = copy.deepcopy(NM.CONFIG_B)
    edit(cfg)
    with pytest.raises(ConfigError, match=key):
        NebanexConfig.from_dict(cfg)


def test_the_description_names_every_tensor_one_cache_and_one_state_per_layer():
    arch = resolve_architecture(NM.CONFIG_B)
    spec = arch.build_spec(arch.config_class.from_dict(NM.CONFIG_B))
    assert [ls.block for ls in spec.layers] == ["pre_norm", "pre_norm_mixer_only", "pre_norm"]
    assert [(r.layer, r.cache, r.state) for r in spec.run_order] == [(0, 0, 0), (1, 1, 1), (2, 2, 2)]
    model = build_model(spec)
    names = {s.name: s.shape for s in model.param_specs()}
    assert names["embed"] == (257, 100) and names["head"] == (257, 100)
    assert names["final.norm"] == (100,) and names["final.norm.b"] == (100,)
    assert names["l0.norm1"] == (100,) and names["l0.norm1.b"] == (100,) and names["l0.norm2.b"] == (100,)
    assert "l1.norm2" not in names and not any(n.startswith("l1.mlp.") for n in names)
    assert names["l0.mix.left.q"] == (36, 100) and names["l0.mix.left.q.b"] == (36,) and names["l0.mix.left.k"] == (36, 100)
    assert names["l0.mix.left.v"] == (60, 100) and names["l0.mix.left.v.b"] == (60,)
    assert names["l0.mix.left.q.norm"] == (36,) and names["l0.mix.left.k.norm"] == (36,)
    assert names["l0.mix.left.g"] == (60, 100) and names["l0.mix.left.o"] == (100, 60) and names["l0.mix.left.o.b"] == (100,)
    assert names["l0.mix.left.rel"][1] == 3
    assert names["l2.mix.left.k"] == (8, 100) and names["l2.mix.left.q"] == (40, 100)
    assert names["l0.mix.right.q"] == (30, 100) and names["l0.mix.right.v"] == (36, 100) and names["l0.mix.right.o"] == (100, 36)
    assert names["l0.mix.right.norm"] == (12,) and names["l0.mix.right.a2.b"] == (30,)
    assert names["l0.mix.right.a1"][1] == 100 and names["l0.mix.right.a2"][0] == 30
    assert names["l0.mix.left.out"] == (100,) and names["l0.mix.right.out"] == (100,)
    assert names["l0.mlp.e4.gate"] == (50, 100) and names["l0.mlp.e4.down"] == (100, 50) and "l0.mlp.e5.gate" not in names
    assert names["l0.mlp.router"] == (5, 100) and names["l0.mlp.router.b"] == (5,) and "l0.mlp.shared.gate" not in names
    assert names["l2.mlp.shared.gate"] == (20, 100) and names["l2.mlp.shared.down"] == (100, 20)
    # every layer has keys and values of its own sizes, and a state record [heads, key size, value size]
    assert sorted(g.cache_ids for g in model.cache_groups) == [(0,), (1,), (2,)]
    assert all(g.need.window is None for g in model.cache_groups)
    assert {i: n.shape for i, n in model.state_needs.items()} == {0: (3, 10, 12), 1: (1, 36, 70), 2: (2, 6, 100)}
    assert all(n.dtype == torch.float32 for n in model.state_needs.values())
    assert model.graph_safe


def test_the_stored_tensors_decide_the_table_rows_and_the_decay_rank(tmp_path, emulated):
    cfg, seed, _, _ = NM.CONFIGS["A"]
    reqs = H.make_requests(cfg["vocab"], [30], seed=1)
    for rows, rank in [(4, 1), (10, 7), (32, 16)]:
        d = NM.write_model(str(tmp_path / f"m{rows}"), cfg, seed, rows, rank)
        eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=4, max_tokens=64, max_requests=1)
        H.assert_rows_match(H.replay(eng, H.trace_whole(reqs)), plain_rows(d, reqs), 1e-5, f"rows {rows} rank {rank}")
    # the two projections of the decay must agree, and other axes are checked as ever
    bad = NM.write_model(str(tmp_path / "bad"), cfg, seed, 8, 5, change=lambda w: w.update({"l0.mix.right.a2": w["l0.mix.right.a2"][:, :4].contiguous()}))
    with pytest.raises(ValueError, match="inner width"):
        Engine.from_dir(bad, dtype="float32", device="cpu", page_size=4, max_tokens=64)
    bad = NM.write_model(str(tmp_path / "bad2"), cfg, seed, 8, 5, change=lambda w: w.update({"l0.mix.left.rel": w["l0.mix.left.rel"][:, :3].contiguous()}))
    with pytest.raises(WeightsError, match="l0.mix.left.rel"):
        Engine.from_dir(bad, dtype="float32", device="cpu", page_size=4, max_tokens=64)


def test_a_missing_tensor_is_named(tmp_path, emulated):
    cfg, seed, rows, rank = NM.CONFIGS["A"]
    d = NM.write_model(str(tmp_path / "m"), cfg, seed, rows, rank, change=lambda w: w.pop("l1.mix.right.a2.b"))
    with pytest.raises(WeightsError, match="l1.mix.right.a2.b"):
        Engine.from_dir(d, dtype="float32", device="cpu", page_size=4, max_tokens=64)


# ----------------------------------------------------------------------------- pins of the plain mechanisms
def test_distance_buckets_are_exact_up_close_and_logarithmic_beyond():
    assert [P.distance_bucket(n, 10, 70) for n in range(6)] == [0, 1, 2, 3, 4, 5]
    # 5 * 14^(k/5) is where row 5 + k starts: 5, 8.5, 14.4, 24.4, 41.3, 70
    assert [P.distance_bucket(n, 10, 70) for n in (8, 9, 14, 15, 24, 25, 41, 42, 69, 70, 5000)] == [5, 6, 6, 7, 7, 8, 8, 9, 9, 9, 9]
    for rows, far in [(8, 20), (6, 9), (16, 50), (32, 300), (4, 3)]:
        b = [P.distance_bucket(n, rows, far) for n in range(far + 40)]
        assert b[: rows // 2] == list(range(rows // 2)) and b == sorted(b) and max(b) == rows - 1 and b[far] == rows - 1
    # the engine's table by distance is the same function
    rel = torch.arange(8 * 3, dtype=torch.float32).view(8, 3)
    table = distance_bias_table(rel, 20)
    assert table.shape == (3, 21)
    for n in range(21):
        assert table[:, n].tolist() == rel[P.distance_bucket(n, 8, 20)].tolist()


def test_the_query_factor_steps_with_the_logarithm_of_the_position():
    f = P.query_factor(range(40), 0.5, 16)
    assert f[:15].tolist() == [1.0] * 15 and f[15] == pytest.approx(1 + 0.5 * math.log(2)) and f[30] == f[15]
    assert f[31] == pytest.approx(1 + 0.5 * math.log(3))


def test_the_state_scan_goes_on_from_a_carried_state_and_forgets_by_its_decay():
    g = torch.Generator().manual_seed(0)
    t, nh, dk, dv = 12, 2, 3, 4
    q, k, a = (torch.randn(t, nh, dk, generator=g, dtype=F64) for _ in range(3))
    a = torch.sigmoid(a)
    v = torch.randn(t, nh, dv, generator=g, dtype=F64)
    whole, last = P.decayed_state_scan(q, k, v, a)
    head, s = P.decayed_state_scan(q[:5], k[:5], v[:5], a[:5])
    tail, s2 = P.decayed_state_scan(q[5:], k[5:], v[5:], a[5:], s)
    assert torch.allclose(torch.cat([head, tail]), whole, atol=1e-12) and torch.allclose(s2, last, atol=1e-12)
    # closed form: o_t = sum_j (q_t * prod_{j < i <= t} a_i) . k_j v_j
    for tt in (0, 4, 11):
        want = torch.zeros(nh, dv, dtype=F64)
        for j in range(tt + 1):
            w = (q[tt] * a[j + 1 : tt + 1].prod(0) * k[j]).sum(-1)
            want += w[:, None] * v[j]
        assert torch.allclose(whole[tt], want, atol=1e-10)
    # a decay of zero in every channel leaves only the current token
    o, _ = P.decayed_state_scan(q, k, v, torch.zeros_like(a))
    assert torch.allclose(o[7], (q[7] * k[7]).sum(-1)[:, None] * v[7], atol=1e-12)


def test_the_router_takes_the_largest_logits_and_weighs_them_among_themselves():
    w = {"m.router": torch.eye(4, dtype=F64), "m.router.b": torch.tensor([0.0, 0.0, 0.5, 0.0], dtype=F64)}
    idx, weight, _ = P.route(torch.tensor([[1.0, 3.0, 2.0, -1.0]], dtype=F64), w, "m.", 2)
    assert idx.tolist() == [[1, 2]]
    assert weight[0].tolist() == pytest.approx(torch.softmax(torch.tensor([3.0, 2.5], dtype=F64), 0).tolist())


# ----------------------------------------------------------------------------- the engine's bookkeeping
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuttings_agree_with_plain(models, emulated, name):
    cfg = NM.CONFIGS[name][0]
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
    cfg = NM.CONFIGS[name][0]
    reqs = H.make_requests(cfg["vocab"], [23, 9, 37, 30, 14, 26, 3, 19], seed=3)
    ref = plain_rows(models[name], reqs)
    trace = H.trace_mixed(reqs, seed=1, max_live=3, decode_tail=5)
    need = H.max_live_tokens(trace, round_to=4)
    eng = Engine.from_dir(models[name], dtype="float32", device="cpu", page_size=4, max_tokens=need, max_requests=3)
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, 1e-5, name)
    assert max(len(r["entries"]) for r in trace) == 3          # eight requests went through three state slots


def test_the_residual_stream_after_every_layer(models, emulated):
    """A model cut after layer n is the same model with n entries in its list of layers: the plain model's stream
    after each layer gives that model's logits."""
    cfg, seed, rows, rank = NM.CONFIGS["A"]
    tokens = H.make_requests(cfg["vocab"], [19], seed=2)["r0"]
    c, w = P.read_model(models["A"])
    streams = []
    full = P.forward(c, w, tokens, streams)
    assert len(streams) == 2 and streams[0].shape == (19, 64)
    again = P.soft_cap(P.layer_norm(streams[-1], w["final.norm"], w["final.norm.b"], 1e-6) @ w["head"].T, 8.0)
    assert torch.equal(again, full)
    eng = Engine.from_dir(models["A"], dtype="float32", device="cpu", page_size=4, max_tokens=64, max_requests=1)
    H.assert_rows_match(H.replay(eng, H.trace_whole({"r0": tokens})), {"r0": full}, 1e-5, "streams")


def test_each_branch_mixer_also_stands_alone_in_a_layer(emulated):
    """A model described by hand: the attention with its distance bias alone in one layer (its output bias joins the
    product there), the linear attention alone in the next; against the plain mechanisms."""
    from easy_gpt.cpp_amd.parts import LayerSpec, ModelSpec, PartSpec, RunSpec

    width, vocab, eps = 48, 50, 1e-5
    norm = lambda prefix, name: PartSpec("layernorm", dict(eps=eps, name=name, bias_name=name + ".b"), prefix=prefix)
    left = dict(heads=3, kv_heads=1, dim=8, vdim=12, scale=0.3, bias_max=7, q_temp=dict(coef=0.5, every=3))
    right = dict(heads=2, dim=5, vdim=9, tau=2.0)
    spec = ModelSpec(
        hidden_size=width, vocab_size=vocab, max_position=1 << 20,
        embedding=PartSpec("token_embedding_scaled", dict(scale=2.0, name="embed")),
        layers=(
            LayerSpec("pre_norm_mixer_only", PartSpec("distance_bias_attention", dict(
                n_heads=3, n_kv_heads=1, key_dim=8, value_dim=12, scale=0.3, eps=eps, bias_far=7, bias_rows=6, query_growth=(0.5, 3)),
                prefix="a."), None, {"mixer": norm("a.", "n")}),
            LayerSpec("pre_norm_mixer_only", PartSpec("gated_linear_attention", dict(
                n_heads=2, key_dim=5, value_dim=9, tau=2.0, eps=eps, decay_rank=3), prefix="b."), None, {"mixer": norm("b.", "n")}),
        ),
        run_order=(RunSpec(0, cache=0), RunSpec(1, state=0)),
        final_norm=norm("", "fn"), output_head=PartSpec("linear_head", dict(tied=False, name="head")),
    )
    model = build_model(spec)
    g = torch.Generator().manual_seed(3)
    w = {}
    for ps in model.param_specs():
        t = torch.randn(ps.shape, generator=g) * (0.3 if len(ps.shape) > 1 else 0.5)
        if ps.role == "norm_scale":
            t = 1.0 + 0.2 * t
        if ps.name == "b.a2.b":
            t = t + 1.5
        w[ps.name] = t.to(torch.bfloat16).to(torch.float32)
    model.load(lambda name: w[name], torch.float32, "cpu")
    eng = Engine(model, page_size=4, max_tokens=64, max_requests=2)
    tokens = H.make_requests(vocab, [21], seed=4)["r0"]
    w64 = {k: v.to(F64) for k, v in w.items()}
    x = w64["embed"][torch.tensor(tokens)] * 2.0
    x = x + P.biased_attention(P.layer_norm(x, w64["a.n"], w64["a.n.b"], eps), w64, "a.", left, eps)
    x = x + P.gated_linear_attention(P.layer_norm(x, w64["b.n"], w64["b.n.b"], eps), w64, "b.", right, eps)
    want = P.layer_norm(x, w64["fn"], w64["fn.b"], eps) @ w64["head"].T
    for trace in (H.trace_whole({"r0": tokens}), H.trace_portions({"r0": tokens})):
        H.assert_rows_match(H.replay(eng, trace), {"r0": want}, 1e-5, "branches alone")
