"""Pekasun on the CPU: configuration and registry, the model's description (layers that run on another layer's
weights), tensor names, the cache manager's kept first pages, and the engine's bookkeeping with the tests' slow
stand-in for the kernels against the plain implementation (tests/plain_pekasun.py)."""
import copy
import json
import os

import pytest
import torch

import helpers as H
import pekasun_models as PM
import plain_pekasun as P
from emulated_kernels import EmulatedKernels
from plain_cache import PlainCacheManager
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.cache import CacheManager
from easy_gpt.cpp_amd.config import ConfigError, PekasunConfig, resolve_architecture
from easy_gpt.cpp_amd.engine import Engine
from easy_gpt.cpp_amd.parts import CacheNeed, build_model
from easy_gpt.cpp_amd.weights import WeightsError


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    return {name: PM.write_model(str(tmp_path_factory.mktemp(f"pekasun_{name}")), cfg, seed)
            for name, (cfg, seed) in PM.CONFIGS.items()}


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
    arch = resolve_architecture(PM.CONFIG_B)
    assert arch.name == "Pekasun"
    cfg = PekasunConfig.from_dict(PM.CONFIG_B)
    assert (cfg.vocab, cfg.width, cfg.eps, len(cfg.layers)) == (257, 96, 1e-5, 5)
    a, l = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.keep_first, a.scale) == ("attention", 3, 3, 32, 16, 7, 1, 0.3)
    assert (l.kind, l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank, l.window) == ("latent_attention", 1, 8, 16, 8, 24, 33)
    assert (l.rotation.base, l.rotation.dims, l.rotation.factor) == (500.0, 12, None)
    assert cfg.layers[1].ff is None and cfg.layers[2].ff == 112
    assert cfg.layers[3].mixer.rotation.factor == 8.0 and cfg.layers[3].mixer.rotation.slow == 1.0
    assert PekasunConfig.from_dict(PM.CONFIG_C).layers[2].mixer.window is None


@pytest.mark.parametrize("edit, key", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=2), "kv_heads"),
    (lambda c: c["layers"][0].update(type="mamba"), "mamba"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][2]["mlp"].update(kind="experts"), "kind"),
    (lambda c: c["layers"][4].update(weights_of=4), "weights_of"),
    (lambda c: c["layers"][4].update(weights_of=2), "sizes"),
])
def test_a_wrong_configuration_is_refused_by_name(edit, key):
    cfg = copy.deepcopy(PM.CONFIG_B)
    edit(cfg)
    with pytest.raises(ConfigError, match=key):
        PekasunConfig.from_dict(cfg)


def test_a_layer_on_another_layers_weights_is_a_second_run_with_a_cache_of_its_own():
    arch = resolve_architecture(PM.CONFIG_A)
    spec = arch.build_spec(arch.config_class.from_dict(PM.CONFIG_A))
    assert len(spec.layers) == 2                                   # only the layers with tensors
    assert [(r.layer, r.cache) for r in spec.run_order] == [(0, 0), (1, 1), (0, 2), (1, 3)]
    model = build_model(spec)
    names = {s.name: s.shape for s in model.param_specs()}
    assert names["embed"] == (300, 64) and names["embed.norm"] == () and names["final.norm"] == () and names["head"] == (300, 64)
    assert names["l0.norm1"] == () and names["l0.mix.q"] == (2 * 24, 64) and names["l0.mix.dkv"] == (48, 64)
    assert names["l0.mix.dkv.norm"] == (40,) and names["l0.mix.uk"] == (32, 40) and names["l0.mix.uv"] == (48, 40)
    assert names["l0.mix.sink"] == (2,) and names["l0.mix.g"] == (48, 64) and names["l0.mix.o"] == (64, 48)
    assert names["l1.mix.q"] == (64, 64) and names["l1.mix.k"] == (32, 64) and names["l1.mix.v"] == (64, 64)
    assert names["l1.mix.q.norm"] == (16,) and names["l1.mix.k.norm"] == (16,) and names["l1.mix.o"] == (64, 128)
    assert names["l1.mlp.gate"] == (96, 64) and names["l1.mlp.down"] == (64, 96)
    assert not any(n.startswith(("l2.", "l3.")) for n in names)
    # two groups of caches: the latent layers' (window 20) and the attention layers' (window 12, three kept tokens)
    needs = sorted((g.need.window, g.need.keep_first, g.cache_ids) for g in model.cache_groups)
    assert needs == [(12, 3, (1, 3)), (20, 0, (0, 2))]


def test_a_missing_tensor_is_named(models, tmp_path, emulated):
    cfg, seed = PM.CONFIGS["A"]
    d = PM.write_model(str(tmp_path / "m"), cfg, seed, change=lambda w: w.pop("l1.mix.k.norm"))
    with pytest.raises(WeightsError, match="l1.mix.k.norm"):
        Engine.from_dir(d, dtype="float32", device="cpu", page_size=4, max_tokens=64)


# ----------------------------------------------------------------------------- kept first pages
@pytest.mark.parametrize("page_size, window, keep", [(4, 6, 3), (4, 5, 9), (16, 16, 1), (2, 3, 2), (8, 8, 0)])
def test_pages_of_kept_first_tokens_are_never_given_back(page_size, window, keep):
    need = CacheNeed.keys_and_values(1, 8, window, keep_first=keep)
    pages = 64
    real, plain = CacheManager([need], page_size, pages, 2), PlainCacheManager([need], page_size, pages, 2)
    a, b = real.admit("a"), plain.admit("a")
    n = 0
    for count in [1, 2, 7, 1, 1, 13, 2, 1, 30, 1, 1, 1, 5]:
        real.reserve(a, count)
        plain.reserve(b, count)
        real.commit(a, count)
        plain.commit(b, count)
        n += count
        real.check()
        assert a.tables[0] == b.tables[0]
        table = a.tables[0]
        first_needed = max(0, n - window + 1)
        for idx, page in enumerate(table):
            holds_kept = idx * page_size < keep
            holds_window = (idx + 1) * page_size > first_needed
            assert (page >= 0) == (holds_kept or holds_window), (n, idx, table)
    real.release(a)
    assert real.free_pages() == [pages]


# ----------------------------------------------------------------------------- the engine's bookkeeping
@pytest.mark.parametrize("name", ["A", "B", "C", "E", "F"])
def test_cuttings_agree_with_plain(models, emulated, name):
    cfg = PM.CONFIGS[name][0]
    reqs = H.make_requests(cfg["vocab"], [5, 41, 1, 23], seed=11)
    ref = plain_rows(models[name], reqs)
    for page_size, trace in [(4, H.trace_whole(reqs)), (16, H.trace_last_decoded(reqs, 9)), (3, H.trace_portions(reqs))]:
        eng = Engine.from_dir(models[name], dtype="float32", device="cpu", page_size=page_size, max_tokens=64, max_requests=2)
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(v) for v in reqs.values())
        H.assert_rows_match(rows, ref, 1e-5, f"{name} page {page_size}")
        assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("name", ["A", "B"])
def test_mixed_batches_with_page_reuse(models, emulated, name):
    cfg = PM.CONFIGS[name][0]
    reqs = H.make_requests(cfg["vocab"], [23, 9, 37, 30, 14, 26], seed=3)
    ref = plain_rows(models[name], reqs)
    trace = H.trace_mixed(reqs, seed=1, decode_tail=5)
    need = H.max_live_tokens(trace, round_to=4)
    eng = Engine.from_dir(models[name], dtype="float32", device="cpu", page_size=4, max_tokens=need, max_requests=4)
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, 1e-5, name)
    assert max(len(r["entries"]) for r in trace) >= 3
    assert all(pool.high_water <= pool.num_pages for pool in eng.cache.pools)


def test_the_residual_stream_after_every_layer_run(models, emulated):
    """The plain model's stream after each run, against the engine's: a model cut after run n is the same model
    with n entries in its list of layers."""
    cfg, seed = PM.CONFIGS["A"]
    tokens = H.make_requests(cfg["vocab"], [19], seed=2)["r0"]
    c, w = P.read_model(models["A"])
    _, streams = P.forward(c, w, tokens, return_layers=True)
    assert streams.shape == (4, 19, 64)
    # the last stream gives the logits
    logits = P.scalar_norm(streams[-1], w["final.norm"], 1e-6) @ w["head"].T
    eng = Engine.from_dir(models["A"], dtype="float32", device="cpu", page_size=4, max_tokens=64, max_requests=1)
    rows = H.replay(eng, H.trace_whole({"r0": tokens}))
    H.assert_rows_match(rows, {"r0": logits}, 1e-5, "streams")


# ----------------------------------------------------------------------------- the attention kernel's shape rule
def test_the_window_attention_rule_returns_what_the_kernel_takes():
    """Over a grid of sizes: row tiles of 4 or 8, 1 to 64 splits, LDS within 160 KB; None exactly where a size is not
    covered (then the general kernel runs)."""
    from easy_gpt.cpp_amd.kernels.hip import HipKernels

    rule = HipKernels._window_attention_shape
    for elem in (2, 4):
        for dk, dv in [(16, 32), (64, 64), (160, 128), (256, 192), (256, 256), (72, 16), (40, 24), (264, 64), (64, 272), (12, 16)]:
            for t, b, max_q in [(1, 1, 1), (8, 8, 1), (64, 64, 1), (300, 3, 200), (2048, 1, 2048), (40000, 2, 32000)]:
                for nq, nkv in [(14, 2), (16, 1), (3, 3)]:
                    for window, keep in [(0, 0), (1024, 4), (7, 0)]:
                        shape = rule(t, b, nq, nkv, dk, dv, 16, window, keep, max_q, 4096, elem)
                        covered = dk % (16 // elem) == 0 and dk <= 256 and dv % 16 == 0 and dv <= 256
                        assert (shape is not None) == covered, (elem, dk, dv)
                        if shape is None:
                            continue
                        tiles, splits = shape
                        assert tiles in (4, 8) and 1 <= splits <= 64
                        chunk, e = (64, 8) if elem == 2 else (32, 4)
                        krow = -(-dk // (4 * e)) * 4 * e + e
                        dv_tiles = next(n for n in (2, 4, 6, 8, 12, 16) if n * 16 >= dv)
                        assert ((16 * tiles + chunk) * krow + dv_tiles * 16 * (chunk + e)) * elem <= 160 * 1024
            assert rule(8, 8, 4, 2, dk, dv, 40, 0, 0, 1, 512, elem) is None          # pages that are no multiple of 16
