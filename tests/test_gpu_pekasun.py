"""Pekasun models on the GPU against the plain implementation (tests/plain_pekasun.py): every way of cutting
requests into steps, in float32 and bfloat16, on small configurations that differ in every size; windows and kept
first tokens passed in prompts and in decoding; pages used again; long decoding; generation through the entry
point; bin/trace_run as a subprocess."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
import pekasun_models as PM
import plain_pekasun as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# as fractions of the largest logit: float32 is the rounding of float32 sums in another order; bfloat16 rounds
# activations between kernels (never the stream, statistics, scores or partial sums)
TOL = {"float32": 3e-5, "bfloat16": 4e-2}

# a configuration whose sizes are multiples of 16 throughout and whose windows are longer than a page
CONFIG_D = {
    "architecture": "Pekasun", "vocab": 523, "width": 256, "norm": {"eps": 1e-5},
    "layers": [
        PM.layer(PM.attention(8, 2, 64, 64, 80, 4, 0.125), 320),
        PM.layer(PM.latent(4, 64, 32, 64, 96, 48, 0.1, base=50000.0,
                           scaling={"factor": 2.0, "original": 128, "fast": 32.0, "slow": 1.0}), 320),
        PM.layer(PM.attention(8, 2, 64, 64, 80, 4, 0.125), 320, weights_of=0),
        PM.layer(PM.latent(2, 32, 32, 128, 128, 100, 0.12, base=10000.0), 192),
    ],
}
ALL = dict(PM.CONFIGS, D=(CONFIG_D, 8))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    return {name: PM.write_model(str(tmp_path_factory.mktemp(f"pekasun_{name}")), cfg, seed) for name, (cfg, seed) in ALL.items()}


@pytest.fixture(autouse=True)
def product_kernels():
    from easy_gpt.cpp_amd import kernels

    kernels.use_backend(None)
    assert kernels.backend().name == "hip-gfx950"


def engine(model_dir, dtype, **kw):
    from easy_gpt.cpp_amd.engine import Engine

    return Engine.from_dir(model_dir, dtype=dtype, device="cuda:0", **kw)


def plain_rows(model_dir, reqs):
    cfg, w = P.read_model(model_dir)
    return {rid: P.forward(cfg, w, ids) for rid, ids in reqs.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
def test_every_cutting_agrees_with_plain(models, name, dtype):
    cfg = ALL[name][0]
    reqs = H.make_requests(cfg["vocab"], [150, 1, 47, 2, 96], seed=21)
    ref = plain_rows(models[name], reqs)
    cuttings = {"whole": H.trace_whole(reqs), "last decoded": H.trace_last_decoded(reqs, 40), "portions": H.trace_portions(reqs),
                "mixed": H.trace_mixed(reqs, seed=5, decode_tail=20)}
    for what, trace in cuttings.items():
        for page_size in (16, 32, 48) if what == "whole" else (16, 48) if what == "mixed" else (16,):
            need = H.max_live_tokens(trace, 64)
            eng = engine(models[name], dtype, page_size=page_size, max_tokens=need, max_requests=4)
            rows = H.replay(eng, trace)
            assert len(rows) == sum(len(v) for v in reqs.values())
            H.assert_rows_match(rows, ref, TOL[dtype], f"{name} {dtype} {what} pages of {page_size}")
            assert eng.cache.free_pages() == [p.num_pages for p in eng.cache.pools]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("use_graphs", [True, False])
def test_mixed_batches_with_pages_and_slots_used_again(models, dtype, use_graphs):
    """Ten requests through four slots and a pool that holds a third of their tokens; with the steps replayed from
    graphs and kernel by kernel."""
    name = "A"
    cfg = ALL[name][0]
    reqs = H.make_requests(cfg["vocab"], [70, 23, 110, 64, 37, 90, 5, 130, 49, 81], seed=33)
    ref = plain_rows(models[name], reqs)
    trace = H.trace_mixed(reqs, seed=9, decode_tail=24)
    need = H.max_live_tokens(trace, 16)
    eng = engine(models[name], dtype, page_size=16, max_tokens=need, max_requests=4, use_graphs=use_graphs)
    rows = H.replay(eng, trace)
    H.assert_rows_match(rows, ref, TOL[dtype], f"mixed {dtype}")
    assert sum(-(-len(v) // 16) for v in reqs.values()) > 2 * eng.cache.pools[0].num_pages
    assert max(len(r["entries"]) for r in trace) == 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_long_decoding_passes_every_window_and_gives_pages_back(models, name, dtype):
    cfg = ALL[name][0]
    reqs = H.make_requests(cfg["vocab"], [260], seed=44)
    ref = plain_rows(models[name], reqs)
    eng = engine(models[name], dtype, page_size=16, max_tokens=320, max_requests=2)
    rows = H.replay(eng, H.trace_last_decoded(reqs, 257))         # three tokens as a prompt, then one by one
    H.assert_rows_match(rows, ref, TOL[dtype], f"long decoding {name} {dtype}")
    assert len(rows) == 260
    # a windowed group held few pages at the end
    eng.add_request("again")
    from easy_gpt.cpp_amd.engine import StepEntry

    eng.step([StepEntry("again", reqs["r0"], [259])])
    windowed = [g for g, need in enumerate(eng.cache.groups) if need.window is not None and need.window < 100]
    tables = eng.cache.requests["again"].tables
    assert windowed and all(sum(p >= 0 for p in tables[g]) < len(tables[g]) for g in windowed)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_longer_than_any_graph_in_one_step(models, dtype):
    """2,600 tokens in one step (steps beyond 2,048 tokens run kernel by kernel), then tokens one by one."""
    name = "D"
    cfg = ALL[name][0]
    reqs = H.make_requests(cfg["vocab"], [2610], seed=88)
    ref = plain_rows(models[name], reqs)
    eng = engine(models[name], dtype, page_size=16, max_tokens=2624, max_requests=1)
    rows = H.replay(eng, H.trace_last_decoded(reqs, 10))
    assert len(rows) == 2610
    H.assert_rows_match(rows, ref, TOL[dtype], f"long prompt {dtype}")


def test_a_batch_gives_each_request_what_it_gets_alone(models):
    """float32: the logits of a request in a batch of unequal requests against the same request alone."""
    name = "C"
    cfg = ALL[name][0]
    reqs = H.make_requests(cfg["vocab"], [90, 7, 33, 64], seed=55)
    from easy_gpt.cpp_amd.engine import StepEntry

    eng = engine(models[name], "float32", page_size=16, max_tokens=512, max_requests=4)
    for rid in reqs:
        eng.add_request(rid)
    together = eng.step([StepEntry(rid, ids, [len(ids) - 1]) for rid, ids in reqs.items()]).cpu().clone()
    scale = float(together.abs().max())
    for i, (rid, ids) in enumerate(reqs.items()):
        eng.finish(rid)
        eng.add_request(rid)
        alone = eng.step([StepEntry(rid, ids, [len(ids) - 1])]).cpu()
        assert float((alone[0] - together[i]).abs().max()) <= 2e-6 * scale, rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(models, dtype):
    from easy_gpt.cpp_amd.generate import LLM

    name = "A"
    cfg = ALL[name][0]
    prompts = list(H.make_requests(cfg["vocab"], [5, 40, 17, 1], seed=66).values())
    llm = LLM(models[name], dtype=dtype, cache_tokens=1024, prefill_chunk=16)
    outs = llm.generate(prompts, max_new_tokens=24, greedy=True, ignore_eos=True)
    c, w = P.read_model(models[name])
    for prompt, out in zip(prompts, outs):
        assert len(out) == 24
        logits = P.forward(c, w, prompt + out)
        for i, tok in enumerate(out):
            row = logits[len(prompt) + i - 1]
            gap = float(row.max() - row[tok])
            assert gap <= (1e-4 if dtype == "float32" else 5e-2) * float(row.abs().max()), (dtype, i, tok, gap)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_as_a_subprocess(models, tmp_path, dtype):
    name = "B"
    cfg = ALL[name][0]
    reqs = H.make_requests(cfg["vocab"], [70, 23, 110, 37], seed=77)
    ref = plain_rows(models[name], reqs)
    trace = H.trace_mixed(reqs, seed=4, decode_tail=32, want_all=False)
    out_dir = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", models[name], "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(H.max_live_tokens(trace, 64))]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    rows, fed = {}, {}
    for rec in trace:
        p.stdin.write(json.dumps(rec) + "\n")
        p.stdin.flush()
        assert p.stdout.readline().strip() == f"done {rec['step']}"
        wanted = sum(len(e["want"]) for e in rec["entries"])
        if wanted:
            data = np.fromfile(os.path.join(out_dir, f"{rec['step']}.f32"), dtype="<f4").reshape(wanted, cfg["vocab"])
            r = 0
            for e in rec["entries"]:
                for w in e["want"]:
                    rows[(e["id"], fed.get(e["id"], 0) + w)] = torch.from_numpy(data[r].copy())
                    r += 1
        for e in rec["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    assert len(rows) > 60
    H.assert_rows_match(rows, ref, TOL[dtype], f"trace_run {dtype}")


def test_the_command_line_generates_with_a_pekasun_folder(models, tmp_path):
    """bin/easy_llm on a Pekasun folder, greedy in float32: the tokens are the plain model's (the weights of the tests
    leave no near-ties), from a prompt on the command line and from a prompt file in portions of 16."""
    name = "A"
    prompt = [5, 17, 3, 250, 9, 44, 1]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "easy_llm"), "--model", models[name], "--dtype", "float32", "--greedy",
           "--ignore-eos", "--max-new-tokens", "12"]
    p = subprocess.run(cmd + [" ".join(map(str, prompt))], capture_output=True, text=True, timeout=110, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    c, w = P.read_model(models[name])
    out = [int(t) for t in p.stdout.split()]
    assert len(out) == 12
    logits = P.forward(c, w, prompt + out)
    for i, tok in enumerate(out):
        row = logits[len(prompt) + i - 1]
        assert float(row.max() - row[tok]) <= 1e-4 * float(row.abs().max()), (i, tok)
    (tmp_path / "prompts.txt").write_text("3 4 5\n" + " ".join(str(7 + i % 90) for i in range(50)) + "\n")
    p = subprocess.run(cmd + ["-f", str(tmp_path / "prompts.txt"), "--prefill-chunk", "16", "--cache-tokens", "512"],
                       capture_output=True, text=True, timeout=110, cwd=str(tmp_path),
                       env=dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", "")))
    assert p.returncode == 0, p.stderr[-2000:]
    lines = (tmp_path / "prompts_output.txt").read_text().splitlines()
    assert len(lines) == 2 and all(len(ln.split()) == 12 for ln in lines)
