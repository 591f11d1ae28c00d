"""The kernels that the Nebanex design added, each alone against the plain functions of tests/plain_nebanex.py: the
scaled embedding, the layer norm fused with the residual addition, the mean of two normed branches, the tanh cap,
the norm over a whole projection with the query factor and the store into pages, attention with a bias by head and
distance (both kernels), the per-head norm with its SiLU gate, the decays, the state scan, and the mixture of
experts.  Where random inputs would hide a fault (one far key among hundreds, the distances at a bucket's two
edges, a token far back in the state), the inputs are made so that it shows."""
import math

import pytest
import torch

import plain_nebanex as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def k():
    from easy_gpt.cpp_amd import kernels

    kernels.use_backend(None)
    return kernels.backend()


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def close(got, want, dtype, what="", tol=None):
    got, want = got.detach().to("cpu", F64), want.to(F64)
    err = float((got - want).abs().max())
    scale = max(float(want.abs().max()), 1e-6)
    assert err <= (tol or TOL[dtype]) * scale, f"{what}: max |diff| {err:.3e} against scale {scale:.3f}"


def i32(*v):
    return torch.tensor(list(v), dtype=torch.int32, device=DEV)


def added(o):
    """What a scan leaves: partial sums [splits, T, W] over ranges of the key channels, added."""
    return o.sum(0) if o.dim() == 3 else o


# ----------------------------------------------------------------------------- stream operations
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_a_factor(k, dtype):
    table = rnd(37, 100, seed=1, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32)
    out = torch.empty((5, 100), dtype=torch.float32, device=DEV)
    k.embed_scaled(ids.to(DEV), table.to(DEV), 12.5, out)
    close(out, table.to(F64)[ids.long()] * 12.5, torch.float32, "scaled embedding")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden, splits", [(100, 0), (256, 3), (4100, 1)])
def test_layer_norm_with_the_addition_into_the_stream(k, dtype, hidden, splits):
    t = 9
    h = rnd(t, hidden, seed=2, scale=3.0) + 40.0                    # a mean far larger than the deviations
    delta = rnd(max(splits, 1), t, hidden, seed=3)
    w, b = (rnd(hidden, seed=4) + 1).to(dtype), rnd(hidden, seed=5).to(dtype)
    given = delta.to(DEV) if splits else delta[0].to(dtype).to(DEV)
    total = delta.sum(0) if splits else delta[0].to(dtype).float()
    hd = h.clone().to(DEV)
    out = torch.empty((t, hidden), dtype=dtype, device=DEV)
    k.add_layernorm(hd, given, None, w.to(DEV), b.to(DEV), 1e-5, out)
    close(hd, h.to(F64) + total.to(F64), torch.float32, "the stream after the addition", 1e-6)
    want = P.layer_norm(h.to(F64) + total.to(F64), w.to(F64), b.to(F64), 1e-5)
    close(out, want, dtype, "layer norm")
    # selected rows: the stream stays as it is
    before = hd.clone()
    rows = i32(7, 0, 3)
    out = torch.empty((3, hidden), dtype=dtype, device=DEV)
    k.add_layernorm(hd, given, rows, w.to(DEV), None, 1e-5, out)
    assert torch.equal(hd, before)
    x = before.cpu().to(F64)[[7, 0, 3]] + total.to(F64)[[7, 0, 3]]
    close(out, P.layer_norm(x, w.to(F64), torch.zeros(hidden, dtype=F64), 1e-5), dtype, "rows, no bias")
    # nothing to add
    out = torch.empty((t, hidden), dtype=dtype, device=DEV)
    k.add_layernorm(hd, None, None, w.to(DEV), b.to(DEV), 1e-5, out)
    close(out, P.layer_norm(before.cpu().to(F64), w.to(F64), b.to(F64), 1e-5), dtype, "no delta")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [100, 1024])
def test_the_mean_of_two_normed_branches(k, dtype, hidden):
    t = 7
    a, b = rnd(2, t, hidden, seed=6, scale=2.0), rnd(t, hidden, seed=7, scale=0.1).to(dtype)
    ba, wa, wb = rnd(hidden, seed=8).to(dtype), (rnd(hidden, seed=9) + 1).to(dtype), (rnd(hidden, seed=10) + 1).to(dtype)
    out = k.normed_pair_mean(a.to(DEV), b.to(DEV), ba.to(DEV), None, wa.to(DEV), wb.to(DEV), 1e-6, 0.5)
    assert out.shape == (1, t, hidden) and out.dtype == torch.float32
    want = 0.5 * (P.rms_norm(a.sum(0).to(F64) + ba.to(F64), wa.to(F64), 1e-6) + P.rms_norm(b.to(F64), wb.to(F64), 1e-6))
    close(out[0], want, torch.float32, "normed pair")


def test_the_cap_on_logits(k):
    x = torch.tensor([[-1000.0, -30.0, -1.0, 0.0, 1e-3, 5.0, 29.0, 31.0, 4000.0]], device=DEV)
    want = P.soft_cap(x.cpu().to(F64), 30.0)
    k.tanh_cap(x, 30.0)
    close(x, want, torch.float32, "cap")
    assert float(x.abs().max()) <= 30.0


# ----------------------------------------------------------------------------- the left mixer's preparation
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv, splits, every", [(4, 2, 16, 32, 0, 4), (3, 3, 12, 20, 3, 1), (2, 1, 200, 8, 1, 0), (8, 1, 64, 48, 2, 96), (40, 8, 96, 32, 1, 5)])
def test_norms_over_the_whole_projection_the_query_factor_and_the_store(k, dtype, nq, nkv, dk, dv, splits, every):
    t, ps, eps, coef, extra = 13, 4, 1e-3, 0.4, 9
    used = (nq + nkv) * dk + nkv * dv
    proj = rnd(max(splits, 1), t, used + extra, seed=2, scale=2.0)
    whole = proj.sum(0) if splits else proj[0].to(dtype).to(F64)
    given = proj.to(DEV) if splits else proj[0].to(dtype).to(DEV)
    bias = rnd(used, seed=11, scale=0.5).to(dtype)
    qw, kw = (rnd(nq * dk, seed=3) + 1).to(dtype), (rnd(nkv * dk, seed=4) + 1).to(dtype)
    positions = torch.tensor([0, 1, 2, 3, 4, 6, 7, 8, 126, 127, 128, 255, 100000], dtype=torch.int32)
    slots = torch.randperm(6 * ps, generator=torch.Generator().manual_seed(5))[:t].to(torch.int32)
    k_cache = torch.zeros((6, nkv, ps, dk), dtype=dtype, device=DEV)
    v_cache = torch.zeros((6, nkv, dv, ps), dtype=dtype, device=DEV)
    q_out = torch.empty((t, nq * dk), dtype=dtype, device=DEV)
    k.whole_norm_store(given, bias.to(DEV), q_out, qw.to(DEV), kw.to(DEV), eps, positions.to(DEV), coef, every,
                       slots.to(DEV), k_cache, v_cache, nq, nkv, dk, dv, ps)
    x = whole.to(F64)[:, :used] + bias.to(F64)
    q = P.rms_norm(x[:, : nq * dk], qw.to(F64), eps)
    if every:
        q = q * P.query_factor(positions.tolist(), coef, every)[:, None]
    kk = P.rms_norm(x[:, nq * dk : (nq + nkv) * dk], kw.to(F64), eps).view(t, nkv, dk)
    vv = x[:, (nq + nkv) * dk :].view(t, nkv, dv)
    close(q_out, q, dtype, "queries")
    page, off = (slots // ps).long(), (slots % ps).long()
    close(k_cache.cpu()[page, :, off, :], kk, dtype, "keys in their pages")
    close(v_cache.cpu()[page, :, :, off], vv, dtype, "values in their pages")


# ----------------------------------------------------------------------------- attention with a bias by distance
def paged(keys, values, page_size, dtype, seed, spare=3):
    n, nkv, dk = keys.shape
    dv = values.shape[2]
    n_pages = -(-n // page_size)
    order = torch.randperm(n_pages + spare, generator=torch.Generator().manual_seed(seed))[:n_pages]
    k_cache = torch.full((n_pages + spare, nkv, page_size, dk), float("nan"), dtype=dtype)
    v_cache = torch.full((n_pages + spare, nkv, dv, page_size), float("nan"), dtype=dtype)
    for j in range(n):
        k_cache[order[j // page_size], :, j % page_size, :] = keys[j].to(dtype)
        v_cache[order[j // page_size], :, :, j % page_size] = values[j].to(dtype)
    return k_cache.to(DEV), v_cache.to(DEV), order.to(torch.int32).reshape(1, -1).to(DEV)


def plain_biased(q, keys, values, first_pos, scale, rel, far):
    """q [m, nq, dk] at positions first_pos.., keys [n, nkv, dk], values [n, nkv, dv], rel [rows, nq] -> [m, nq, dv]."""
    m, nq, _ = q.shape
    n, nkv, _ = keys.shape
    kh = keys.to(F64).repeat_interleave(nq // nkv, dim=1)
    vh = values.to(F64).repeat_interleave(nq // nkv, dim=1)
    s = torch.einsum("ihd,jhd->hij", q.to(F64), kh) * scale + P.distance_bias(n, rel.to(F64), far)[:, first_pos : first_pos + m]
    seen = torch.ones(n, n).tril().bool()[first_pos : first_pos + m]
    pr = torch.softmax(s.masked_fill(~seen, -math.inf), dim=-1)
    return torch.einsum("hij,jhd->ihd", pr, vh)


def run_biased(k, q, k_cache, v_cache, table, kv_len, page_size, scale, rel, far, dv):
    from easy_gpt.cpp_amd.parts.branch_mixers import distance_bias_table

    m, nq, dk = q.shape
    out = torch.empty((m, nq * dv), dtype=q.dtype, device=DEV)
    k.window_attention(q.reshape(m, nq * dk).to(DEV).contiguous(), out, k_cache, v_cache, table, i32(0), i32(m), i32(kv_len),
                       nq, k_cache.shape[1], dk, dv, page_size, scale, 0, 0, None, m, kv_len,
                       dist_bias=distance_bias_table(rel, far).to(DEV))
    return out.view(m, nq, dv)


SHAPES = [(4, 2, 16, 32, 8, 20), (3, 3, 12, 20, 6, 9), (4, 1, 64, 48, 12, 90), (8, 2, 128, 64, 32, 300), (2, 1, 40, 24, 4, 3),
          (1, 1, 256, 16, 10, 700)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv, rows, far", SHAPES)
def test_attention_with_a_distance_bias_whole_in_portions_and_token_by_token(k, dtype, nq, nkv, dk, dv, rows, far):
    n, ps, scale = 333, 16, 1.0 / math.sqrt(dk)
    keys, values = rnd(n, nkv, dk, seed=1, dtype=dtype), rnd(n, nkv, dv, seed=2, dtype=dtype)
    q = rnd(n, nq, dk, seed=3, scale=2.0, dtype=dtype)
    rel = rnd(rows, nq, seed=4, scale=3.0)
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=5)
    want = plain_biased(q, keys, values, 0, scale, rel, far)
    got = run_biased(k, q, k_cache, v_cache, table, n, ps, scale, rel, far, dv)
    close(got, want, dtype, "whole prompt")
    for first, m in [(0, 2), (2, 62), (64, 1), (65, 130), (195, 3), (198, 135), (331, 2), (100, 1), (332, 1)]:
        got = run_biased(k, q[first : first + m], k_cache, v_cache, table, first + m, ps, scale, rel, far, dv)
        close(got, want[first : first + m], dtype, f"portion at {first} of {m}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv, rows, far", [(2, 1, 16, 16, 8, 20), (2, 2, 12, 20, 14, 100), (4, 1, 64, 32, 12, 90), (2, 1, 32, 64, 6, 50)])
def test_every_bucket_of_the_distance_bias_starts_and_ends_where_it_should(k, dtype, nq, nkv, dk, dv, rows, far):
    """Queries of zero, so that the bias alone decides; one row of the table stands 30 above the others: the output is
    the mean of the values at exactly that row's distances.  A bucket that starts or ends one token off shows as a
    wrong mean."""
    n, ps = far + 75, 16
    keys, values = rnd(n, nkv, dk, seed=1, dtype=dtype), rnd(n, nkv, dv, seed=2, dtype=dtype)
    q = torch.zeros(n, nq, dk, dtype=dtype)
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=6)
    buckets = [P.distance_bucket(d, rows, far) for d in range(n)]
    for row in range(rows):
        rel = torch.zeros(rows, nq)
        rel[row, 0], rel[(row + 1) % rows, 1] = 30.0, 30.0
        want = plain_biased(q, keys, values, 0, 1.0, rel, far)
        got = run_biased(k, q, k_cache, v_cache, table, n, ps, 1.0, rel, far, dv)
        close(got, want, dtype, f"row {row}, whole prompt")
        # and for single tokens at the positions where the row's first and last distances come into view
        ds = [d for d in range(n) if buckets[d] == row]
        for p in sorted({min(ds), min(ds) + 1, min(max(ds), n - 2), min(max(ds) + 1, n - 1), n - 1}):
            got = run_biased(k, q[p : p + 1], k_cache, v_cache, table, p + 1, ps, 1.0, rel, far, dv)
            close(got, want[p : p + 1], dtype, f"row {row}, single token at {p}")
            if p >= min(ds):         # head 0 sees only the values at this row's distances
                mean = values[[j for j in range(p + 1) if buckets[p - j] == row]].to(F64)[:, 0].mean(0)
                close(got[0, 0], mean, dtype, f"row {row}: the mean over its distances at {p}", 5e-3 if dtype == torch.float32 else None)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv", [(4, 1, 64, 64), (2, 2, 24, 40)])
def test_one_far_key_among_nine_hundred_with_a_bias_against_it(k, dtype, nq, nkv, dk, dv):
    n, ps, rows, far = 900, 16, 8, 100
    keys, values = rnd(n, nkv, dk, seed=1, scale=0.3, dtype=dtype), rnd(n, nkv, dv, seed=2, dtype=dtype)
    q = rnd(n, nq, dk, seed=3, scale=0.3, dtype=dtype)
    keys[17] = q[-1, 0] * 40.0                       # the last query's first head finds key 17
    rel = torch.zeros(rows, nq)
    rel[rows - 1] = -4.0                             # the far row works against it, but not enough
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=7)
    want = plain_biased(q[-3:], keys, values, n - 3, 1.0, rel, far)
    assert float((want[-1, 0] - values[17, 0].to(F64)).abs().max()) < 0.05 * float(values[17, 0].abs().max())
    close(run_biased(k, q[-3:], k_cache, v_cache, table, n, ps, 1.0, rel, far, dv), want, dtype, "portion of three")
    close(run_biased(k, q[-1:], k_cache, v_cache, table, n, ps, 1.0, rel, far, dv), want[-1:], dtype, "single token")


def test_a_batch_of_unequal_requests_gets_what_each_gets_alone(k):
    from easy_gpt.cpp_amd.parts.branch_mixers import distance_bias_table

    dtype, nq, nkv, dk, dv, ps, rows, far = torch.float32, 4, 2, 32, 48, 16, 8, 30
    lens, news = [70, 5, 130, 33], [1, 5, 64, 2]
    rel = rnd(rows, nq, seed=9, scale=2.0)
    bias = distance_bias_table(rel, far).to(DEV)
    width = max(-(-n // ps) for n in lens)
    total_pages = sum(-(-n // ps) for n in lens)
    k_cache = torch.zeros((total_pages, nkv, ps, dk), dtype=dtype)
    v_cache = torch.zeros((total_pages, nkv, dv, ps), dtype=dtype)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    qs, wants, at = [], [], 0
    for b, (n, m) in enumerate(zip(lens, news)):
        keys, values = rnd(n, nkv, dk, seed=10 + b), rnd(n, nkv, dv, seed=20 + b)
        q = rnd(m, nq, dk, seed=30 + b, scale=2.0)
        for j in range(n):
            page = at + j // ps
            table[b, j // ps] = page
            k_cache[page, :, j % ps, :] = keys[j]
            v_cache[page, :, :, j % ps] = values[j]
        at += -(-n // ps)
        qs.append(q)
        wants.append(plain_biased(q, keys, values, n - m, 0.2, rel, far))
    q_all = torch.cat(qs).reshape(-1, nq * dk).to(DEV)
    out = torch.empty((q_all.shape[0], nq * dv), dtype=dtype, device=DEV)
    starts = [sum(news[:b]) for b in range(len(news))]
    k.window_attention(q_all, out, k_cache.to(DEV), v_cache.to(DEV), table.to(DEV), i32(*starts), i32(*news), i32(*lens), nq, nkv,
                       dk, dv, ps, 0.2, 0, 0, None, max(news), max(lens), dist_bias=bias)
    for b, (s, m) in enumerate(zip(starts, news)):
        close(out[s : s + m].view(m, nq, dv), wants[b], dtype, f"request {b}")


# ----------------------------------------------------------------------------- the right mixer
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dv, splits", [(2, 24, 0), (3, 100, 2), (1, 64, 1)])
def test_per_head_norm_with_the_silu_gate(k, dtype, heads, dv, splits):
    t, off, eps = 6, 5, 1e-5
    x = rnd(3, t, heads * dv, seed=1, scale=2.0) if splits == 2 else rnd(t, heads * dv, seed=1, scale=3.0)      # partial sums, or one tensor
    g = rnd(max(splits, 1), t, off + heads * dv + 3, seed=2)
    gate = g.sum(0) if splits else g[0].to(dtype).to(F64)
    w = (rnd(dv, seed=3) + 1).to(dtype)
    out = torch.empty((t, heads * dv), dtype=dtype, device=DEV)
    k.head_norm_gate(x.to(DEV), w.to(DEV), eps, g.to(DEV) if splits else g[0].to(dtype).to(DEV), off, out, heads, dv)
    gg = gate.to(F64)[:, off : off + heads * dv]
    want = P.rms_norm(added(x).to(F64).view(t, heads, dv), w.to(F64), eps).reshape(t, -1) * gg * torch.sigmoid(gg)
    close(out, want, dtype, "head norm and gate")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rank, channels, tau", [(5, 30, 1.0), (16, 96, 8.0), (1, 7, 4.0)])
def test_decays_from_the_low_rank_projection(k, dtype, rank, channels, tau):
    t, off = 9, 11
    low = rnd(2, t, off + rank + 2, seed=1, scale=2.0)
    w, b = rnd(channels, rank, seed=2, scale=3.0).to(dtype), rnd(channels, seed=3, scale=3.0).to(dtype)
    got = k.channel_decay(low.to(DEV), off, rank, w.to(DEV), b.to(DEV), tau)
    z = low.sum(0).to(F64)[:, off : off + rank] @ w.to(F64).T + b.to(F64)
    close(got, torch.sigmoid(z) ** (1.0 / tau), torch.float32, "decays", 1e-5)
    assert got.dtype == torch.float32 and float(got.min()) >= 0.0 and float(got.max()) <= 1.0


def scan_inputs(t, heads, dk, dv, seed, dtype, splits=1):
    width = 2 * heads * dk + heads * dv + 4
    proj = rnd(splits, t, width, seed=seed, scale=1.0 / math.sqrt(splits))
    decay = torch.sigmoid(rnd(t, heads * dk, seed=seed + 1) + 2.0)
    whole = proj.sum(0) if splits > 0 else None
    return proj, whole, decay, (3, 3 + heads * dk, 3 + 2 * heads * dk + 1)


def plain_scan(whole, decay, offs, heads, dk, dv, q_scale, state=None):
    t = whole.shape[0]
    q = whole[:, offs[0] : offs[0] + heads * dk].to(F64).view(t, heads, dk) * q_scale
    kk = whole[:, offs[1] : offs[1] + heads * dk].to(F64).view(t, heads, dk)
    v = whole[:, offs[2] : offs[2] + heads * dv].to(F64).view(t, heads, dv)
    return P.decayed_state_scan(q, kk, v, decay.to(F64).view(t, heads, dk), state)


@pytest.mark.parametrize("heads, dk, dv", [(2, 6, 100), (3, 10, 12), (2, 16, 24), (1, 36, 70), (2, 64, 80), (4, 32, 48), (2, 128, 128),
                                           (1, 160, 64), (1, 256, 16), (1, 300, 9)])
def test_the_state_scan_whole_and_cut_anywhere(k, heads, dk, dv):
    t, q_scale = 150, dk ** -0.5
    proj, whole, decay, offs = scan_inputs(t, heads, dk, dv, 3, torch.float32, splits=2)
    want, last = plain_scan(whole, decay, offs, heads, dk, dv, q_scale)
    states = torch.full((3, heads, dk, dv), float("nan"), device=DEV)
    fresh = torch.tensor([True], device=DEV)
    got = k.decayed_state_scan(proj.to(DEV), torch.float32, *offs, q_scale, decay.to(DEV), states, i32(1), fresh, i32(0), i32(t),
                               heads, dk, dv)
    close(added(got).view(t, heads, dv), want, torch.float32, "whole")
    close(states[1], last, torch.float32, "the state it leaves")
    assert torch.isnan(states[0]).all() and torch.isnan(states[2]).all()
    # the same tokens in portions of changing size, down to single tokens: the same bits
    again = torch.full((3, heads, dk, dv), float("nan"), device=DEV)
    outs, pos = [], 0
    for n in [1, 2, 7, 8, 9, 1, 1, 33, 2, 64, 3, 19]:
        part = proj[:, pos : pos + n].contiguous().to(DEV)
        outs.append(k.decayed_state_scan(part, torch.float32, *offs, q_scale, decay[pos : pos + n].contiguous().to(DEV), again, i32(2),
                                         torch.tensor([pos == 0], device=DEV), i32(0), i32(n), heads, dk, dv))
        pos += n
    assert pos == t
    assert torch.equal(torch.cat(outs, dim=-2), got) and torch.equal(again[2], states[1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_state_scan_takes_a_rounded_product_and_a_batch_of_unequal_requests(k, dtype):
    heads, dk, dv, q_scale = 2, 32, 48, 0.3
    lens = [40, 1, 17, 2]
    t = sum(lens)
    proj, _, decay, offs = scan_inputs(t, heads, dk, dv, 5, dtype)
    rounded = proj[0].to(dtype)
    slots, starts = [3, 0, 4, 1], [sum(lens[:b]) for b in range(len(lens))]
    before = rnd(6, heads, dk, dv, seed=9)
    states = before.clone().to(DEV)
    fresh = torch.tensor([True, False, False, True], device=DEV)
    got = k.decayed_state_scan(rounded.to(DEV), dtype, *offs, q_scale, decay.to(DEV), states, i32(*slots), fresh, i32(*starts),
                               i32(*lens), heads, dk, dv)
    for b, (s, n) in enumerate(zip(starts, lens)):
        start = None if bool(fresh[b]) else before[slots[b]].to(F64)
        want, last = plain_scan(rounded[s : s + n].to(F64), decay[s : s + n], offs, heads, dk, dv, q_scale, start)
        close(added(got)[s : s + n].view(n, heads, dv), want, torch.float32, f"request {b}")
        close(states[slots[b]], last, torch.float32, f"state of request {b}")
    assert torch.equal(states[2].cpu(), before[2]) and torch.equal(states[5].cpu(), before[5])


def test_a_token_far_back_stays_in_a_state_that_does_not_decay(k):
    """Decays of one: after 900 tokens the query that matches token 17's key still finds its value."""
    heads, dk, dv, t = 1, 32, 64, 900
    width = 2 * dk + dv
    proj = rnd(1, t, width, seed=1, scale=0.005)
    key = torch.zeros(dk)
    key[5] = 4.0
    proj[0, 17, dk : 2 * dk] = key
    proj[0, 17, 2 * dk :] = rnd(dv, seed=2)
    proj[0, t - 1, :dk] = key
    decay = torch.ones(t, dk)
    states = torch.zeros((1, heads, dk, dv), device=DEV)
    outs = []
    for first, n in [(0, 600), (600, 299), (899, 1)]:
        outs.append(k.decayed_state_scan(proj[:, first : first + n].contiguous().to(DEV), torch.float32, 0, dk, 2 * dk, 1.0,
                                         decay[first : first + n].to(DEV), states, i32(0), torch.tensor([first == 0], device=DEV),
                                         i32(0), i32(n), heads, dk, dv))
    want, _ = plain_scan(proj[0], decay, (0, dk, 2 * dk), heads, dk, dv, 1.0)
    close(torch.cat([added(o) for o in outs]).view(t, heads, dv), want, torch.float32, "no decay")
    found = 16.0 * proj[0, 17, 2 * dk :]
    assert float((added(outs[-1])[0].cpu() - found).abs().max()) < 0.01 * float(found.abs().max())


# ----------------------------------------------------------------------------- the mixture of experts
def plain_mixture(x, router, bias, wgu, wd, top):
    xx = x.to(F64)
    ff = wgu.shape[1] // 2
    w = {"m.router": router.to(F64), "m.router.b": bias.to(F64)}
    for e in range(wgu.shape[0]):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = wgu[e, :ff].to(F64), wgu[e, ff:].to(F64), wd[e].to(F64)
    return P.expert_mixture(xx, w, "m.", {"router": {"top": top}})


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t, hidden, ff, experts, top", [(7, 64, 48, 6, 2), (1, 100, 50, 5, 1), (40, 100, 30, 3, 3), (600, 128, 64, 8, 2),
                                                         (300, 256, 80, 10, 4), (3, 36, 10, 70, 5), (130, 72, 20, 2, 1)])
def test_the_mixture_of_experts(k, dtype, t, hidden, ff, experts, top):
    x = rnd(t, hidden, seed=1).to(dtype)
    router, bias = rnd(experts, hidden, seed=2, scale=0.5).to(dtype), rnd(experts, seed=3).to(dtype)
    wgu = rnd(experts, 2 * ff, hidden, seed=4, scale=hidden ** -0.5).to(dtype)
    wd = rnd(experts, hidden, ff, seed=5, scale=ff ** -0.5).to(dtype)
    got = k.expert_mixture(x.to(DEV), router.to(DEV), bias.to(DEV), wgu.to(DEV), wd.to(DEV), top)
    assert got.dtype == torch.float32 and got.shape == (t, hidden)
    want = plain_mixture(x, router, bias, wgu, wd, top)
    # (the router sees the same rounded input here and there, so its choices are the same)
    close(got, want, dtype, "mixture")


def test_every_token_of_a_batch_gets_what_it_gets_alone_and_equal_logits_go_to_the_lower_index(k):
    """Inputs and router rows of small integers: the logits are exact whatever the order of the sums, and many of them
    are equal."""
    t, hidden, ff, experts, top = 50, 64, 32, 6, 2
    g = torch.Generator().manual_seed(1)
    x = torch.randint(-2, 3, (t, hidden), generator=g).float()
    router, bias = torch.randint(-1, 2, (experts, hidden), generator=g).float(), torch.zeros(experts)
    router[4] = router[1]                            # experts 1 and 4 always tie
    wgu, wd = rnd(experts, 2 * ff, hidden, seed=4, scale=0.1), rnd(experts, hidden, ff, seed=5, scale=0.2)
    dev = [a.to(DEV) for a in (router, bias, wgu, wd)]
    together = k.expert_mixture(x.to(DEV), *dev, top)
    for i in (0, 1, 17, 49):
        assert torch.equal(k.expert_mixture(x[i : i + 1].to(DEV), *dev, top)[0], together[i])
    z = x.to(F64) @ router.to(F64).T
    assert torch.equal(z[:, 1], z[:, 4]) and int((z.sort(-1).values.diff(dim=-1) == 0).sum()) > t
    close(together, plain_mixture(x, router, bias, wgu, wd, top), torch.float32, "ties")
