"""The kernels of the mixers that treat single heads, each alone against the plain functions of
tests/plain_pekasun.py: the normed embedding, per-head norms with the store into pages, the preparation of latent
attention (latent norm, interleaved rotation with stretched frequencies), the sigmoid gate, and the attention
kernel with separate key and value sizes, window, kept first tokens and sink.  Where random inputs would hide a
fault (one far key among hundreds, the keys at a window's two edges, the sink), queries and keys are made so that
one score stands out."""
import math

import pytest
import torch

import plain_pekasun as P

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


def close(got, want, dtype, what=""):
    got, want = got.detach().to("cpu", F64), want.to(F64)
    err = float((got - want).abs().max())
    scale = max(float(want.abs().max()), 1e-6)
    assert err <= TOL[dtype] * scale, f"{what}: max |diff| {err:.3e} against scale {scale:.3f}"


def paged(keys, values, page_size, dtype, seed, spare=3):
    """Dense keys [n, nkv, dk] and values [n, nkv, dv] laid into pages in a shuffled order: (k_cache, v_cache, table)."""
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


def plain_attention(q, keys, values, first_pos, scale, window, keep_first, sink):
    """q [m, nq, dk] at positions first_pos.., keys [n, nkv, dk], values [n, nkv, dv] -> [m, nq, dv] in float64."""
    m, nq, _ = q.shape
    n, nkv, _ = keys.shape
    rep = nq // nkv
    kh = keys.to(F64).repeat_interleave(rep, dim=1)
    vh = values.to(F64).repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q.to(F64), kh) * scale
    vis = P.visible_window_keep_first(n, window if window else 1 << 60, keep_first)[first_pos : first_pos + m]
    pr = P.softmax_with_sink(scores, vis, None if sink is None else sink.to(F64))
    return torch.einsum("hij,jhd->ihd", pr, vh)


def run_attention(k, q, k_cache, v_cache, table, kv_len, page_size, scale, window, keep_first, sink, dv):
    m, nq, dk = q.shape
    nkv = k_cache.shape[1]
    out = torch.empty((m, nq * dv), dtype=q.dtype, device=DEV)
    i32 = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
    k.window_attention(q.reshape(m, nq * dk).to(DEV).contiguous(), out, k_cache, v_cache, table, i32(0), i32(m), i32(kv_len),
                       nq, nkv, dk, dv, page_size, scale, window, keep_first,
                       None if sink is None else sink.to(DEV), m, kv_len)
    return out.view(m, nq, dv)


# ----------------------------------------------------------------------------- elementwise mechanisms
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [48, 256, 1000])
def test_embedding_with_its_norm(k, dtype, hidden):
    table = rnd(37, hidden, seed=1, scale=3.0, dtype=dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32)
    gain = torch.full((hidden,), 1.25, dtype=dtype)
    out = torch.empty((5, hidden), dtype=torch.float32, device=DEV)
    k.embed_rmsnorm(ids.to(DEV), table.to(DEV), gain.to(DEV), 1e-5, out)
    want = P.scalar_norm(table.to(F64)[ids.long()], torch.tensor(1.25, dtype=F64), 1e-5)
    close(out, want, torch.float32, "normed embedding")            # the stream is float32 in both precisions


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv, splits", [(4, 2, 16, 32, 0), (3, 3, 40, 24, 3), (2, 1, 200, 8, 1)])
def test_head_norms_and_the_store_into_pages(k, dtype, nq, nkv, dk, dv, splits):
    t, ps, eps = 11, 4, 1e-3
    width = (nq + nkv) * dk + nkv * dv
    proj = rnd(max(splits, 1), t, width, seed=2, scale=2.0)
    whole = proj.sum(0)
    given = proj.to(DEV) if splits else whole.to(dtype).to(DEV)
    if not splits:
        whole = whole.to(dtype).to(F64)
    qw, kw = rnd(dk, seed=3, dtype=dtype) + 1, rnd(dk, seed=4, dtype=dtype) + 1
    slots = torch.randperm(6 * ps, generator=torch.Generator().manual_seed(5))[:t].to(torch.int32)
    k_cache = torch.zeros((6, nkv, ps, dk), dtype=dtype, device=DEV)
    v_cache = torch.zeros((6, nkv, dv, ps), dtype=dtype, device=DEV)
    q_out = torch.empty((t, nq * dk), dtype=dtype, device=DEV)
    k.head_norm_store(given, q_out, qw.to(DEV), kw.to(DEV), eps, True, slots.to(DEV), k_cache, v_cache, nq, nkv, dk, dv, ps)
    x = whole.to(F64)
    q = P.vector_norm(x[:, : nq * dk].view(t, nq, dk), qw.to(F64), eps)
    kk = P.vector_norm(x[:, nq * dk : (nq + nkv) * dk].view(t, nkv, dk), kw.to(F64), eps)
    vv = P.unit_rms(x[:, (nq + nkv) * dk :].view(t, nkv, dv), eps)
    close(q_out.view(t, nq, dk), q, dtype, "queries")
    page, off = (slots // ps).long(), (slots % ps).long()
    close(k_cache.cpu()[page, :, off, :], kk, dtype, "keys in their pages")
    close(v_cache.cpu()[page, :, :, off], vv, dtype, "values in their pages")
    # without weights and without the values' norm the heads pass as they are
    k.head_norm_store(given, q_out, None, None, eps, False, slots.to(DEV), k_cache, v_cache, nq, nkv, dk, dv, ps)
    close(q_out, x[:, : nq * dk], dtype, "queries as they are")
    close(v_cache.cpu()[page, :, :, off], x[:, (nq + nkv) * dk :].view(t, nkv, dv), dtype, "values as they are")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, dim, rot, dims, rank, scaling", [
    (2, 16, 8, 8, 40, {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}),
    (1, 8, 16, 12, 24, None),
    (3, 32, 64, 64, 96, {"factor": 2.0, "original": 512, "fast": 32.0, "slow": 1.0}),
])
def test_latent_preparation(k, dtype, nq, dim, rot, dims, rank, scaling):
    from easy_gpt.cpp_amd.parts import PartSpec, make_part

    t, ps, eps, extra = 9, 8, 1e-4, 5
    width = nq * (dim + rot) + rank + rot + extra
    x = rnd(t, width, seed=6, scale=1.5).to(dtype)
    positions = torch.tensor([0, 1, 2, 3, 700, 701, 4095, 31, 64], dtype=torch.int32)
    rot_cfg = {"base": 10000.0, "dims": dims, "scaling": scaling}
    pos_part = make_part("position_encoding", PartSpec("rope_interleaved", dict(theta=10000.0, rotary_dim=dims, scaling=scaling)),
                         head_dim=rot)
    inv_freq, _ = pos_part.rotary(DEV)
    freqs, mag = P.yarn_frequencies(rot_cfg)
    assert abs(pos_part.magnitude - mag) < 1e-12
    close(inv_freq, freqs, torch.float32, "frequencies")
    cos_sin = k.rope_table(positions.to(DEV), inv_freq)
    cw = rnd(rank, seed=7, dtype=dtype) + 1
    slots = torch.randperm(3 * ps, generator=torch.Generator().manual_seed(8))[:t].to(torch.int32)
    k_cache = torch.zeros((3, 1, ps, rank + rot), dtype=dtype, device=DEV)
    v_cache = torch.zeros((3, 1, rank, ps), dtype=dtype, device=DEV)
    q_plain = torch.empty((t, nq, dim), dtype=dtype, device=DEV)
    q_full = torch.zeros((t, nq, rank + rot), dtype=dtype, device=DEV)
    k.latent_prep(x.to(DEV), q_plain, q_full, cw.to(DEV), eps, cos_sin, pos_part.magnitude, dims, slots.to(DEV), k_cache, v_cache,
                  nq, dim, rot, rank, ps)
    xd = x.to(F64)
    q = xd[:, : nq * (dim + rot)].view(t, nq, dim + rot)
    base = nq * (dim + rot)
    c = P.vector_norm(xd[:, base : base + rank], cw.to(F64), eps)
    shared = P.rotate_interleaved(xd[:, base + rank : base + rank + rot], positions, freqs, mag)
    q_rot = P.rotate_interleaved(q[..., dim:].transpose(0, 1), positions, freqs, mag).transpose(0, 1)
    # float32 angles of positions in the thousands differ from float64 ones by 1e-4 of a turn
    tol_dtype = dtype
    close(q_plain, q[..., :dim], tol_dtype, "plain query parts")
    got, want = q_full[..., rank:].cpu().to(F64), q_rot
    assert float((got - want).abs().max()) <= (2e-3 if dtype == torch.float32 else 5e-2) * float(want.abs().max())
    assert float(q_full[..., :rank].abs().max()) == 0.0            # the caller's part is left alone
    page, off = (slots // ps).long(), (slots % ps).long()
    keys = k_cache.cpu()[page, 0, off, :].to(F64)
    close(keys[:, :rank], c, dtype, "latent as key")
    assert float((keys[:, rank:] - shared).abs().max()) <= (2e-3 if dtype == torch.float32 else 5e-2) * float(shared.abs().max())
    close(v_cache.cpu()[page, 0, :, off], c, dtype, "latent as value")
    # at small positions the angles are exact enough for the float32 line
    small = positions < 100
    close(q_full[..., rank:][small.to(DEV)], q_rot[small], dtype, "rotated query parts at small positions")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads", [0, 3])
def test_sigmoid_gate(k, dtype, heads):
    t, n, width, off = 7, 48, 100, 31
    gate = rnd(2, t, width, seed=9, scale=3.0)
    x = rnd(t, n, seed=10).to(dtype)
    given = x.view(t, heads, n // heads).transpose(0, 1).contiguous() if heads else x
    out = torch.empty((t, n), dtype=dtype, device=DEV)
    k.sigmoid_gate(given.to(DEV), heads, gate.to(DEV), off, out)
    close(out, x.to(F64) * torch.sigmoid(gate.sum(0).to(F64)[:, off : off + n]), dtype, "gate")


# ----------------------------------------------------------------------------- attention
SHAPES = [(4, 2, 16, 32), (3, 3, 40, 24), (8, 1, 128, 96), (2, 2, 48, 48), (1, 1, 72, 16)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv", SHAPES)
@pytest.mark.parametrize("window, keep_first, with_sink", [(0, 0, False), (21, 0, True), (21, 5, False), (16, 40, True), (1, 0, True)])
def test_attention_against_plain(k, dtype, nq, nkv, dk, dv, window, keep_first, with_sink):
    n, ps = 150, 16
    keys, values = rnd(n, nkv, dk, seed=11).to(dtype), rnd(n, nkv, dv, seed=12).to(dtype)
    q = rnd(n, nq, dk, seed=13, scale=1.5).to(dtype)
    sink = rnd(nq, seed=14, scale=2.0) if with_sink else None
    scale = 1.7 / math.sqrt(dk)
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=15)
    want = plain_attention(q, keys, values, 0, scale, window, keep_first, sink)
    # the whole prompt in one call
    got = run_attention(k, q, k_cache, v_cache, table, n, ps, scale, window, keep_first, sink, dv)
    close(got, want, dtype, "whole prompt")
    # a portion in the middle, a portion of two tokens, and single tokens, against the same cache
    for first, m in [(37, 50), (95, 2), (0, 1), (149, 1), (63, 1), (64, 1)]:
        got = run_attention(k, q[first : first + m], k_cache, v_cache, table, first + m, ps, scale, window, keep_first, sink, dv)
        close(got, want[first : first + m], dtype, f"rows {first}..{first + m}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq, nkv, dk, dv", [(4, 2, 16, 32), (8, 1, 128, 96), (6, 2, 72, 16)])
@pytest.mark.parametrize("window, keep_first, with_sink", [(0, 0, True), (70, 0, False), (40, 33, True)])
def test_attention_with_32_rows_to_a_wavefront(k, dtype, nq, nkv, dk, dv, window, keep_first, with_sink):
    """The shape that steps of thousands of rows take, forced on a small one."""
    from easy_gpt.cpp_amd.kernels.hip import HipKernels

    n, ps = 333, 16
    keys, values = rnd(n, nkv, dk, seed=81).to(dtype), rnd(n, nkv, dv, seed=82).to(dtype)
    q = rnd(n, nq, dk, seed=83, scale=1.5).to(dtype)
    sink = rnd(nq, seed=84, scale=2.0) if with_sink else None
    scale = 1.7 / math.sqrt(dk)
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=85)
    want = plain_attention(q, keys, values, 0, scale, window, keep_first, sink)
    before = HipKernels.wide_rows_from, HipKernels.wide_rows_key_size
    HipKernels.wide_rows_from = HipKernels.wide_rows_key_size = 0
    try:
        assert HipKernels._window_attention_shape(n, 1, nq, nkv, dk, dv, ps, window, keep_first, n, n, q.element_size())[0] == 8
        got = run_attention(k, q, k_cache, v_cache, table, n, ps, scale, window, keep_first, sink, dv)
        close(got, want, dtype, "whole prompt")
        got = run_attention(k, q[200:301], k_cache, v_cache, table, 301, ps, scale, window, keep_first, sink, dv)
        close(got, want[200:301], dtype, "a portion")
    finally:
        HipKernels.wide_rows_from, HipKernels.wide_rows_key_size = before


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_far_key_among_hundreds_is_found(k, dtype):
    """Key 3 of 900 fits the query; every other key is noise.  The output is key 3's value."""
    n, ps, dk, dv = 900, 16, 64, 32
    keys, values = rnd(n, 1, dk, seed=16, scale=0.05), rnd(n, 1, dv, seed=17)
    q = rnd(1, 2, dk, seed=18, scale=0.05)
    keys[3, 0, 0], q[0, :, 0] = 6.0, 6.0
    keys, values, q = keys.to(dtype), values.to(dtype), q.to(dtype)
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=19)
    got = run_attention(k, q, k_cache, v_cache, table, n, ps, 1.0, 0, 0, None, dv)
    close(got, plain_attention(q, keys, values, n - 1, 1.0, 0, 0, None), dtype, "far key")
    close(got[0, 0], values[3, 0], dtype, "the far key's value")
    # behind a window it is gone, and kept as one of the first tokens it is back
    got = run_attention(k, q, k_cache, v_cache, table, n, ps, 1.0, 500, 3, None, dv)
    assert float((got[0, 0].cpu().to(F64) - values[3, 0].to(F64)).abs().max()) > 0.5
    got = run_attention(k, q, k_cache, v_cache, table, n, ps, 1.0, 500, 4, None, dv)
    close(got[0, 0], values[3, 0], dtype, "kept first token")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window, keep_first", [(16, 0), (17, 3), (33, 16), (5, 1), (64, 17)])
@pytest.mark.parametrize("single", [True, False])
def test_the_keys_at_the_edges_of_window_and_kept_tokens(k, dtype, window, keep_first, single):
    """For every query position, the key just inside the window, the key just outside it, the last kept token and the
    first one that is not kept are each made to fit the query in turn: the output is that key's value if it is
    visible, and noise if it is not.  In prompts (all rows in one call) and for single tokens."""
    n, ps, dk, dv = 100, 16, 32, 16
    base_keys, values = rnd(n, 1, dk, seed=20, scale=0.02), rnd(n, 1, dv, seed=21)
    q = rnd(n, 1, dk, seed=22, scale=0.02)
    q[:, 0, 1] = 8.0
    for p in [window - 1, window, window + 1, 47, 48, 63, 64, 99]:
        for j in {p - window + 1, p - window, keep_first - 1, keep_first}:
            if not 0 <= j <= p:
                continue
            keys = base_keys.clone()
            keys[j, 0, 1] = 8.0
            kd, vd, qd = keys.to(dtype), values.to(dtype), q.to(dtype)
            k_cache, v_cache, table = paged(kd, vd, ps, dtype, seed=23 + j)
            if single:
                got = run_attention(k, qd[p : p + 1], k_cache, v_cache, table, p + 1, ps, 1.0, window, keep_first, None, dv)[0, 0]
            else:
                got = run_attention(k, qd[: p + 1], k_cache, v_cache, table, p + 1, ps, 1.0, window, keep_first, None, dv)[p, 0]
            visible = p - j < window or j < keep_first
            d = float((got.cpu().to(F64) - vd[j, 0].to(F64)).abs().max())
            assert (d < 0.05) == visible, (p, j, visible, d)
            close(got, plain_attention(qd[p : p + 1], kd[: p + 1], vd[: p + 1], p, 1.0, window, keep_first, None)[0, 0], dtype, (p, j))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_sink_takes_its_share_and_nothing_else(k, dtype):
    n, ps, dk, dv, nq = 40, 16, 16, 16, 3
    keys, values, q = rnd(n, 1, dk, seed=30).to(dtype), rnd(n, 1, dv, seed=31).to(dtype), rnd(1, nq, dk, seed=32).to(dtype)
    k_cache, v_cache, table = paged(keys, values, ps, dtype, seed=33)
    sink = torch.tensor([-40.0, 0.0, 9.0])
    got = run_attention(k, q, k_cache, v_cache, table, n, ps, 0.3, 0, 0, sink, dv)
    free = run_attention(k, q, k_cache, v_cache, table, n, ps, 0.3, 0, 0, None, dv)
    close(got, plain_attention(q, keys, values, n - 1, 0.3, 0, 0, sink), dtype, "sink")
    close(got[0, 0], free[0, 0].cpu(), dtype, "a sink far below the scores changes nothing")
    assert float(got[0, 2].abs().max()) < 0.2 * float(free[0, 2].abs().max())      # a sink far above them takes nearly all
    # the sink is not scaled: with a scale of 0 all keys weigh exp(0) and the sink exp(sink)
    got = run_attention(k, q, k_cache, v_cache, table, n, ps, 0.0, 0, 0, sink, dv)
    mean = values.to(F64).mean(0)[0]
    close(got[0, 1], mean * n / (n + 1.0), dtype, "unscaled sink")


def test_a_batch_of_unequal_requests_gives_each_its_own(k):
    """float32: a request's rows alone and among others, as a portion and token by token, differ by rounding only (the
    kernel deals rows and keys over wavefronts by the step's shape)."""
    dtype, ps, nq, nkv, dk, dv = torch.float32, 16, 4, 2, 48, 32
    lens, news = [70, 5, 33], [1, 5, 9]
    ks = [rnd(n, nkv, dk, seed=40 + i) for i, n in enumerate(lens)]
    vs = [rnd(n, nkv, dv, seed=50 + i) for i, n in enumerate(lens)]
    qs = [rnd(m, nq, dk, seed=60 + i) for i, m in enumerate(news)]
    pages = [-(-n // ps) for n in lens]
    total = sum(pages)
    k_cache = torch.zeros((total, nkv, ps, dk)); v_cache = torch.zeros((total, nkv, dv, ps))
    table = torch.full((3, max(pages)), -1, dtype=torch.int32)
    order = torch.randperm(total, generator=torch.Generator().manual_seed(1)).tolist()
    for b, n in enumerate(lens):
        mine = [order.pop() for _ in range(pages[b])]
        table[b, : pages[b]] = torch.tensor(mine, dtype=torch.int32)
        for j in range(n):
            k_cache[mine[j // ps], :, j % ps] = ks[b][j]
            v_cache[mine[j // ps], :, :, j % ps] = vs[b][j]
    k_cache, v_cache = k_cache.to(DEV), v_cache.to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    starts = [0, news[0], news[0] + news[1]]
    q_all = torch.cat([x.reshape(x.shape[0], -1) for x in qs]).to(DEV)
    out = torch.empty((sum(news), nq * dv), device=DEV)
    sink = rnd(nq, seed=70).to(DEV)
    k.window_attention(q_all, out, k_cache, v_cache, table.to(DEV), i32(starts), i32(news), i32(lens), nq, nkv, dk, dv, ps, 0.2,
                       24, 2, sink, max(news), max(lens))
    for b in range(3):
        alone = torch.empty((news[b], nq * dv), device=DEV)
        k.window_attention(q_all[starts[b] : starts[b] + news[b]].contiguous(), alone, k_cache, v_cache,
                           table[b : b + 1].to(DEV).contiguous(), i32([0]), i32([news[b]]), i32([lens[b]]), nq, nkv, dk, dv, ps,
                           0.2, 24, 2, sink, news[b], lens[b])
        assert float((alone - out[starts[b] : starts[b] + news[b]]).abs().max()) <= 2e-6 * float(out.abs().max())
        for i in range(news[b]):
            one = torch.empty((1, nq * dv), device=DEV)
            k.window_attention(q_all[starts[b] + i : starts[b] + i + 1].contiguous(), one, k_cache, v_cache,
                               table[b : b + 1].to(DEV).contiguous(), i32([0]), i32([1]), i32([lens[b] - news[b] + i + 1]), nq,
                               nkv, dk, dv, ps, 0.2, 24, 2, sink, 1, lens[b])
            assert float((one[0] - out[starts[b] + i]).abs().max()) <= 2e-6 * float(out.abs().max())
