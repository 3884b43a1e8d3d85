"""Gilozen on the GPU against the plain implementation (plain_gilozen.py): every mechanism alone, then
whole models of two small configurations through the step function, the scheduler and the replay.

The weights are drawn here with a spread that keeps activations of order one (standard deviation
fan_in^-1/2; sinks, decay biases and the norms' offsets wide), so that softmax rows are peaked, decays differ
from channel to channel and a sink or a norm that is left out shows."""

import json
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_gilozen as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from from_scratch_inference_engine_amd import ops as o

    o.load()
    return o


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def rel(got, ref):
    got, ref = torch.as_tensor(got, dtype=torch.float64), torch.as_tensor(ref, dtype=torch.float64)
    return ((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()


def tol(dtype, f32=2e-5, bf16=2.0 ** -6):
    return f32 if dtype == torch.float32 else bf16


# ------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, n_parts", [(96, 0), (257, 3), (4100, 0), (1024, 8)])
def test_sandwich_norm(ops, dtype, hidden, n_parts):
    """post norm of the sublayer's output + residual sum + next norm, against the three steps written out;
    the delta as one array or as partial sums; all rows written back, or chosen rows left alone."""
    t = 7
    res = rnd((t, hidden), 1, 3.0)
    delta = rnd((n_parts or 1, t, hidden), 2, 0.5)
    if dtype == torch.bfloat16 and not n_parts:
        delta = delta.bfloat16().float()
    wp, w = 1 + rnd((hidden,), 3, 0.3), 1 + rnd((hidden,), 4, 0.3)
    y = delta.double().sum(0)
    v = res.double() + plain.norm_plain_weight(y, wp.double(), 1e-5)
    ref = plain.norm_plain_weight(v, w.double(), 1e-6)
    d_dev = (delta if n_parts else delta[0].to(dtype)).cuda()
    r_dev = res.cuda().clone()
    out = ops.sandwich_norm(r_dev, d_dev, wp.cuda(), 1e-5, w.cuda(), 1e-6, dtype, write_back=True)
    assert rel(out.float().cpu(), ref) <= tol(dtype, bf16=2.0 ** -7)
    assert rel(r_dev.cpu(), v) <= 2e-6  # the stream is float32 in both precisions
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32).cuda()
    r_dev = res.cuda().clone()
    out = ops.sandwich_norm(r_dev, d_dev, wp.cuda(), 1e-5, w.cuda(), 1e-6, dtype, rows=rows)
    assert rel(out.float().cpu(), ref[rows.cpu().long()]) <= tol(dtype, bf16=2.0 ** -7)
    assert torch.equal(r_dev.cpu(), res)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_activation_alone_and_in_the_products(ops, dtype):
    """GELU (tanh form) of the gate times up: the kernel of its own and the two products that have it in
    their epilogue, all from one interleaved gate/up matrix."""
    m, k, inter = 9, 128, 132
    x = rnd((m, k), 1).to(dtype)
    gate, up = rnd((inter, k), 2, k ** -0.5).to(dtype), rnd((inter, k), 3, k ** -0.5).to(dtype)
    ref = plain.gelu_tanh(x.double() @ gate.double().t()) * (x.double() @ up.double().t())
    w = torch.stack([gate, up], dim=1).reshape(2 * inter, k).contiguous().cuda()
    both = torch.stack([x.double() @ gate.double().t(), x.double() @ up.double().t()], dim=2).reshape(m, 2 * inter)
    got = ops.swiglu(both.to(dtype).cuda(), act="gelu_tanh")
    assert rel(got.float().cpu(), ref) <= tol(dtype)
    silu = ops.swiglu(both.to(dtype).cuda())  # the default is untouched
    g = both[:, 0::2]
    assert rel(silu.float().cpu(), g * torch.sigmoid(g) * both[:, 1::2]) <= tol(dtype)
    if dtype == torch.bfloat16:
        assert rel(ops.gemm_mfma_skinny(x.cuda(), w, epilogue="geglu_tanh").float().cpu(), ref) <= 2.0 ** -6
        assert rel(ops.gemm_mfma_wide_swiglu(x.cuda(), w, act="gelu_tanh").float().cpu(), ref) <= 2.0 ** -6


def test_softcap_and_gated_headnorm(ops):
    x = rnd((5, 301), 1, 20.0)
    assert rel(ops.softcap(x.cuda().clone(), 7.5).cpu(), 7.5 * torch.tanh(x.double() / 7.5)) <= 1e-6
    for dtype in DTYPES:
        heads, width, t = 3, 70, 6
        o, w = rnd((t, heads * width), 2, 4.0), 1 + rnd((width,), 3, 0.3)
        wide = rnd((t, 11 + heads * width), 4).to(dtype)  # the gate is the tail of wider rows
        g = wide[:, 11:].double()
        ref = plain.norm_plain_weight(o.double().reshape(t, heads, width), w.double(), 1e-5).reshape(t, -1) * g * torch.sigmoid(g)
        got = ops.gated_headnorm(o.cuda(), wide.cuda()[:, 11:], w.cuda(), 1e-5, heads)
        assert got.dtype == dtype and rel(got.float().cpu(), ref) <= tol(dtype, bf16=2.0 ** -7)
        shares = torch.stack([0.5 * o, 0.25 * o, 0.25 * o]).cuda()  # o as three planes that are added first
        got = ops.gated_headnorm(shares, wide.cuda()[:, 11:], w.cuda(), 1e-5, heads)
        assert rel(got.float().cpu(), ref) <= tol(dtype, bf16=2.0 ** -7)


def oracle_gla_states(q, k, v, z, tau, state):
    """The recurrence on given q (already scaled), k, v [T, H, *] and decay logits z: returns o and the state."""
    alpha = torch.pow(torch.sigmoid(z), 1.0 / tau)
    out = []
    for i in range(q.shape[0]):
        state = alpha[i].unsqueeze(-1) * state + k[i].unsqueeze(-1) * v[i].unsqueeze(-2)
        out.append(torch.einsum("hdv,hd->hv", state, q[i]))
    return torch.stack(out), state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim", [(2, 20, 24), (1, 130, 70), (3, 64, 128), (2, 100, 9)])
def test_gla_scan_over_portions_and_slots(ops, dtype, heads, dim, vdim):
    """Three requests of unequal length in one step, then each continued (a long portion, two tokens, one
    token), then a slot that is zeroed and used by a new request: against the recurrence from zero.  The
    decay logits are wide, so some channels forget at once and others hardly at all."""
    tau, scale = 3.0, dim ** -0.5
    lens = {"a": [37, 1, 2], "b": [2, 40, 1], "c": [1, 1, 19]}
    total = {r: sum(n) for r, n in lens.items()}
    kw, vw = heads * dim, heads * vdim
    data = {r: (rnd((n, 2 * kw + vw + 5), 10 + i).to(dtype), rnd((n, kw), 20 + i, 3.0)) for i, (r, n) in enumerate(total.items())}
    slots = {"a": 2, "b": 0, "c": 3}
    state = torch.full((5, heads, dim, vdim), 99.0).cuda()  # stale content everywhere
    state[[0, 2, 3]] = 0.0
    fed = {r: 0 for r in lens}
    got = {r: [] for r in lens}
    for step in range(3):
        order = ["b", "c", "a"] if step == 1 else ["a", "b", "c"]
        rows = [(r, fed[r], fed[r] + lens[r][step]) for r in order]
        proj = torch.cat([data[r][0][lo:hi] for r, lo, hi in rows]).cuda()
        z = torch.cat([data[r][1][lo:hi] for r, lo, hi in rows]).cuda()
        starts = np.cumsum([0] + [hi - lo for _, lo, hi in rows]).astype(np.int32)
        o = ops.gla_scan(proj, 5, 5 + kw, 5 + 2 * kw, z, state, torch.from_numpy(starts).cuda(),
                         torch.tensor([slots[r] for r in order], dtype=torch.int32).cuda(), heads, dim, vdim, scale, 1 / tau)
        o = o.sum(0).cpu()  # the shares of the groups of key channels
        for i, (r, lo, hi) in enumerate(rows):
            got[r].append(o[starts[i]:starts[i + 1]])
            fed[r] = hi
    finals = {}
    for r in lens:
        p, logits = data[r][0].double(), data[r][1].double()
        n = total[r]
        ref, finals[r] = oracle_gla_states(p[:, 5:5 + kw].reshape(n, heads, dim) * scale, p[:, 5 + kw:5 + 2 * kw].reshape(n, heads, dim),
                                           p[:, 5 + 2 * kw:].reshape(n, heads, vdim), logits.reshape(n, heads, dim), tau,
                                           torch.zeros(heads, dim, vdim, dtype=torch.float64))
        assert rel(torch.cat(got[r]).reshape(n, heads, vdim), ref) <= 2e-5, r  # float32 inside, whatever the inputs' type
        assert rel(state[slots[r]].cpu(), finals[r]) <= 2e-5
    assert (state[[1, 4]] == 99.0).all()  # nobody else's slot was touched
    # a slot outside the table: the request is skipped, nothing is written
    before = state.clone()
    ops.gla_scan(proj, 5, 5 + kw, 5 + 2 * kw, z, state, torch.from_numpy(starts).cuda(),
                 torch.tensor([-1, -1, -1], dtype=torch.int32).cuda(), heads, dim, vdim, scale, 1 / tau)
    assert torch.equal(before, state)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim, tau", [(2, 48, 40, 0.25), (1, 256, 200, 16.0), (5, 16, 64, 1.0), (2, 72, 130, 2.0)])
def test_gla_scan_chunk_by_chunk_and_token_by_token(ops, dtype, heads, dim, vdim, tau):
    """Portions around the length from which a portion is cut into chunks, whole chunks, one token more and one
    less, a long one, beside single tokens; continued from a state that is not zero.  Decays of every kind in
    one head: channels that forget everything within a token (their logarithms summed over a chunk are far
    below what float32's exponential can hold) next to channels that keep everything, where a loud first token
    must still be there at the end.  Both ways of walking a portion against the recurrence."""
    scale = dim ** -0.5
    lens = [[16, 15, 17, 1, 32, 250, 2, 33], [3, 250, 1, 16, 31, 40, 47, 1]]
    kw, vw = heads * dim, heads * vdim
    slots = [5, 0, 3, 1, 4, 7, 2, 6]
    for chunked in (True, False):
        state = torch.zeros(9, heads, dim, vdim).cuda()
        datas, fed = [], [0] * len(slots)
        for i in range(len(slots)):
            n = lens[0][i] + lens[1][i]
            proj, z = rnd((n, 2 * kw + vw), 30 + i).to(dtype), rnd((n, kw), 50 + i, 4.0)
            z.view(n, heads, dim)[:, :, 0::3] = 25.0   # keeps everything
            z.view(n, heads, dim)[:, :, 1::5] = -60.0  # keeps nothing
            proj[0, kw:kw + kw] *= 30.0  # a loud first key: the keeping channels carry it to the last token
            datas.append((proj, z))
        outs = [[] for _ in slots]
        for step in range(2):
            rows = [(i, fed[i], fed[i] + lens[step][i]) for i in range(len(slots))]
            proj = torch.cat([datas[i][0][lo:hi] for i, lo, hi in rows]).cuda()
            z = torch.cat([datas[i][1][lo:hi] for i, lo, hi in rows]).cuda()
            starts = np.cumsum([0] + [hi - lo for _, lo, hi in rows]).astype(np.int32)
            o = ops.gla_scan(proj, 0, kw, 2 * kw, z, state, torch.from_numpy(starts).cuda(),
                             torch.tensor(slots, dtype=torch.int32).cuda(), heads, dim, vdim, scale, 1 / tau, chunked=chunked)
            assert torch.isfinite(o).all()
            o = o.sum(0).cpu()
            for i, lo, hi in rows:
                outs[i].append(o[starts[i]:starts[i + 1]])
                fed[i] = hi
        for i, (proj, z) in enumerate(datas):
            n, p = proj.shape[0], proj.double()
            ref, final = oracle_gla_states(p[:, :kw].reshape(n, heads, dim) * scale, p[:, kw:2 * kw].reshape(n, heads, dim),
                                           p[:, 2 * kw:].reshape(n, heads, vdim), z.double().reshape(n, heads, dim), tau,
                                           torch.zeros(heads, dim, vdim, dtype=torch.float64))
            got = torch.cat(outs[i]).reshape(n, heads, vdim)
            assert rel(got, ref) <= 2e-5, (chunked, i)
            assert rel(got[-1], ref[-1]) <= 2e-5, (chunked, i)
            assert rel(state[slots[i]].cpu(), final) <= 2e-5, (chunked, i)
        assert (state[8] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_prep_rope_pairs_and_head_gemm(ops, dtype):
    heads, q_rank, kv_rank, rot_dim, pairs, page, t = 3, 40, 52, 12, 4, 8, 11
    width = 64
    stride = 7 + q_rank + kv_rank + rot_dim + heads
    proj = rnd((t, stride), 1, 2.0).to(dtype)
    wq, wkv = 1 + rnd((q_rank,), 2, 0.3), 1 + rnd((kv_rank,), 3, 0.3)
    positions = torch.tensor([0, 1, 5, 300, 7, 8, 9, 1000, 15, 16, 17], dtype=torch.int32)
    inv = torch.pow(torch.tensor(5e4, dtype=torch.float64), -2.0 * torch.arange(pairs, dtype=torch.float64) / (2 * pairs))
    table = ops.rope_table(positions.cuda(), inv.cuda())
    units = 6
    k_pool = torch.full((units, 1, page, width), 7.0, dtype=dtype).cuda()
    v_pool = torch.full((units, 1, width, page), 7.0, dtype=dtype).cuda()
    slots = torch.tensor([8, 9, 13, 44, 15, 16, 17, 40, 23, 24, -1], dtype=torch.int32)
    cq, gate = ops.latent_prep(proj.cuda(), 7, q_rank, 7 + q_rank, kv_rank, rot_dim, pairs, 7 + q_rank + kv_rank + rot_dim, heads,
                               wq.cuda(), wkv.cuda(), 1e-5, table, slots=slots.cuda(), k_pool=k_pool, v_pool=v_pool)
    p = proj.double()
    assert rel(cq.float().cpu(), plain.norm_plain_weight(p[:, 7:7 + q_rank], wq.double(), 1e-5)) <= tol(dtype, bf16=2.0 ** -7)
    assert rel(gate.cpu(), torch.sigmoid(p[:, -heads:])) <= 1e-6
    c = plain.norm_plain_weight(p[:, 7 + q_rank:7 + q_rank + kv_rank], wkv.double(), 1e-5)
    kr = p[:, 7 + q_rank + kv_rank:7 + q_rank + kv_rank + rot_dim].reshape(t, 1, rot_dim)
    kr = plain.rotate_interleaved(kr, positions.tolist(), 5e4, 2 * pairs).reshape(t, rot_dim)  # the last 4 values pass
    row = torch.cat([c, kr, torch.zeros(t, width - kv_rank - rot_dim, dtype=torch.float64)], dim=1)
    kp, vp = k_pool.float().cpu(), v_pool.float().cpu()
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        assert rel(kp[s // page, 0, s % page], row[i]) <= tol(dtype, bf16=2.0 ** -7)
        assert torch.equal(vp[s // page, 0, :, s % page], kp[s // page, 0, s % page])
    written = torch.zeros(units * page, dtype=torch.bool)
    written[[s for s in slots.tolist() if s >= 0]] = True
    assert (kp.reshape(-1, width)[~written] == 7.0).all() and (vp.permute(0, 1, 3, 2).reshape(-1, width)[~written] == 7.0).all()
    # without pools: norms and gates only
    cq2, gate2 = ops.latent_prep(proj.cuda(), 7, q_rank, 0, kv_rank, rot_dim, pairs, 7 + q_rank + kv_rank + rot_dim, heads,
                                 wq.cuda(), None, 1e-5, table)
    assert torch.equal(cq2, cq) and torch.equal(gate2, gate)
    # queries: a matrix of its own for every head, then the turned part behind it
    dim, qh = 20, 20 + rot_dim
    q = rnd((t, heads * qh), 5).to(dtype)
    wk = rnd((heads, kv_rank, dim), 6, dim ** -0.5).to(dtype)
    qa = torch.full((t, heads * width), 5.0, dtype=dtype).cuda()
    ops.head_gemm(q.cuda(), 0, qh, wk.cuda(), qa, 0, width)
    ops.rope_pairs(q.cuda(), dim, qh, qa, kv_rank, width, heads, rot_dim, pairs, width - kv_rank, table)
    qd = q.double().reshape(t, heads, qh)
    ref = torch.cat([torch.einsum("thk,hnk->thn", qd[..., :dim], wk.double()),
                     plain.rotate_interleaved(qd[..., dim:], positions.tolist(), 5e4, 2 * pairs),
                     torch.zeros(t, heads, width - kv_rank - rot_dim, dtype=torch.float64)], dim=-1)
    assert rel(qa.float().cpu().reshape(t, heads, width), ref) <= tol(dtype, bf16=2.0 ** -7)
    # and back: the first kv_rank values of every head through W_uv,h, times the gate
    wv = rnd((heads, 9, kv_rank), 7, kv_rank ** -0.5).to(dtype)
    y = torch.empty((t, heads * 9), dtype=dtype).cuda()
    ops.head_gemm(qa, 0, width, wv.cuda(), y, 0, 9, gate=gate)
    ref = torch.einsum("thk,hnk->thn", qa.double().cpu().reshape(t, heads, width)[..., :kv_rank], wv.double()) * gate.double().cpu().unsqueeze(-1)
    assert rel(y.float().cpu().reshape(t, heads, 9), ref) <= tol(dtype, bf16=2.0 ** -7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t, heads, k, n", [(5, 3, 8, 9), (16, 2, 40, 64), (17, 1, 64, 200), (100, 5, 96, 300), (33, 2, 24, 17)])
def test_head_gemm_on_rows_that_the_matrix_cores_take(ops, dtype, t, heads, k, n):
    """Heads whose values start at multiples of eight columns (the matrix-core kernel's condition in bfloat16):
    token counts around its tiles of sixteen and thirty-two, outputs that do not fill a tile or a wave, a K
    that is not a multiple of the instruction's thirty-two, gaps between the heads in x and in out, a gate; the
    columns of out that belong to no head stay as they were."""
    x_off, x_hs, out_off, out_hs = 16, k + 8, 3, n + 2
    x = rnd((t, x_off + heads * x_hs + 8), t).to(dtype)
    w = rnd((heads, n, k), n, k ** -0.5).to(dtype)
    gate = torch.sigmoid(rnd((t, heads), 3))
    for g in (None, gate):
        out = torch.full((t, out_off + heads * out_hs), 5.0, dtype=dtype).cuda()
        ops.head_gemm(x.cuda(), x_off, x_hs, w.cuda(), out, out_off, out_hs, gate=None if g is None else g.cuda())
        xs = x.double()[:, x_off:x_off + heads * x_hs].reshape(t, heads, x_hs)[..., :k]
        ref = torch.einsum("thk,hnk->thn", xs, w.double()) * (1.0 if g is None else g.double().unsqueeze(-1))
        got = out.float().cpu()
        assert rel(got[:, out_off:].reshape(t, heads, out_hs)[..., :n], ref) <= tol(dtype, f32=1e-5, bf16=2.0 ** -7)
        assert (got[:, :out_off] == 5.0).all() and (got[:, out_off:].reshape(t, heads, out_hs)[..., n:] == 5.0).all()


def attention_with_sinks(ops, case, heads, hd, sinks, scale, share_keys=True):
    from from_scratch_inference_engine_amd.parts.attention import paged_attention

    plan = {k: (torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v) for k, v in case["plan"].items()}
    cache = SimpleNamespace(k_pool=case["k_pool"].cuda(), v_pool=case["v_pool"].cuda(), block_tables=case["tables"].cuda(),
                            page_size=case["k_pool"].shape[2])
    q = case["q"].cuda()
    return paged_attention(q, heads * hd, cache, SimpleNamespace(**plan), heads, 1, hd, None, scale, q.shape[0],
                           sinks=None if sinks is None else sinks.cuda(), share_keys=share_keys).float().cpu()


def oracle_attention(q, k, v, heads, hd, past, sinks, scale):
    n, total = q.shape[0], k.shape[0]
    q = q.double().reshape(n, heads, hd)
    mask = torch.arange(total).unsqueeze(0) <= (past + torch.arange(n)).unsqueeze(1)
    out = []
    for h in range(heads):
        s = (q[:, h] @ k.double().t() * scale).masked_fill(~mask, float("-inf"))
        sink = sinks[h].double() if sinks is not None else torch.tensor(float("-inf"), dtype=torch.float64)
        out.append(plain.softmax_with_sink(s, sink) @ v.double())
    return torch.stack(out, dim=1).reshape(n, heads * hd)


@pytest.mark.parametrize("dtype, scalar, hd", [(torch.float32, True, 48), (torch.bfloat16, True, 48), (torch.bfloat16, False, 48),
                                               (torch.bfloat16, False, 64), (torch.bfloat16, False, 112),
                                               (torch.float32, True, 288), (torch.bfloat16, True, 288)])
def test_attention_with_sinks_on_every_kernel(ops, dtype, scalar, hd):
    """One kv head read by all heads, a sink per head in the denominator: decodes that are cut into items and
    merged, short and long portions (the long ones through the kernel that shares keys where it takes the head
    size), first tokens; sinks from far below to far above the scores, so that a row's weights sum to anything
    between nearly one and nearly nothing."""
    from test_kernels_gpu import paged_case
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    heads, page, scale = 5, 16, 0.3
    seqs = [(0, 1), (0, 2), (700, 1), (0, 150), (300, 2), (123, 70), (2100, 1), (500, 200)]
    sinks = torch.tensor([-30.0, -2.0, 0.5, 3.0, 9.0])
    AttentionPlanner.compute_units = 4096  # as on an idle device: decodes are cut into many items and merged
    try:
        case = paged_case(seqs, heads, 1, hd, page, dtype, seed=hd, scalar=scalar)
    finally:
        AttentionPlanner.compute_units = None
    assert case["plan"]["mfma"] == (not scalar) and case["plan"]["n_merges"] > 0 and case["plan"]["n_large"] > 0
    outs = [attention_with_sinks(ops, case, heads, hd, sinks, scale)]
    if not scalar and ops.attention_mfma_lds_ok(hd, page):
        outs.append(attention_with_sinks(ops, case, heads, hd, sinks, scale, share_keys=False))
    for out in outs:
        row = 0
        for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
            ref = oracle_attention(q, k, v, heads, hd, p, sinks, scale)
            # (the weights may sum to nearly nothing: compare at the scale of the values)
            err = (out[row:row + n].double() - ref).abs().max().item()
            # (float32: scores of a head of hd values reach sqrt(hd) times the scale, and their rounding is the weights')
            assert err <= (3e-6 * max(1.0, hd / 96) if dtype == torch.float32 else 2.0 ** -7) * v.abs().max().item(), f"past {p} new {n}: {err}"
            row += n
    # no sinks: as before
    out = attention_with_sinks(ops, case, heads, hd, None, scale)
    ref = oracle_attention(case["qs"][3], case["ks"][3], case["vs"][3], heads, hd, 0, None, scale)
    assert (out[4:154].double() - ref).abs().max() <= (3e-6 if dtype == torch.float32 else 2.0 ** -7) * case["vs"][3].abs().max()


@pytest.mark.parametrize("dtype, scalar", [(torch.float32, True), (torch.bfloat16, False)])
def test_attention_with_sinks_finds_far_keys_and_page_borders(ops, dtype, scalar):
    """For every query one key carries the softmax (its query and key are scaled up): far back, at the first
    position, on either side of a page's border, at the query's own position; a louder key right after the
    query's position must stay unseen.  The sink takes a known share of the weight."""
    from test_kernels_gpu import paged_case

    heads, hd, page, scale = 4, 64, 16, 1.0
    seqs = [(900, 1), (640, 3), (0, 40)]
    targets = {0: [3], 1: [15, 16, 642], 2: list(range(40))}   # key that query i of request s must find
    targets[2] = [0] * 20 + [17] * 10 + list(range(30, 40))

    def edit(qs, ks, vs):
        for s, (p, n) in enumerate(seqs):
            ks[s].mul_(0.05)
            for i in range(n):
                key = targets[s][i]
                direction = torch.zeros(hd)
                direction[(7 * s + i) % hd] = 1.0
                ks[s][key] += 6.0 * direction
                qs[s][i] = (4.0 * direction).repeat(heads) + 0.05 * qs[s][i]
                if p + i + 1 < p + n:  # a louder key where the query must not look
                    ks[s][p + i + 1] += 9.0 * direction
            for t in (qs[s], ks[s]):  # what the oracle sees is what the pools hold
                t.copy_(t.to(dtype).float())
    case = paged_case(seqs, heads, 1, hd, page, dtype, seed=3, edit=edit, scalar=scalar)
    # the chosen key's score is about 24: a sink of 24 takes about half of the weight, one of -5 nothing
    sinks = torch.tensor([24.0, -5.0, 24.0, -5.0])
    out = attention_with_sinks(ops, case, heads, hd, sinks, scale)
    row = 0
    for s, ((p, n), q, k, v) in enumerate(zip(seqs, case["qs"], case["ks"], case["vs"])):
        ref = oracle_attention(q, k, v, heads, hd, p, sinks, scale)
        got = out[row:row + n].double()
        assert (got - ref).abs().max() <= (1e-5 if dtype == torch.float32 else 2.0 ** -6) * v.abs().max()
        for i in range(n):
            chosen = v[targets[s][i]].double()
            head1 = got[i, hd:2 * hd]          # sink -5: nearly all weight on the chosen key
            assert (head1 - chosen).abs().max() <= 0.05 * chosen.abs().max() + 0.02, (s, i)
            head0 = got[i, :hd]                # sink 24: the weights sum to well below one
            assert head0.abs().max() < 0.9 * chosen.abs().max()
        row += n


# ------------------------------------------------------------------------------------------------
# whole models
# ------------------------------------------------------------------------------------------------
def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, dims=None, kv_from=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale or (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim if dims is None else dims}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# Two configurations that differ from each other in every size and in the order of their layers.
# A: starts with attention, a layer without feed-forward, a layer that borrows the first one's latent with other
#    head counts, a second latent of another width (a second pool), sizes that are no multiples of 8, a cap.
# B: starts and ends with linear attention, one head, a cache row of 128 values (the kernel that shares keys),
#    partly rotated key part, no cap, key channels beyond 128.
CONFIG_A = {"architecture": "Gilozen", "width": 88, "vocab": 211, "norm": {"eps": 1e-6}, "logit_softcap": 6.0, "layers": [
    layer("latent_attention", latent(3, 20, 8, 12, 36, 44), 100),
    layer("gla", {"heads": 3, "dim": 20, "vdim": 28, "tau": 5.0}, None),
    layer("latent_attention", latent(5, 12, 8, 16, 36, 24, kv_from=0), 60),
    layer("gla", {"heads": 2, "dim": 36, "vdim": 70, "tau": 11.0}, 72),
    layer("latent_attention", latent(2, 24, 16, 40, 72, 30, base=500.0), None),
]}
CONFIG_B = {"architecture": "Gilozen", "width": 128, "vocab": 300, "norm": {"eps": 1e-5}, "layers": [
    layer("gla", {"heads": 1, "dim": 132, "vdim": 64, "tau": 2.0}, 256),
    layer("latent_attention", latent(4, 32, 32, 32, 96, 64, dims=16), 128),
    layer("latent_attention", latent(1, 48, 32, 24, 96, 40, dims=16, kv_from=1), 128),
    layer("gla", {"heads": 4, "dim": 16, "vdim": 16, "tau": 16.0}, None),
]}
# C: a cache row beyond the matrix-core kernels' 256 values (both precisions then take the float32-arithmetic kernel)
CONFIG_C = {"architecture": "Gilozen", "width": 64, "vocab": 150, "norm": {"eps": 1e-5}, "logit_softcap": 20.0, "layers": [
    layer("latent_attention", latent(2, 16, 16, 24, 270, 48), 96),
    layer("gla", {"heads": 2, "dim": 16, "vdim": 32, "tau": 4.0}, 96),
]}
# D: linear attention only (no paged cache at all); E: attention only (no state slots), the last layer borrowing
CONFIG_D = {"architecture": "Gilozen", "width": 48, "vocab": 97, "norm": {"eps": 1e-5}, "logit_softcap": 9.0, "layers": [
    layer("gla", {"heads": 2, "dim": 24, "vdim": 40, "tau": 3.0}, 64),
    layer("gla", {"heads": 1, "dim": 40, "vdim": 24, "tau": 1.0}, None),
]}
CONFIG_E = {"architecture": "Gilozen", "width": 56, "vocab": 120, "norm": {"eps": 1e-6}, "layers": [
    layer("latent_attention", latent(2, 16, 8, 24, 40, 32), None),
    layer("latent_attention", latent(4, 8, 16, 8, 24, 16, base=100.0), 80),
    layer("latent_attention", latent(3, 24, 8, 16, 40, 48, kv_from=0), 48),
]}
DECAY_RANK = {"A": 12, "B": 8, "C": 4, "D": 6, "E": 1}


def gilozen_tensors(cfg, rank, seed):
    g = torch.Generator().manual_seed(seed)
    w, out = cfg["width"], {}

    def mat(name, rows, cols):
        out[name] = torch.randn(rows, cols, generator=g) * cols ** -0.5

    def vec(name, n, spread, centre=0.0):
        out[name] = centre + torch.randn(n, generator=g) * spread
    mat("embed", cfg["vocab"], w)
    out["embed"] *= w ** 0.5
    mat("head", cfg["vocab"], w)
    vec("final.norm", w, 0.3)
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        vec(p + "norm1", w, 0.3), vec(p + "norm1b", w, 0.3)
        if lay["type"] == "gla":
            kw, vw = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            mat(p + "mix.q", kw, w), mat(p + "mix.k", kw, w), mat(p + "mix.v", vw, w), mat(p + "mix.g", vw, w)
            mat(p + "mix.a1", rank, w), mat(p + "mix.a2", kw, rank), vec(p + "mix.a2.b", kw, 2.0, 2.0)
            vec(p + "mix.norm", m["vdim"], 0.3, 1.0), mat(p + "mix.o", w, vw)
        else:
            h = m["heads"]
            mat(p + "mix.dq", m["q_rank"], w), vec(p + "mix.dq.norm", m["q_rank"], 0.3, 1.0)
            mat(p + "mix.uq", h * (m["dim"] + m["rot_dim"]), m["q_rank"])
            out[p + "mix.uq"] *= 3.0  # peaked softmax rows
            if "kv_from" not in m:
                mat(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], w), vec(p + "mix.dkv.norm", m["kv_rank"], 0.3, 1.0)
            mat(p + "mix.uk", h * m["dim"], m["kv_rank"]), mat(p + "mix.uv", h * m["vdim"], m["kv_rank"])
            vec(p + "mix.sink", h, 2.0), mat(p + "mix.g", h, w), mat(p + "mix.o", w, h * m["vdim"])
        if lay["mlp"] is not None:
            vec(p + "norm2", w, 0.3), vec(p + "norm2b", w, 0.3)
            mat(p + "mlp.gate", lay["mlp"]["ff"], w), mat(p + "mlp.up", lay["mlp"]["ff"], w), mat(p + "mlp.down", w, lay["mlp"]["ff"])
    return {k: v.bfloat16().contiguous() for k, v in out.items()}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("gilozen")
    out = {}
    for name, cfg in (("A", CONFIG_A), ("B", CONFIG_B), ("C", CONFIG_C), ("D", CONFIG_D), ("E", CONFIG_E)):
        d = helpers.make_model_dir(root / name, cfg, 0, tensors=gilozen_tensors(cfg, DECAY_RANK[name], seed=len(name) + ord(name)))
        out[name] = (d, plain.read_config(d), plain.read_weights(d))
    return out


def close_enough(got, ref, dtype, what):
    """float32: 1e-4 of the largest logit; bfloat16: the difference's root mean square against the logits'."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    if dtype == "float32":
        assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max(), f"{what}: {np.abs(got - ref).max():.3e}"
    else:
        err = np.sqrt(((got - ref) ** 2).mean(-1)) / np.sqrt((ref ** 2).mean())
        assert err.max() <= 0.12, f"{what}: worst row {err.argmax()} off by {err.max():.3f} of the logits' size"


def step_through(runner, plan, seqs):
    """``plan``: steps of [(request, tokens)]; returns {request: logits of all its positions}.  A request is
    opened at its first entry and closed after its last token."""
    from from_scratch_inference_engine_amd.engine.context import StepEntry

    fed, caches, got = {r: 0 for r in seqs}, {}, {r: [] for r in seqs}
    for step in plan:
        entries = []
        for r, n in step:
            if r not in caches:
                caches[r] = runner.manager.open(r)
            entries.append(StepEntry(caches[r], seqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
        out = runner.step(entries).cpu().numpy()
        row = 0
        for (r, n) in step:
            got[r].append(out[row:row + n])
            row += n
            if fed[r] == len(seqs[r]):
                runner.manager.close(caches.pop(r))
        runner.manager.check_invariants()
    return {r: np.concatenate(v) for r, v in got.items() if v}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_model_whole_in_portions_decoded_and_batched(models, name, dtype):
    """The same requests whole, token by token (through the captured decode graphs), in portions down to two
    tokens and one, and in batches of unequal requests that start and end at different steps in a pool so
    small that pages and state slots are taken again: all against the plain implementation."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models[name]
    vocab = cfg["vocab"]
    seqs = {"a": helpers.token_ids(vocab, 75, 1), "b": helpers.token_ids(vocab, 1, 2), "c": helpers.token_ids(vocab, 33, 3),
            "d": helpers.token_ids(vocab, 130, 4), "e": helpers.token_ids(vocab, 18, 5)}
    ref = {r: plain.forward(cfg, w, ids).numpy() for r, ids in seqs.items()}
    model = load_model(d, dtype=dtype)
    assert len(model.cache_layout.paged_groups) == (2 if name == "A" else 1)
    runner = Runner(model, page_size=8, num_pages=34, max_requests=3)
    assert runner.graphs.enabled
    # whole, one after the other (each takes the pages and the slot the last one gave back)
    got = step_through(runner, [[(r, len(ids))] for r, ids in seqs.items()], seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} whole {r}")
    # a first portion, then token by token: decode steps replay graphs, the state and the cache go on
    for r, head in (("a", 40), ("c", 1)):
        got = step_through(runner, [[(r, head)]] + [[(r, 1)]] * (len(seqs[r]) - head), {r: seqs[r]})
        close_enough(got[r], ref[r], dtype, f"{name} decode {r}")
    assert runner.graphs.replays > 50
    # portions of changing size
    sizes, plan, left = [2, 7, 1, 16, 3, 2, 33, 8, 64], [], len(seqs["d"])
    while left:
        n = min(sizes[len(plan) % len(sizes)], left)
        plan.append([("d", n)])
        left -= n
    close_enough(step_through(runner, plan, {"d": seqs["d"]})["d"], ref["d"], dtype, f"{name} portions")
    # batches: three slots, five requests; portions beside single tokens; b and e start where a and c ended
    plan = [[("a", 30), ("c", 2), ("b", 1)], [("a", 1), ("c", 20), ("e", 3)], [("c", 11), ("a", 44), ("e", 1)],
            [("e", 14), ("d", 9)], [("d", 120)], [("d", 1)]]
    got = step_through(runner, plan, seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} batched {r}")
    assert all(a.pages_issued_again() for a in runner.manager.allocators)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["D", "E"])
def test_model_of_one_kind_of_layer(models, name, dtype):
    """A model with state slots and no paged cache, and one with a paged cache and no state: whole, a portion and
    then token by token, and two requests of unequal length together, in a pool that is used again."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models[name]
    seqs = {"a": helpers.token_ids(cfg["vocab"], 70, 1), "b": helpers.token_ids(cfg["vocab"], 23, 2)}
    ref = {r: plain.forward(cfg, w, ids).numpy() for r, ids in seqs.items()}
    runner = Runner(load_model(d, dtype=dtype), page_size=8, num_pages=14, max_requests=2)
    got = step_through(runner, [[(r, len(ids))] for r, ids in seqs.items()], seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} whole {r}")
    got = step_through(runner, [[("a", 37)]] + [[("a", 1)]] * 33, {"a": seqs["a"]})
    close_enough(got["a"], ref["a"], dtype, f"{name} decode")
    got = step_through(runner, [[("a", 50), ("b", 2)], [("a", 19), ("b", 1)], [("a", 1), ("b", 17)], [("b", 3)]], seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} batched {r}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_model_with_cache_rows_beyond_256_values(models, dtype):
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models["C"]
    seqs = {"a": helpers.token_ids(cfg["vocab"], 90, 1), "b": helpers.token_ids(cfg["vocab"], 21, 2)}
    ref = {r: plain.forward(cfg, w, ids).numpy() for r, ids in seqs.items()}
    model = load_model(d, dtype=dtype)
    assert model.cache_layout.paged_groups[0].head_dim == 288
    runner = Runner(model, page_size=16, num_pages=12, max_requests=2)
    got = step_through(runner, [[("a", 50), ("b", 2)], [("a", 39), ("b", 1)]] + [[("a", 1), ("b", 1)]] + [[("b", 1)]] * 17, seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"C {r}")


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(models, name):
    """Prompts of unequal length generated together through the LLM entry point and its scheduler (three at a
    time, portions of at most 16 tokens), in float32: the tokens are the plain implementation's greedy ones; long
    enough that decode steps run from graphs and pages fill up."""
    from from_scratch_inference_engine_amd import GenerationConfig, LLM

    d, cfg, w = models[name]
    prompts = [helpers.token_ids(cfg["vocab"], n, 20 + n) for n in (1, 9, 40, 23)]
    n_new = 48
    llm = LLM(d, dtype="float32", block_size=8, num_blocks=64, max_batch=3, eos_id=-1, prefill_chunk=16)
    got = llm.generate_ids_batch(prompts, GenerationConfig(max_tokens=n_new))
    for prompt, mine in zip(prompts, got):
        assert len(mine) == n_new
        logits = plain.forward(cfg, w, prompt + mine)[len(prompt) - 1:-1]
        top2 = logits.topk(2, dim=-1).values
        for i, tok in enumerate(mine):  # the plain choice, unless the two best are a rounding apart
            assert tok == int(logits[i].argmax()) or (top2[i, 0] - logits[i, tok]) <= 1e-4 * logits.abs().max(), (len(prompt), i)
    assert llm.engine.runner.graphs.replays > 0


@pytest.mark.parametrize("name", ["A", "D", "E"])
def test_replay_program_runs_the_model(models, tmp_path, name):
    """bin/trace_run on the architecture (mixed layers, state only, cache only): a prompt in portions beside
    another request's single tokens."""
    d, cfg, w = models[name]
    a, b = helpers.token_ids(cfg["vocab"], 50, 7), helpers.token_ids(cfg["vocab"], 20, 8)
    tb = helpers.TraceBuilder()
    tb.step([("a", a[:17], [16]), ("b", b[:1], [0])])
    for i in range(1, 20):
        lo, hi = 17 + (i - 1) * 2, min(50, 17 + i * 2)
        entries = [("b", b[i:i + 1], [0])] + ([("a", a[lo:hi], list(range(hi - lo)))] if lo < 50 else [])
        tb.step(entries, end=["b"] if i == 19 else [])
    tb.step([], end=["a"])
    for dtype in ("float32", "bfloat16"):
        per = helpers.collect(tb, helpers.run_trace(d, dtype, tb.steps, 128, tmp_path / dtype))
        for rid, ids in (("a", a), ("b", b)):
            ref = plain.forward(cfg, w, ids).numpy()
            pos = sorted(per[rid])
            close_enough(np.stack([per[rid][p] for p in pos]), ref[pos], dtype, f"replay {rid}")


def test_command_line_writes_a_random_model_and_generates(tmp_path):
    """random-model from a config.json that states the decays' rank (``a_rank``; a folder's config.json may leave
    it to the checkpoint), then generate from that folder and, without a folder, from the configuration and the
    seed: the same weights, so the same tokens."""
    import copy
    import os
    import subprocess
    import sys

    raw = copy.deepcopy(CONFIG_A)
    for lay in raw["layers"]:
        if lay["type"] == "gla":
            lay["mixer"]["a_rank"] = 6
    (tmp_path / "cfg.json").write_text(json.dumps(raw))
    env = dict(os.environ, PYTHONPATH=str(helpers.ROOT))
    base = [sys.executable, "-m", "from_scratch_inference_engine_amd"]
    made = subprocess.run(base + ["random-model", "--config", str(tmp_path / "cfg.json"), "--out", str(tmp_path / "m"), "--seed", "5"],
                          capture_output=True, text=True, env=env, timeout=300)
    assert made.returncode == 0, made.stderr[-2000:]
    common = ["--prompt-ids", "3 1 4 1 5 9 2 6", "--max-tokens", "12", "--num-blocks", "64", "--max-batch", "4", "--dtype", "float32"]
    a = subprocess.run(base + ["generate", "--model-dir", str(tmp_path / "m")] + common, capture_output=True, text=True, env=env, timeout=300)
    b = subprocess.run(base + ["generate", "--config", str(tmp_path / "cfg.json"), "--random-weights", "5"] + common,
                       capture_output=True, text=True, env=env, timeout=300)
    assert a.returncode == 0 and b.returncode == 0, a.stderr[-2000:] + b.stderr[-2000:]
    tokens = a.stdout.strip().splitlines()[-1].split()
    assert len(tokens) == 12 and all(0 <= int(t) < raw["vocab"] for t in tokens)
    cfg, w = plain.read_config(tmp_path / "m"), plain.read_weights(tmp_path / "m")
    ids = [3, 1, 4, 1, 5, 9, 2, 6] + [int(t) for t in tokens]
    logits = plain.forward(cfg, w, ids)[7:-1]
    for i, t in enumerate(tokens):
        assert int(t) == int(logits[i].argmax()) or (logits[i].max() - logits[i, int(t)]) <= 1e-4 * logits.abs().max(), i
    # the folder's weights are bfloat16 roundings of the seed's float32 values: the same tokens unless two are a rounding apart
    assert b.stdout.strip().splitlines()[-1].split()[:4] == tokens[:4]
