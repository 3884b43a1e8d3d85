"""Botulorn on the GPU against the plain implementation (plain_botulorn.py): every mechanism alone, then whole
models of small configurations through the step function, the scheduler and the replay program.

The weights are drawn here with a spread that keeps activations of order one (standard deviation fan_in^-1/2,
wide norm weights and biases, value-mixing weights far from 0), and the q and k head norms are scaled up so that
softmax rows are peaked: a key that is wrongly seen or missed, a value that is not mixed, a pair row that is off by
one then moves the logits far beyond rounding."""

import json
import math
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_botulorn as plain

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
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


def tol(dtype, f32=2e-5, bf16=2.0 ** -6):
    return f32 if dtype == torch.float32 else bf16


def as_dtype(t, dtype):
    """The values a tensor has once stored in ``dtype``, as float64 numpy (what the oracle is given)."""
    return t.to(dtype).double().numpy()


# ------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, parts_a, parts_b", [(96, None, None), (257, 0, 3), (4100, 0, 0), (1024, 8, 0), (72, 2, 5),
                                                      (6000, None, 0)])
def test_layer_norm_adds_two_deltas_and_gives_two_outputs(ops, dtype, hidden, parts_a, parts_b):
    """residual + delta + delta2 (each absent, whole, or partial sums), one pass for two norms of the same
    stream, the sum written back; and chosen rows without writing back."""
    t, eps = 7, 1e-5
    res = rnd((t, hidden), 1, 3.0) + 0.7  # (a mean that is not zero: a norm that forgets to centre shows)

    def delta(parts, seed):
        if parts is None:
            return None
        return rnd((t, hidden), seed).to(dtype) if parts == 0 else rnd((parts, t, hidden), seed)
    d1, d2 = delta(parts_a, 2), delta(parts_b, 3)
    w1, b1, w2, b2 = rnd((hidden,), 4) + 1.0, rnd((hidden,), 5), rnd((hidden,), 6) + 1.0, rnd((hidden,), 7)
    total = res.double()
    for d in (d1, d2):
        if d is not None:
            total = total + (d.double().sum(0) if d.ndim == 3 else d.double())
    ref1 = plain.layer_norm(total.numpy(), w1.double().numpy(), b1.double().numpy(), eps)
    ref2 = plain.layer_norm(total.numpy(), w2.double().numpy(), b2.double().numpy(), eps)
    dev = lambda x: None if x is None else x.cuda()
    r = res.clone().cuda()
    o1, o2 = ops.layer_norm(r, w1.cuda(), b1.cuda(), eps, dtype, delta=dev(d1), delta2=dev(d2), weight2=w2.cuda(),
                            bias2=b2.cuda(), write_back=True)
    assert rel(o1.float().cpu(), ref1) <= tol(dtype) and rel(o2.float().cpu(), ref2) <= tol(dtype)
    assert rel(r.cpu(), total) <= 1e-6
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    r = res.clone().cuda()
    o = ops.layer_norm(r, w1.cuda(), b1.cuda(), eps, dtype, delta=dev(d1), delta2=dev(d2), rows=rows.cuda())
    assert rel(o.float().cpu(), ref1[rows.long().numpy()]) <= tol(dtype)
    assert torch.equal(r.cpu(), res)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("buckets, mul_prev, mul_cur", [(37, 5, 1), (1, 1, 1), (1000003, 99991, 7919)])
def test_pair_embedding_over_portions_steps_and_slots(ops, dtype, buckets, mul_prev, mul_cur):
    """Three requests fed in unequal portions over several steps, one of them in a slot that another request
    has used: every row is the token's row times the scale plus the row that the hash of (previous, token) names,
    the previous token coming from the same portion or from the slot's state; a request's first token takes the
    last row.  (The large table is stood in for by one of 50 rows: only the hash's arithmetic is at stake.)"""
    vocab, hidden, scale = 70000, 20, 2.5
    rows = min(buckets, 49) + 1
    table, pairs = rnd((vocab, hidden), 1).to(dtype), rnd((rows, hidden), 2).to(dtype)
    n_buckets = rows - 1
    if n_buckets != buckets:  # keep the multipliers' size, shrink the modulus
        buckets = n_buckets
    seqs = {"a": helpers.token_ids(vocab, 9, 1), "b": helpers.token_ids(vocab, 4, 2), "c": helpers.token_ids(vocab, 6, 3)}
    last = torch.zeros((4, 1), dtype=torch.int32).cuda()
    last[2] = 55  # what an earlier request left in slot 2
    slot = {"a": 0, "b": 2, "c": 1}
    plan = [[("a", 3), ("b", 1)], [("b", 2), ("a", 1)], [("a", 5), ("b", 1)], [("c", 6)]]
    fed = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    for step in plan:
        ids, starts, slots, reset = [], [0], [], []
        for r, n in step:
            if r == "c":
                slot["c"] = slot["b"]  # b has ended: c takes its slot
            if fed[r] == 0:
                reset.append(slot[r])
            ids += seqs[r][fed[r]:fed[r] + n]
            starts.append(starts[-1] + n)
            slots.append(slot[r])
        for s in reset:
            last[s] = 0  # (the engine zeroes the slots of the requests that start)
        out = ops.pair_embedding(table.cuda(), pairs.cuda(), torch.tensor(ids, dtype=torch.int32).cuda(),
                                 torch.tensor(starts, dtype=torch.int32).cuda(), torch.tensor(slots, dtype=torch.int32).cuda(),
                                 last, mul_prev, mul_cur, scale).cpu()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at += n
            fed[r] += n
    for r, ids in seqs.items():
        ref = plain.embed(ids, table.double().numpy(), scale, pairs.double().numpy(), buckets, mul_prev, mul_cur)
        assert rel(torch.cat(got[r]), ref) <= 1e-6, r


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t, page", [(11, 4), (83, 8), (299, 8)])
@pytest.mark.parametrize("heads, kv, dim, vdim, rot, stretch, norms",
                         [(6, 3, 24, 40, 16, (4.0, 32.0, 8.0, 2.0), True), (4, 4, 64, 16, 64, None, True),
                          (2, 1, 32, 32, 0, None, False), (3, 1, 20, 7, 10, (1.0, 64.0, 4.0, 1.0), True)])
def test_attention_prep_and_gate(ops, dtype, t, page, heads, kv, dim, vdim, rot, stretch, norms):
    """The kernel between projection and attention against the plain functions: head norms, the rotation of the
    first ``rot`` values with stretched frequencies, values blended with another layer's, gates; what lands in the
    pools at the tokens' slots (padded heads, zeros at the end, nothing elsewhere).  A few tokens at scattered
    slots, and a portion of a prompt whose values go eight slots at a time where they lie so."""
    from from_scratch_inference_engine_amd.parts.rope import RotaryEncoding

    eps, lam = 1e-5, 0.35
    padded = dim if dim == vdim else -(-max(dim, vdim) // 16) * 16
    width = heads * dim + kv * dim + kv * vdim + heads
    proj = rnd((t, width + 3), 1).to(dtype)  # (rows longer than what is used)
    other = rnd((t, kv * vdim + 5), 2).to(dtype)
    qw, kw = (rnd((dim,), 3) + 1.0, rnd((dim,), 4) + 1.0) if norms else (None, None)
    positions = ((torch.arange(t) * 389) % 1500).to(torch.int32)
    positions[:3] = torch.tensor([0, 1, 2], dtype=torch.int32)
    table = None
    rot_cfg = {"base": 500.0, "dims": rot}
    if stretch is not None:
        rot_cfg["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    if rot:
        enc = RotaryEncoding(dim, 500.0, rotary_dim=rot, layout="half", stretch=stretch)
        enc.prepare("cuda", dtype)
        table = ops.rope_table(positions.cuda(), enc.inv_freq, enc.magnitude)
    # the first half of the tokens from a slot in the middle of a page, the second half from a page's start
    # (whole runs of eight slots there), one token without a slot, the last ones in a page of their own
    half = t // 2 if t < 16 else (t // 2) // 8 * 8  # (a run of eight starts at a token whose number is a multiple of eight)
    slots = torch.cat([page * 2 + 1 + torch.arange(half), page * (4 + half // page) + torch.arange(t - half)]).to(torch.int32)
    slots[5] = -1
    slots[-2:] = slots[-3] + 2 * page + torch.arange(2, dtype=torch.int32)
    units = int(slots.max()) // page + 2
    k_pool = torch.full((units, kv, page, padded), 7.0, dtype=dtype).cuda()
    v_pool = torch.full((units, kv, padded, page), -9.0, dtype=dtype).cuda()
    k_off, v_off = heads * dim, heads * dim + kv * dim
    g_off = v_off + kv * vdim
    q, gate = ops.attention_prep(proj.cuda(), 0, k_off, v_off, g_off, heads, kv, dim, vdim, padded,
                                 None if qw is None else qw.cuda(), None if kw is None else kw.cuda(), eps, rot // 2, table,
                                 True, v_other=other.cuda()[:, :kv * vdim], v_other_stride=other.shape[1],
                                 mix=torch.tensor(lam).cuda(), slots=slots.cuda(), k_pool=k_pool, v_pool=v_pool)
    p64 = proj.double().numpy()
    qr, kr = p64[:, :k_off].reshape(t, heads, dim), p64[:, k_off:v_off].reshape(t, kv, dim)
    if norms:
        qr, kr = plain.rms_norm(qr, qw.double().numpy(), eps), plain.rms_norm(kr, kw.double().numpy(), eps)
    qr, kr = plain.rotate_half(qr, positions.numpy(), rot_cfg), plain.rotate_half(kr, positions.numpy(), rot_cfg)
    vr = (1 - lam) * p64[:, v_off:g_off].reshape(t, kv, vdim) + lam * other.double().numpy()[:, :kv * vdim].reshape(t, kv, vdim)
    gr = plain.sigmoid(p64[:, g_off:g_off + heads])
    qg = q.float().cpu().numpy().reshape(t, heads, padded)
    assert rel(qg[..., :dim], qr) <= tol(dtype) and not qg[..., dim:].any()
    assert rel(gate.cpu(), gr) <= 1e-6
    kp, vp = k_pool.float().cpu().numpy(), v_pool.float().cpu().numpy()
    written = set()
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        u, o = divmod(s, page)
        written.add((u, o))
        assert rel(kp[u, :, o, :dim], kr[i]) <= tol(dtype) and not kp[u, :, o, dim:].any()
        assert rel(vp[u, :, :vdim, o], vr[i]) <= tol(dtype) and not vp[u, :, vdim:, o].any()
    for u in range(units):
        for o in range(page):
            if (u, o) not in written:
                assert (kp[u, :, o] == 7.0).all() and (vp[u, :, :, o] == -9.0).all()
    # after attention: the first vdim values of every padded head, times the gate
    x = rnd((t, heads * padded), 9).to(dtype)
    y = ops.gate_heads(x.cuda(), padded, vdim, heads, gate).float().cpu().numpy()
    ref = x.double().numpy().reshape(t, heads, padded)[..., :vdim] * gr[..., None]
    assert rel(y.reshape(t, heads, vdim), ref) <= tol(dtype)


# ------------------------------------------------------------------------------ attention with kept first keys
def kept_case(seqs, heads, kv, hd, page, dtype, window, keep, seed, scalar, edit=None):
    """Pools, tables and the planner's items for requests (past, new) of an attention whose window keeps the first
    ``keep`` keys: the pages that the window has passed are gone from the tables (as the cache manager hands them
    back), except those of the kept keys."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-(p + n) // page) for p, n in seqs) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    k_pool, v_pool = torch.full((n_pages, kv, page, hd), 7.0), torch.full((n_pages, kv, hd, page), -9.0)
    tables = torch.full((len(seqs), max(-(-(p + n) // page) for p, n in seqs)), -1, dtype=torch.int32)
    qs, ks, vs = [], [], []
    for p, n in seqs:
        qs.append(torch.randn(n, heads * hd, generator=g).to(dtype).float())
        ks.append(torch.randn(p + n, kv * hd, generator=g).to(dtype).float())
        vs.append(torch.randn(p + n, kv * hd, generator=g).to(dtype).float())
    if edit is not None:
        edit(qs, ks, vs)
    for s, (p, n) in enumerate(seqs):
        total, held = p + n, -(-(p + n) // page)
        dead = max(0, p - window + 1) // page  # pages that no query of this step reads through its window
        kept_pages = -(-keep // page) if keep else 0
        k_all, v_all = torch.full((held * page, kv, hd), 7.0), torch.full((held * page, kv, hd), -9.0)
        k_all[:total], v_all[:total] = ks[s].reshape(total, kv, hd), vs[s].reshape(total, kv, hd)
        for i in range(held):
            if kept_pages <= i < dead:
                continue
            unit = order.pop()
            tables[s, i] = unit
            k_pool[unit] = k_all[i * page:(i + 1) * page].permute(1, 0, 2)
            v_pool[unit] = v_all[i * page:(i + 1) * page].permute(1, 2, 0)
    host = SimpleNamespace(n_seqs=len(seqs), q_lens=[n for _, n in seqs], past_lens=[p for p, _ in seqs], q_starts=[0],
                           page_size=page, compute_dtype=torch.float32 if scalar else dtype, pad=None)
    for _, n in seqs:
        host.q_starts.append(host.q_starts[-1] + n)
    host.n_tokens = host.q_starts[-1]
    plan = AttentionPlanner(heads, kv, hd, window, keep).plan(host)
    return dict(q=torch.cat(qs).to(dtype), k_pool=k_pool.to(dtype), v_pool=v_pool.to(dtype), tables=tables, plan=plan,
                qs=qs, ks=ks, vs=vs)


def run_kept(case, heads, kv, hd, window, scale, share_keys=True):
    from from_scratch_inference_engine_amd.parts.attention import paged_attention

    plan = {k: (torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v) for k, v in case["plan"].items()}
    cache = SimpleNamespace(k_pool=case["k_pool"].cuda(), v_pool=case["v_pool"].cuda(), block_tables=case["tables"].cuda(),
                            page_size=case["k_pool"].shape[2])
    q = case["q"].cuda()
    return paged_attention(q, heads * hd, cache, SimpleNamespace(**plan), heads, kv, hd, window, scale, q.shape[0],
                           share_keys=share_keys).float().cpu().numpy()


def oracle_kept(q, k, v, heads, kv, hd, past, window, keep, scale):
    total, n = k.shape[0], q.shape[0]
    mask = plain.visible(total, window, keep)[past:]
    rep = heads // kv
    kk = np.repeat(k.double().numpy().reshape(total, kv, hd), rep, axis=1)
    vv = np.repeat(v.double().numpy().reshape(total, kv, hd), rep, axis=1)
    s = np.einsum("ihd,jhd->hij", q.double().numpy().reshape(n, heads, hd), kk) * scale
    s = np.where(mask[None], s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return np.einsum("hij,jhe->ihe", p, vv).reshape(n, heads * hd)


def kernel_families():
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    out = [(torch.float32, True), (torch.bfloat16, True)]
    if AttentionPlanner.mfma_keeps_first:
        out.append((torch.bfloat16, False))
    return out


@pytest.mark.parametrize("family", range(3))
@pytest.mark.parametrize("heads, kv, hd, window, keep, page", [(4, 2, 64, 80, 3, 16), (6, 1, 32, 40, 9, 8), (2, 2, 48, 17, 1, 16),
                                                               (8, 2, 128, 200, 35, 16)])
def test_attention_that_keeps_first_keys_on_every_kernel(ops, family, heads, kv, hd, window, keep, page):
    """Random queries and keys: decodes far past the window (cut into items and merged, the kept keys an item of
    their own), short and long portions whose windows have or have not left the kept keys, first tokens."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    families = kernel_families()
    if family >= len(families):
        pytest.skip("the matrix-core kernels do not read kept first keys")
    dtype, scalar = families[family]
    scale = 0.2
    seqs = [(0, 1), (0, 2), (700, 1), (0, 150), (300, 2), (123, 70), (2100, 1), (500, 200), (window + keep - 1, 3), (keep, 40)]
    outs = []
    for units in (4096, 1):  # an idle device (many short items, merged) and a full one (whole items)
        AttentionPlanner.compute_units = units
        try:
            case = kept_case(seqs, heads, kv, hd, page, dtype, window, keep, seed=hd + keep, scalar=scalar)
        finally:
            AttentionPlanner.compute_units = None
        assert case["plan"]["mfma"] == (not scalar)
        outs.append(run_kept(case, heads, kv, hd, window, scale))
        if not scalar and ops.attention_mfma_lds_ok(hd, page):
            outs.append(run_kept(case, heads, kv, hd, window, scale, share_keys=False))
    for out in outs:
        row = 0
        for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
            ref = oracle_kept(q, k, v, heads, kv, hd, p, window, keep, scale)
            err = np.abs(out[row:row + n] - ref).max()
            assert err <= (3e-6 if dtype == torch.float32 else 2.0 ** -7) * v.abs().max().item(), f"past {p} new {n}: {err}"
            row += n


@pytest.mark.parametrize("family", range(3))
def test_attention_finds_kept_keys_and_window_edges(ops, family):
    """For every query one key carries the softmax: the last kept key, the oldest key of the window, the query's own
    position, a key on either side of a page's border; and louder keys just outside (the first key that is not
    kept, the newest key the window has left, the key after the query) must stay unseen."""
    families = kernel_families()
    if family >= len(families):
        pytest.skip("the matrix-core kernels do not read kept first keys")
    dtype, scalar = families[family]
    heads, kv, hd, page, window, keep, scale = 4, 2, 64, 16, 48, 5, 1.0
    seqs = [(900, 1), (640, 4), (0, 62), (60, 3)]  # (at most hd queries a request: each has a direction of its own)
    # (request, query) -> the key it must find
    targets = {0: [4], 1: [640 - 47, 0, 642, 643 - 47], 2: None, 3: [4, 61 - 47, 16]}
    targets[2] = [min(i, 2) for i in range(30)] + [i - 47 if i >= 52 else 4 for i in range(30, 58)] + list(range(58, 62))
    targets[2][47] = 15
    targets[2][57] = 17

    def edit(qs, ks, vs):
        for s, (p, n) in enumerate(seqs):
            ks[s].mul_(0.05)
            for i in range(n):
                pos, key = p + i, targets[s][i]
                assert key <= pos and (pos - key < window or key < keep)
                direction = torch.zeros(hd)
                direction[(7 * s + 3 * i) % hd] = 1.0
                ks[s][key] += (6.0 * direction).repeat(kv)
                qs[s][i] = (4.0 * direction).repeat(heads) + 0.05 * qs[s][i]
                for hidden_key in (keep, pos - window, pos + 1):  # louder keys where the query must not look
                    if 0 <= hidden_key < p + n and hidden_key != key and not (hidden_key <= pos and (pos - hidden_key < window or hidden_key < keep)):
                        ks[s][hidden_key] += (9.0 * direction).repeat(kv)
            for t in (qs[s], ks[s]):
                t.copy_(t.to(dtype).float())
    case = kept_case(seqs, heads, kv, hd, page, dtype, window, keep, seed=5, scalar=scalar, edit=edit)
    out = run_kept(case, heads, kv, hd, window, scale)
    row = 0
    for s, ((p, n), q, k, v) in enumerate(zip(seqs, case["qs"], case["ks"], case["vs"])):
        ref = oracle_kept(q, k, v, heads, kv, hd, p, window, keep, scale)
        got = out[row:row + n]
        assert np.abs(got - ref).max() <= (1e-5 if dtype == torch.float32 else 2.0 ** -6) * v.abs().max().item(), s
        for i in range(n):
            chosen = v[targets[s][i]].double().numpy().reshape(kv, hd)
            for h in range(heads):
                mine = got[i, h * hd:(h + 1) * hd]
                assert np.abs(mine - chosen[h // (heads // kv)]).max() <= 0.06 * np.abs(chosen).max() + 0.03, (s, i, h)
        row += n


# ------------------------------------------------------------------------------------------------
# whole models
# ------------------------------------------------------------------------------------------------
def rotation(base, dims, stretch=None):
    rot = {"base": base, "dims": dims}
    if stretch is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    return rot


def attention(heads, kv, dim, vdim, window, keep, rot, scale=None, v_mix=False):
    mask = {"size": window}
    if keep is not None:
        mask["keep_first"] = keep
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": mask, "rot": rot, "scale": scale or dim ** -0.5}
    if v_mix:
        m["v_mix"] = True
    return m


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, rot, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "mask": {"size": window}, "rot": rot, "scale": scale or (dim + rot_dim) ** -0.5}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# A: starts with attention whose values are wider than its keys, partly rotated with stretched frequencies; a latent
#    layer without feed-forward; a second value-mixing layer with another window, more kept keys than a page holds
#    and one kv head a query head; a layer that mixes nothing, keeps nothing and has keys as wide as values.
# B: starts with latent attention (cache rows of 128 values, stretched), multipliers and buckets of 1, a scale of 1,
#    values narrower than keys, a window wider than any request, one kept key.
# C: attention only, one layer, grouped heads of 128 (the matrix-core kernels' widest tiles in bfloat16).
CONFIG_A = {"architecture": "Botulorn", "width": 72, "vocab": 150, "norm": {"eps": 1e-6},
            "embedding": {"scale": 3.5, "bigram": {"buckets": 37, "mul_prev": 5, "mul_cur": 1}}, "layers": [
    layer("attention", attention(6, 3, 24, 40, 20, 3, rotation(500.0, 16, (4.0, 32.0, 8.0, 2.0)), v_mix=True), 96),
    layer("latent_attention", latent(3, 16, 8, 12, 40, 28, 17, rotation(10000.0, 8)), None),
    layer("attention", attention(3, 3, 24, 40, 33, 9, rotation(100.0, 24), scale=0.3, v_mix=True), 64),
    layer("attention", attention(2, 1, 32, 32, 12, None, rotation(10000.0, 32, (2.0, 16.0, 4.0, 1.0))), 80),
]}
CONFIG_B = {"architecture": "Botulorn", "width": 128, "vocab": 300, "norm": {"eps": 1e-5},
            "embedding": {"scale": 1.0, "bigram": {"buckets": 1, "mul_prev": 1, "mul_cur": 1}}, "layers": [
    layer("latent_attention", latent(4, 32, 32, 32, 96, 64, 40, rotation(1000000.0, 32, (2.0, 64.0, 16.0, 1.0))), 128),
    layer("attention", attention(4, 4, 64, 16, 25, 1, rotation(10000.0, 64, (1.0, 64.0, 16.0, 1.0)), v_mix=True), 128),
    layer("latent_attention", latent(1, 48, 16, 24, 80, 40, 1000, rotation(50.0, 16)), None),
    layer("attention", attention(8, 2, 32, 48, 1000, 0, rotation(10000.0, 8)), 64),
]}
CONFIG_C = {"architecture": "Botulorn", "width": 64, "vocab": 97, "norm": {"eps": 1e-5},
            "embedding": {"scale": 8.0, "bigram": {"buckets": 501, "mul_prev": 1009, "mul_cur": 31}}, "layers": [
    layer("attention", attention(4, 2, 128, 128, 30, 6, rotation(10000.0, 64), v_mix=True), 96),
]}


# D: sizes that are multiples of nothing: a width that is no multiple of four, heads of 20 with values of 12 and five
#    rotated pairs, three query heads a kv head, more kept keys than the window is long, a latent of 50 + 6 values.
CONFIG_D = {"architecture": "Botulorn", "width": 90, "vocab": 101, "norm": {"eps": 1e-5},
            "embedding": {"scale": 0.5, "bigram": {"buckets": 4099, "mul_prev": 3, "mul_cur": 65537}}, "layers": [
    layer("latent_attention", latent(5, 10, 6, 14, 50, 22, 9, rotation(77.0, 6, (3.0, 8.0, 2.0, 1.0))), 50),
    layer("attention", attention(6, 2, 20, 12, 4, 10, rotation(1000.0, 10), v_mix=True), None),
    layer("attention", attention(2, 2, 28, 12, 64, 2, rotation(1000.0, 0), v_mix=True), 34),
]}


def botulorn_tensors(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    w = cfg["width"]

    def mat(rows, cols, gain=1.0):
        return torch.randn((rows, cols), generator=g) * (gain / math.sqrt(cols))

    def vec(n, centre, spread):
        return centre + torch.randn((n,), generator=g) * spread
    out = {"embed": torch.randn((cfg["vocab"], w), generator=g) / cfg["embedding"]["scale"],
           "bigram": torch.randn((cfg["embedding"]["bigram"]["buckets"] + 1, w), generator=g) * 0.7,
           "final.norm": vec(w, 1.0, 0.2), "final.norm.b": vec(w, 0.0, 0.2), "head": mat(cfg["vocab"], w, 2.0)}
    for i, lay in enumerate(cfg["layers"]):
        m, p = lay["mixer"], f"l{i}.mix."
        out[f"l{i}.norm1"], out[f"l{i}.norm1.b"] = vec(w, 1.0, 0.2), vec(w, 0.0, 0.2)
        if lay["type"] == "attention":
            h, kv, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "q": mat(h * d, w), p + "k": mat(kv * d, w), p + "v": mat(kv * e, w), p + "g": mat(h, w, 2.0),
                        p + "q.norm": vec(d, 2.0, 0.5), p + "k.norm": vec(d, 2.0, 0.5), p + "o": mat(w, h * e)})
            if m.get("v_mix"):
                out[p + "vmix"] = torch.tensor(0.35 + 0.1 * i)
        else:
            h, d, r, e = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            out.update({p + "dq": mat(m["q_rank"], w), p + "dq.norm": vec(m["q_rank"], 1.5, 0.3),
                        p + "uq": mat(h * (d + r), m["q_rank"], 2.0), p + "dkv": mat(m["kv_rank"] + r, w, 2.0),
                        p + "dkv.norm": vec(m["kv_rank"], 1.5, 0.3), p + "uk": mat(h * d, m["kv_rank"], 2.0),
                        p + "uv": mat(h * e, m["kv_rank"]), p + "o": mat(w, h * e)})
        if lay["mlp"] is not None:
            ff = lay["mlp"]["ff"]
            out[f"l{i}.norm2"], out[f"l{i}.norm2.b"] = vec(w, 1.0, 0.2), vec(w, 0.0, 0.2)
            out.update({f"l{i}.mlp.gate": mat(ff, w, 1.5), f"l{i}.mlp.up": mat(ff, w), f"l{i}.mlp.down": mat(w, ff)})
    return {k: v.to(torch.bfloat16).contiguous() for k, v in out.items()}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("botulorn")
    out = {}
    for name, cfg in (("A", CONFIG_A), ("B", CONFIG_B), ("C", CONFIG_C), ("D", CONFIG_D)):
        d = helpers.make_model_dir(root / name, cfg, 0, tensors=botulorn_tensors(cfg, seed=ord(name)))
        out[name] = (d, plain.read_config(d), plain.read_weights(d))
    return out


def close_enough(got, ref, dtype, what):
    """float32: 1e-4 of the largest logit; bfloat16: the difference's root mean square against the logits'."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    if dtype == "float32":
        bad = np.abs(got - ref).max(-1) > 1e-4 * np.abs(ref).max()
        assert not bad.any(), f"{what}: first wrong position {int(np.argmax(bad))}, {np.abs(got - ref).max():.3e}"
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


def test_the_plain_model_feels_every_mechanism(models):
    """The oracle itself: taking a mechanism away (the pair rows, the kept keys, the window, value mixing, the gate,
    the stretch of the frequencies) moves its logits by far more than the tolerances of the tests below."""
    import copy

    d, cfg, w = models["A"]
    ids = helpers.token_ids(cfg["vocab"], 90, 1)
    ref = plain.forward(cfg, w, ids)
    size = np.abs(ref).max()

    def moved(cfg2, w2):
        return np.abs(plain.forward(cfg2, w2, ids) - ref).max() / size
    c = copy.deepcopy(cfg)
    c["layers"][0]["mixer"]["mask"]["keep_first"] = 2
    assert moved(c, w) > 1e-3
    c = copy.deepcopy(cfg)
    c["layers"][0]["mixer"]["mask"]["size"] += 1
    assert moved(c, w) > 1e-3
    c = copy.deepcopy(cfg)
    c["layers"][1]["mixer"]["mask"]["size"] -= 1
    assert moved(c, w) > 1e-3
    c = copy.deepcopy(cfg)
    del c["layers"][0]["mixer"]["rot"]["scaling"]
    assert moved(c, w) > 1e-3
    c = copy.deepcopy(cfg)
    c["embedding"]["bigram"]["mul_cur"] = 2
    assert moved(c, w) > 1e-3
    for name, value in (("l2.mix.vmix", 0.0), ("l2.mix.g", 0.0), ("l0.norm2.b", 0.0)):
        w2 = dict(w)
        w2[name] = w[name] * value
        assert moved(cfg, w2) > 1e-3, name


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_model_whole_in_portions_decoded_and_batched(models, name, dtype):
    """The same requests whole, token by token (through the captured decode graphs, far enough that every window
    passes over decoded tokens), in portions down to two tokens and one, and in batches of unequal requests that
    start and end at different steps in a pool so small that pages and state slots are taken again."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models[name]
    vocab = cfg["vocab"]
    seqs = {"a": helpers.token_ids(vocab, 75, 1), "b": helpers.token_ids(vocab, 1, 2), "c": helpers.token_ids(vocab, 33, 3),
            "d": helpers.token_ids(vocab, 130, 4), "e": helpers.token_ids(vocab, 18, 5)}
    ref = {r: plain.forward(cfg, w, ids) for r, ids in seqs.items()}
    model = load_model(d, dtype=dtype)
    runner = Runner(model, page_size=8, num_pages=40, max_requests=3)
    assert runner.graphs.enabled
    got = step_through(runner, [[(r, len(ids))] for r, ids in seqs.items()], seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} whole {r}")
    for r, head in (("a", 10), ("c", 1)):
        got = step_through(runner, [[(r, head)]] + [[(r, 1)]] * (len(seqs[r]) - head), {r: seqs[r]})
        close_enough(got[r], ref[r], dtype, f"{name} decode {r}")
    assert runner.graphs.replays > 50
    sizes, plan, left = [2, 7, 1, 16, 3, 2, 33, 8, 64], [], len(seqs["d"])
    while left:
        n = min(sizes[len(plan) % len(sizes)], left)
        plan.append([("d", n)])
        left -= n
    close_enough(step_through(runner, plan, {"d": seqs["d"]})["d"], ref["d"], dtype, f"{name} portions")
    plan = [[("a", 30), ("c", 2), ("b", 1)], [("a", 1), ("c", 20), ("e", 3)], [("c", 11), ("a", 44), ("e", 1)],
            [("e", 14), ("d", 9)], [("d", 120)], [("d", 1)]]
    got = step_through(runner, plan, seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} batched {r}")
    assert all(a.pages_issued_again() for a in runner.manager.allocators)


def test_long_decoding_hands_pages_back_and_keeps_the_first(models):
    """Four hundred decoded tokens in float32 in a pool that holds a fraction of them: the windows hand their pages
    back, the pages of the kept first keys stay, and every logit is the plain one."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models["A"]
    ids = helpers.token_ids(cfg["vocab"], 400, 11)
    ref = plain.forward(cfg, w, ids)
    runner = Runner(load_model(d, dtype="float32"), page_size=8, num_pages=12, max_requests=1)
    got = step_through(runner, [[("a", 5)]] + [[("a", 1)]] * 395, {"a": ids})
    close_enough(got["a"], ref, "float32", "long decode")
    kept = [runner.manager.kept_pages(g) for g in range(len(runner.manager.groups))]
    assert sorted(kept) == [0, 0, 1, 2]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(models, name):
    """Prompts of unequal length generated together through the LLM entry point and its scheduler (three at a
    time, portions of at most 16 tokens), in float32: the tokens are the plain implementation's greedy ones."""
    from from_scratch_inference_engine_amd import GenerationConfig, LLM

    d, cfg, w = models[name]
    prompts = [helpers.token_ids(cfg["vocab"], n, 20 + n) for n in (1, 9, 40, 23)]
    n_new = 48
    llm = LLM(d, dtype="float32", block_size=8, num_blocks=64, max_batch=3, eos_id=-1, prefill_chunk=16)
    got = llm.generate_ids_batch(prompts, GenerationConfig(max_tokens=n_new))
    for prompt, mine in zip(prompts, got):
        assert len(mine) == n_new
        logits = plain.forward(cfg, w, prompt + mine)[len(prompt) - 1:-1]
        for i, tok in enumerate(mine):  # the plain choice, unless the two best are a rounding apart
            assert tok == int(logits[i].argmax()) or (logits[i].max() - logits[i, tok]) <= 1e-4 * np.abs(logits).max(), (len(prompt), i)
    assert llm.engine.runner.graphs.replays > 0


@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_program_runs_the_model(models, tmp_path, name):
    """bin/trace_run on the architecture: a prompt in portions beside another request's single tokens, then a third
    request in the slot and pages that the second gave back."""
    d, cfg, w = models[name]
    a, b, c = (helpers.token_ids(cfg["vocab"], n, 7 + n) for n in (50, 20, 9))
    tb = helpers.TraceBuilder()
    tb.step([("a", a[:17], [16]), ("b", b[:1], [0])])
    for i in range(1, 20):
        lo, hi = 17 + (i - 1) * 2, min(50, 17 + i * 2)
        entries = [("b", b[i:i + 1], [0])] + ([("a", a[lo:hi], list(range(hi - lo)))] if lo < 50 else [])
        tb.step(entries, end=["b"] if i == 19 else [])
    tb.step([("c", c, list(range(9)))], end=["a", "c"])
    for dtype in ("float32", "bfloat16"):
        per = helpers.collect(tb, helpers.run_trace(d, dtype, tb.steps, 128, tmp_path / dtype))
        for rid, ids in (("a", a), ("b", b), ("c", c)):
            ref = plain.forward(cfg, w, ids)
            pos = sorted(per[rid])
            close_enough(np.stack([per[rid][p] for p in pos]), ref[pos], dtype, f"replay {rid}")


def test_command_line_writes_a_random_model_and_generates(tmp_path):
    """random-model from a config.json, then generate from that folder and, without a folder, from the configuration
    and the seed: the architecture is served by the same command line as the others."""
    (tmp_path / "cfg.json").write_text(json.dumps(CONFIG_A))
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
    assert len(tokens) == 12 and all(0 <= int(t) < CONFIG_A["vocab"] for t in tokens)
    cfg, w = plain.read_config(tmp_path / "m"), plain.read_weights(tmp_path / "m")
    ids = [3, 1, 4, 1, 5, 9, 2, 6] + [int(t) for t in tokens]
    logits = plain.forward(cfg, w, ids)[7:-1]
    for i, t in enumerate(tokens):
        assert int(t) == int(logits[i].argmax()) or (logits[i].max() - logits[i, int(t)]) <= 1e-4 * np.abs(logits).max(), i
    assert len(b.stdout.strip().splitlines()[-1].split()) == 12
