"""Botulorn without a GPU: the configuration, the tensors the builder expects, the stretched frequencies against
the plain implementation's, the cache manager's kept first pages, and the attention planner's items for a window
that keeps a request's first keys."""

import copy
import random

import numpy as np
import pytest
import torch

import plain_botulorn as plain
from from_scratch_inference_engine_amd.cache.manager import CacheManager, PagedNeed
from from_scratch_inference_engine_amd.config.base import ConfigError
from from_scratch_inference_engine_amd.models.registry import build_model_spec, parse_config
from from_scratch_inference_engine_amd.parts.rope import RotaryEncoding
from from_scratch_inference_engine_amd.weights.loader import expected_tensors

RAW = {"architecture": "Botulorn", "width": 48, "vocab": 90, "norm": {"eps": 1e-6},
       "embedding": {"scale": 2.0, "bigram": {"buckets": 11, "mul_prev": 3, "mul_cur": 2}}, "layers": [
    {"type": "attention", "mlp": {"kind": "dense", "ff": 64},
     "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "v_mix": True,
               "mask": {"size": 10, "keep_first": 2},
               "rot": {"base": 100.0, "dims": 8, "scaling": {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 1.0}}}},
    {"type": "latent_attention", "mlp": None,
     "mixer": {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 12, "q_rank": 10, "scale": 0.3, "mask": {"size": 7},
               "rot": {"base": 50.0, "dims": 4}}},
    {"type": "attention", "mlp": {"kind": "dense", "ff": 32},
     "mixer": {"heads": 2, "kv_heads": 2, "dim": 12, "vdim": 24, "scale": 0.3, "v_mix": True, "mask": {"size": 5},
               "rot": {"base": 100.0, "dims": 12}}},
]}


def test_configuration_round_trip_and_tensors():
    cfg = parse_config(RAW)
    assert parse_config(cfg.to_dict()) == cfg
    assert cfg.layers[0].mixer.keep_first == 2 and cfg.layers[2].mixer.keep_first == 0
    assert cfg.layers[0].mixer.rot.stretch == (3.0, 16.0, 4.0, 1.0) and cfg.layers[1].mixer.rot.stretch is None
    spec = build_model_spec(cfg)
    names = {n: tuple(s.shape) for n, s in expected_tensors(spec.bindings).items()}
    assert names["bigram"] == (12, 48) and names["l0.mix.vmix"] == () and names["l2.mix.vmix"] == ()
    assert names["l0.mix.v"] == (48, 48) and names["l0.mix.g"] == (4, 48) and names["l0.mix.o"] == (48, 96)
    assert names["l1.mix.dkv"] == (16, 48) and names["l0.norm2.b"] == (48,) and "l1.norm2" not in names
    mixers = [layer.mixer for layer in spec.layers]
    assert mixers[0].value_mix == "source" and mixers[2].value_mix == "mixed"
    assert mixers[0].padded == 32 and mixers[0].cache_need() == PagedNeed(2, 32, 10, 2)
    assert mixers[1].cache_need().window == 7 and mixers[2].cache_need().keep_first == 0


@pytest.mark.parametrize("edit, message", [
    (lambda r: r["layers"][0]["mixer"]["mask"].pop("size"), "size"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda r: r["layers"][2]["mixer"].update(vdim=20), "agree"),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda r: r["layers"][1].update(type="gla"), "not a mixer"),
    (lambda r: r["embedding"].pop("bigram"), "bigram"),
    (lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].update(factor=0.5), "factor"),
])
def test_configuration_refuses(edit, message):
    raw = copy.deepcopy(RAW)
    edit(raw)
    with pytest.raises(ConfigError, match=message):
        parse_config(raw)


@pytest.mark.parametrize("rot", [{"base": 20000.0, "dims": 48, "scaling": {"factor": 6.0, "original": 256, "fast": 24.0, "slow": 0.5}},
                                 {"base": 500.0, "dims": 16, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}},
                                 {"base": 1e6, "dims": 24, "scaling": {"factor": 1.0, "original": 100, "fast": 3.0, "slow": 3.0}},
                                 {"base": 100.0, "dims": 6}])
def test_stretched_frequencies_are_the_plain_ones(rot):
    sc = rot.get("scaling")
    enc = RotaryEncoding(rot["dims"] + 8, rot["base"], rotary_dim=rot["dims"], layout="half",
                         stretch=None if sc is None else (sc["factor"], sc["original"], sc["fast"], sc["slow"]))
    f, m = plain.yarn_frequencies(rot)
    assert np.allclose(enc.frequencies(), f, rtol=1e-14, atol=0) and abs(enc.magnitude - m) < 1e-15
    if sc is not None and sc["factor"] > 1:
        plain_f = np.array([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)])
        assert (f <= plain_f * (1 + 1e-12)).all() and (f >= plain_f / sc["factor"] * (1 - 1e-12)).all() and (f < plain_f).any()


def test_cache_manager_keeps_the_first_pages():
    """A window hands its pages back, except those of the kept first keys; a request that ends gives everything back."""
    m = CacheManager([PagedNeed(1, 8, 10, 5), PagedNeed(1, 8, 10, 0), PagedNeed(2, 8, None)], 4, 40, 2)
    rc = m.open("a")
    for n in (3, 9, 1, 1, 30, 2, 1):
        m.reserve(rc, n)
        m.commit(rc, n)
        m.check_invariants()
        first = max(0, rc.length - 10 + 1) // 4
        for g, kept in ((0, 2), (1, 0)):
            held = [i for i, p in enumerate(rc.tables[g]) if p >= 0]
            assert held == sorted(set(range(min(kept, len(rc.tables[g])))) | set(range(first, len(rc.tables[g]))))
        assert all(p >= 0 for p in rc.tables[2])
    assert m.max_pages_held(1000, 16)[0] == m.max_pages_held(1000, 16)[1] + 2
    m.close(rc)
    assert all(a.num_free == a.num_pages for a in m.allocators)


def test_planner_items_cover_the_window_and_the_kept_keys():
    """Every query sees each key of its window and each kept key exactly once over its items, alone or in a batch,
    whole or split; split rows have one partial slot per item and a merge that names them."""
    from from_scratch_inference_engine_amd import ops
    from from_scratch_inference_engine_amd.ops.functions import ATTN_KEEP_WALK
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    try:
        ops.load()
    except ops.KernelLibraryMissing as e:  # pragma: no cover
        pytest.skip(f"no kernel library: {e}")
    rng = random.Random(3)
    for trial in range(60):
        window, keep = rng.choice([5, 17, 48, 96, 300]), rng.choice([1, 4, 9, 40])
        seqs = [(rng.choice([0, 1, keep, window - 1, window + keep, 333, 2500]), rng.choice([1, 1, 2, 5, 40, 150]))
                for _ in range(rng.randint(1, 5))]
        host = type("Host", (), {})()
        host.n_seqs, host.past_lens, host.q_lens = len(seqs), [p for p, _ in seqs], [n for _, n in seqs]
        host.q_starts = [0]
        for n in host.q_lens:
            host.q_starts.append(host.q_starts[-1] + n)
        host.n_tokens, host.page_size, host.compute_dtype, host.pad = host.q_starts[-1], 16, torch.float32, None
        planner = AttentionPlanner(8, 2, 64, window, keep)
        planner.compute_units = rng.choice([1, 64, 4096])
        plan = planner.plan(host)
        seen, slots = {}, {}
        for it in plan["items"]:
            s, row0, nq, pos0, kb, ke, partial, last = (int(x) for x in it)
            kept, walk = last & ~ATTN_KEEP_WALK, bool(last & ATTN_KEEP_WALK)
            assert kept in (0, keep)
            ranges = [(kb, ke)] + ([(0, min(kept, kb))] if walk else [])
            for t in range(nq):
                pos = pos0 + t
                keys = [k for lo, hi in ranges for k in range(lo, hi) if k <= pos and (pos - k < window or k < kept)]
                seen.setdefault(row0 + t, []).extend(keys)
                if partial >= 0:
                    slots.setdefault(row0 + t, []).append(partial + t)
        merges = {int(m[0]): m for m in plan["merges"]}
        used = set()
        for s, (p, n) in enumerate(seqs):
            for t in range(n):
                row, pos = host.q_starts[s] + t, p + t
                want = [k for k in range(pos + 1) if pos - k < window or k < keep]
                assert sorted(seen[row]) == want, (trial, seqs, row)
                if row in slots:
                    first, count, stride = (int(x) for x in merges[row][1:])
                    assert slots[row] == [first + i * stride for i in range(count)]
                    assert not used & set(slots[row])
                    used |= set(slots[row])
                else:
                    assert row not in merges
