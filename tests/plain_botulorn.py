"""A plain, slow Botulorn: whole sequences, float64, no cache, one function per mechanism.

It shares nothing with the engine: it reads config.json and model.safetensors itself (numpy) and
computes every token of a sequence from scratch.  The tests compare the engine with it.
"""

from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np


# ----------------------------------------------------------------------------------- files
def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def read_weights(folder) -> dict:
    """name -> float64 array (int64 for integer tables) from model.safetensors."""
    data = (Path(folder) / "model.safetensors").read_bytes()
    (n,) = struct.unpack("<Q", data[:8])
    header = json.loads(data[8:8 + n])
    body = data[8 + n:]
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        raw, shape = body[lo:hi], meta["shape"]
        if meta["dtype"] == "BF16":
            bits = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            arr = bits.view(np.float32).astype(np.float64)
        elif meta["dtype"] == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif meta["dtype"] == "I32":
            arr = np.frombuffer(raw, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {meta['dtype']}")
        out[name] = arr.reshape(shape)
    return out


# ------------------------------------------------------------------------------ mechanisms
def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def embed(tokens, table, scale, bigram, buckets, mul_prev, mul_cur):
    """Token rows times ``scale`` plus a hashed row for every (previous, current) pair; the first token of a
    sequence takes the table's last row."""
    x = table[tokens] * scale
    rows = [buckets] + [(tokens[t - 1] * mul_prev + tokens[t] * mul_cur) % buckets for t in range(1, len(tokens))]
    return x + bigram[rows]


def yarn_frequencies(rot):
    """(frequency per pair, factor on cos and sin) of a rotation with or without YaRN scaling."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = sc["factor"], sc["original"]

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(half) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, rot):
    """x [T, heads, d]: the first rot.dims values of every head turn, pair (i, i + dims/2)."""
    dims = rot["dims"]
    if not dims:
        return x
    half = dims // 2
    f, m = yarn_frequencies(rot)
    a = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    c, s = (np.cos(a) * m)[:, None, :], (np.sin(a) * m)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return np.concatenate([u * c - v * s, v * c + u * s, x[..., dims:]], axis=-1)


def visible(n, size, keep_first=0):
    """[query, key] mask: key <= query and (query - key < size or key < keep_first)."""
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def softmax_attention(q, k, v, scale, mask):
    """q [T, H, d], k [T, H, d], v [T, H, e] -> [T, H, e]"""
    s = np.einsum("ihd,jhd->hij", q, k) * scale
    s = np.where(mask[None], s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(-1, keepdims=True)
    return np.einsum("hij,jhe->ihe", p, v)


def attention_mixer(h, w, p, m, eps, v_first):
    """The grouped-query mixer.  ``v_first``: None in the first value-mixing layer (and in layers without
    mixing), else that layer's values.  Returns (output, this layer's values before mixing)."""
    t = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(t, H, d)
    k = (h @ w[p + "k"].T).reshape(t, G, d)
    v = (h @ w[p + "v"].T).reshape(t, G, e)
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)
    pos = np.arange(t)
    q, k = rotate_half(q, pos, m["rot"]), rotate_half(k, pos, m["rot"])
    raw_v = v
    if m.get("v_mix") and v_first is not None:
        lam = float(w[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    rep = H // G
    mask = visible(t, m["mask"]["size"], m["mask"].get("keep_first", 0))
    o = softmax_attention(q, np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1), m["scale"], mask)
    o = o * sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(t, H * e) @ w[p + "o"].T, raw_v


def latent_mixer(h, w, p, m, eps):
    t = h.shape[0]
    H, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(t, H, d + r)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    pos = np.arange(t)
    rot = dict(m["rot"], dims=r)
    k_rot = rotate_half(down[:, None, rank:], pos, rot)              # [T, 1, r]
    q_rot = rotate_half(q[..., d:], pos, rot)
    k_plain = (c @ w[p + "uk"].T).reshape(t, H, d)
    v = (c @ w[p + "uv"].T).reshape(t, H, e)
    qq = np.concatenate([q[..., :d], q_rot], axis=-1)
    kk = np.concatenate([k_plain, np.repeat(k_rot, H, axis=1)], axis=-1)
    o = softmax_attention(qq, kk, v, m["scale"], visible(t, m["mask"]["size"]))
    return o.reshape(t, H * e) @ w[p + "o"].T


def feed_forward(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


# ------------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    bg = cfg["embedding"]["bigram"]
    x = embed(list(tokens), w["embed"], cfg["embedding"]["scale"], w["bigram"], bg["buckets"], bg["mul_prev"], bg["mul_cur"])
    v_first, after = None, []
    for i, layer in enumerate(cfg["layers"]):
        a = layer_norm(x, w[f"l{i}.norm1"], w[f"l{i}.norm1.b"], eps)
        if layer["type"] == "attention":
            y, raw_v = attention_mixer(a, w, f"l{i}.mix.", layer["mixer"], eps, v_first)
            if layer["mixer"].get("v_mix") and v_first is None:
                v_first = raw_v
        elif layer["type"] == "latent_attention":
            y = latent_mixer(a, w, f"l{i}.mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + feed_forward(layer_norm(x, w[f"l{i}.norm2"], w[f"l{i}.norm2.b"], eps), w, f"l{i}.mlp.")
        x = x + y
        after.append(x)
    logits = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
    return (logits, np.stack(after)) if return_layers else logits
