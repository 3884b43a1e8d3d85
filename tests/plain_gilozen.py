"""Plain, slow implementation of the Gilozen decoder: whole sequences, no cache, one function
for each mechanism, float64 on the CPU.

It shares no code with the engine: config.json is read with ``json``, the weights with the
``safetensors`` package.  Notation: ``x`` [T, W] is the residual stream of one sequence whose
positions are 0..T-1, ``h`` a sublayer's input, weights are stored [out, in].
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64


def read_config(model_dir) -> dict:
    return json.loads((Path(model_dir) / "config.json").read_text())


def read_weights(model_dir) -> dict:
    from safetensors import safe_open

    out = {}
    with safe_open(str(Path(model_dir) / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            out[name] = t if t.dtype in (torch.int32, torch.int64) else t.to(F)
    return out


# ------------------------------------------------------------------------------------------
# small pieces
# ------------------------------------------------------------------------------------------
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_plain_weight(x, w, eps):
    return unit_rms(x, eps) * w


def norm_zero_centred(x, w, eps):
    """The layer norms store their factor less one: the factor is 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gated_feed_forward(h, gate, up, down):
    return (gelu_tanh(h @ gate.t()) * (h @ up.t())) @ down.t()


def rotate_interleaved(x, positions, base: float, dims: int):
    """x [T, heads, n]: the first ``dims`` values of every head are pairs (2i, 2i+1), pair i turned by
    the angle position * base^(-2i/dims); the rest passes."""
    i = torch.arange(dims // 2, dtype=F)
    ang = torch.as_tensor(positions, dtype=F).reshape(-1, 1, 1) * torch.pow(torch.tensor(base, dtype=F), -2.0 * i / dims)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def softmax_with_sink(scores, sink):
    """scores [T, S] of one head (masked entries -inf), sink a number: weights exp(s_j) / (sum_k exp(s_k)
    + exp(sink)).  The sink has no value: the weights of a row sum to less than one."""
    m = torch.maximum(scores.max(dim=-1, keepdim=True).values, sink.reshape(1, 1))
    e = torch.exp(scores - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - m))


# ------------------------------------------------------------------------------------------
# mixers
# ------------------------------------------------------------------------------------------
def latent_of(h, w, p: str, m: dict, eps: float):
    """What a latent-attention layer keeps per token: the normed latent [T, kv_rank] and the rotated
    shared key part [T, rot_dim]."""
    r, rd = m["kv_rank"], m["rot_dim"]
    d = h @ w[p + "dkv"].t()
    c = norm_plain_weight(d[:, :r], w[p + "dkv.norm"], eps)
    t = h.shape[0]
    kr = rotate_interleaved(d[:, r:].reshape(t, 1, rd), range(t), m["rot"]["base"], m["rot"]["dims"]).reshape(t, rd)
    return c, kr


def latent_attention(h, w, p: str, m: dict, eps: float, kept):
    """``kept`` = (latent, rotated key part) of this layer or of the layer it borrows them from."""
    t = h.shape[0]
    nh, dim, rd, vd, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = kept
    cq = norm_plain_weight(h @ w[p + "dq"].t(), w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].t()).reshape(t, nh, dim + rd)
    q_plain = q[..., :dim]
    q_rot = rotate_interleaved(q[..., dim:], range(t), m["rot"]["base"], m["rot"]["dims"])
    k_plain = (c @ w[p + "uk"].t()).reshape(t, nh, dim)
    v = (c @ w[p + "uv"].t()).reshape(t, nh, vd)
    gate = torch.sigmoid(h @ w[p + "g"].t())
    causal = torch.ones(t, t, dtype=torch.bool).tril()
    heads = []
    for a in range(nh):
        s = (q_plain[:, a] @ k_plain[:, a].t() + q_rot[:, a] @ kr.t()) * m["scale"]
        s = s.masked_fill(~causal, float("-inf"))
        heads.append(softmax_with_sink(s, w[p + "sink"][a]) @ v[:, a] * gate[:, a:a + 1])
    return torch.cat(heads, dim=-1) @ w[p + "o"].t()


def gla(h, w, p: str, m: dict, eps: float):
    """Gated linear attention, token by token: S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t."""
    t = h.shape[0]
    nh, dim, vd = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].t()).reshape(t, nh, dim) * dim ** -0.5
    k = (h @ w[p + "k"].t()).reshape(t, nh, dim)
    v = (h @ w[p + "v"].t()).reshape(t, nh, vd)
    z = (h @ w[p + "a1"].t()) @ w[p + "a2"].t() + w[p + "a2.b"]
    alpha = torch.pow(torch.sigmoid(z), 1.0 / m["tau"]).reshape(t, nh, dim)
    state = torch.zeros(nh, dim, vd, dtype=F)
    out = torch.zeros(t, nh, vd, dtype=F)
    for i in range(t):
        state = alpha[i].unsqueeze(-1) * state + k[i].unsqueeze(-1) * v[i].unsqueeze(-2)
        out[i] = torch.einsum("hdv,hd->hv", state, q[i])
    out = norm_plain_weight(out, w[p + "norm"], eps).reshape(t, nh * vd)
    g = h @ w[p + "g"].t()
    return (out * (g * torch.sigmoid(g))) @ w[p + "o"].t()


# ------------------------------------------------------------------------------------------
# the model
# ------------------------------------------------------------------------------------------
def forward(cfg: dict, w: dict, ids, layers_out=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids, dtype=torch.int64)]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = norm_zero_centred(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            if "kv_from" in m and m["kv_from"] is not None:
                mine = kept[m["kv_from"]]
            else:
                mine = kept[i] = latent_of(h, w, p + "mix.", m, eps)
            y = latent_attention(h, w, p + "mix.", m, eps, mine)
        elif layer["type"] == "gla":
            y = gla(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_zero_centred(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = norm_zero_centred(x, w[p + "norm2"], eps)
            y = gated_feed_forward(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
            x = x + norm_zero_centred(y, w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = norm_zero_centred(x, w["final.norm"], eps) @ w["head"].t()
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
