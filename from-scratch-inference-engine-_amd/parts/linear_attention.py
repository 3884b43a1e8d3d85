"""Gated linear attention: a recurrent mixer whose cache is a state of fixed size per request."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..cache.manager import StateNeed
from .base import Mixer, ParamDecl, register_part
from .linear import Linear


@register_part("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Per head a state S [key_dim, value_dim] in float32 that every token updates and reads:

        S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t,

    q = (W_q x) key_dim^(-1/2), k = W_k x, v = W_v x, and a decay per key channel
    alpha = sigmoid(W_a2 (W_a1 x) + b)^(1/tau) through a low rank.  Every head's o is RMS-normed over its
    value columns (one weight, shared by the heads), multiplied by act(W_g x) and projected by W_o.

    The projections that read x are one matrix (q, k, v, g rows one after the other).  The state lives in the
    cache manager's per-request slots: zero when a request starts, carried from step to step; a portion of a
    prompt and a single decoded token go through the same kernel, which walks a request's tokens in order.
    The decays, the state and the sums are float32 whatever the activations' type."""

    graph_safe = True  # the step's requests and slots are read from the device tables

    def __init__(self, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, decay_rank: int, tau: float,
                 norm_eps: float, gate_activation: str = "silu"):
        if key_dim > 256:
            raise ValueError(f"gated linear attention: {key_dim} key channels a head are more than the kernel takes (256)")
        if not tau > 0:
            raise ValueError(f"gated linear attention: tau {tau} must be positive")
        ops.gate_act_code(gate_activation)
        self.hidden_size, self.n_heads, self.key_dim, self.value_dim = hidden_size, n_heads, key_dim, value_dim
        self.decay_rank, self.tau, self.norm_eps, self.gate_activation = decay_rank, float(tau), float(norm_eps), gate_activation
        self.k_width, self.v_width = n_heads * key_dim, n_heads * value_dim
        self.qkvg = Linear(hidden_size, 2 * self.k_width + 2 * self.v_width)
        self.a1 = Linear(hidden_size, decay_rank)
        self.a2 = Linear(decay_rank, self.k_width, bias=True)
        self.o = Linear(self.v_width, hidden_size)
        self.norm_weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"qkvg_weight": ParamDecl((2 * self.k_width + 2 * self.v_width, self.hidden_size)),
                "a1_weight": ParamDecl((self.decay_rank, self.hidden_size)),
                "a2_weight": ParamDecl((self.k_width, self.decay_rank)),
                "a2_bias": ParamDecl((self.k_width,), "vector", "bias"),
                "norm_weight": ParamDecl((self.value_dim,), "vector", "norm"),
                "o_weight": ParamDecl((self.hidden_size, self.v_width))}

    qkvg_weight = property(lambda s: s.qkvg.weight, lambda s, t: setattr(s.qkvg, "weight", t))
    a1_weight = property(lambda s: s.a1.weight, lambda s, t: setattr(s.a1, "weight", t))
    a2_weight = property(lambda s: s.a2.weight, lambda s, t: setattr(s.a2, "weight", t))
    a2_bias = property(lambda s: s.a2.bias, lambda s, t: setattr(s.a2, "bias", t))
    o_weight = property(lambda s: s.o.weight, lambda s, t: setattr(s.o, "weight", t))

    def prepare(self, device, compute_dtype) -> None:
        copies = bool(self.options.get("weight_copies", True))
        self.qkvg.prepare(copies)
        self.o.prepare(copies)

    def release_optional_memory(self) -> int:
        return self.qkvg.drop_copy() + self.o.drop_copy()

    def cache_need(self) -> StateNeed:
        return StateNeed((self.n_heads, self.key_dim, self.value_dim), "float32")

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        p = self.qkvg(x)
        z = self.a2(self.a1(x), out_dtype=torch.float32)  # the decays before the sigmoid, bias added, float32 from here on
        o = ops.gla_scan(p, 0, self.k_width, 2 * self.k_width, z, cache.state, ctx.q_starts, ctx.seq_slots, self.n_heads,
                         self.key_dim, self.value_dim, self.key_dim ** -0.5, 1.0 / self.tau)
        y = ops.gated_headnorm(o, p[:, 2 * self.k_width + self.v_width:], self.norm_weight, self.norm_eps, self.n_heads,
                               self.gate_activation)
        return self.o.for_residual(y, ctx)
