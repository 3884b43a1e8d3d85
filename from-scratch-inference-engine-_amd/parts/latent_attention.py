"""Attention whose keys and values of all heads are made from one cached latent vector a token."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..cache.manager import PagedNeed
from .attention import AttentionPlanner, paged_attention
from .base import Mixer, ParamDecl, Part, PositionEncoding, register_part
from .linear import Linear

MAX_WIDTH = 512  # the widest cache row that an attention kernel takes (the matrix-core kernels: 256)


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    """Queries through a latent: c_q = rmsnorm(W_dq x), q = W_uq c_q, per head ``head_dim`` plain values and
    ``rot_dim`` that the position encoding turns.  Keys and values through a latent: c = rmsnorm(first
    ``kv_rank`` rows of W_dkv x); the last ``rot_dim`` rows, turned, are a key part that all heads share.
    Head h's key is [W_uk,h c | shared part], its value W_uv,h c, the score their product with the query
    times ``scale``, the softmax causal (over the latest ``window`` positions only, if given) with a sink per head
    (``sink=True``), the head's result multiplied by sigmoid(W_g x)_h (``gate=True``), and W_o over the heads.

    Only c and the shared part are cached: one row of ``width`` values a token (their sum rounded up to 16,
    zeros at the end; up to 256 values the matrix-core kernels serve bfloat16, wider rows up to 512 go to the
    float32-arithmetic kernel in both precisions) in a paged cache of a single kv head.  Attention runs over those rows as they are,
    with the engine's kernels for grouped queries (every head reads the same keys): head h's query becomes
    [W_uk,h^T q_h | turned part], the values are the rows themselves, and W_uv,h is applied to the result.
    ``own_latent=False``: the layer has no W_dkv and reads the cache of the layer that the model's schedule
    names (its own W_uk, W_uv, queries and everything else).

    The projections that read x are one matrix (dq rows, dkv rows, gate rows)."""

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.sub_parts().values())

    def __init__(self, hidden_size: int, n_heads: int, head_dim: int, rot_dim: int, value_dim: int, kv_rank: int,
                 q_rank: int, scale: float, norm_eps: float, position: PositionEncoding, own_latent: bool = True,
                 sink: bool = True, gate: bool = True, window: Optional[int] = None):
        self.width = -(-(kv_rank + rot_dim) // 16) * 16
        if self.width > MAX_WIDTH:
            raise ValueError(f"latent attention: kv_rank {kv_rank} + rot_dim {rot_dim} is more than the attention "
                             f"kernels take in a cache row ({MAX_WIDTH})")
        self.rot_pairs = (getattr(position, "rotary_dim", 0) // 2) if position.rotates else 0
        layout = getattr(position, "layout", None)
        if position.rotates and (layout not in ("interleaved", "half") or 2 * self.rot_pairs > rot_dim):
            raise ValueError("latent attention: the position encoding must turn pairs (neighbours, or value i with "
                             "value i + rotary_dim / 2) within rot_dim")
        # what the kernels are told: a positive number of neighbouring pairs, a negative one of pairs (i, i + pairs)
        self.kernel_pairs = -self.rot_pairs if layout == "half" else self.rot_pairs
        if window is not None and window < 1:
            raise ValueError("latent attention: window must be >= 1")
        self.window = window
        self.hidden_size, self.n_heads, self.head_dim, self.rot_dim = hidden_size, n_heads, head_dim, rot_dim
        self.value_dim, self.kv_rank, self.q_rank = value_dim, kv_rank, q_rank
        self.scale, self.norm_eps, self.position = float(scale), float(norm_eps), position
        self.own_latent, self.has_sink, self.has_gate = bool(own_latent), bool(sink), bool(gate)
        self.q_head = head_dim + rot_dim
        self.kv_rows = kv_rank + rot_dim if own_latent else 0
        self.gate_rows = n_heads if gate else 0
        self.down = Linear(hidden_size, q_rank + self.kv_rows + self.gate_rows)
        self.uq = Linear(q_rank, n_heads * self.q_head)
        self.o = Linear(n_heads * value_dim, hidden_size)
        self.q_norm_weight = self.kv_norm_weight = self.uk_weight = self.uv_weight = self.sink = None
        self._uk_by_head = self._uv_by_head = self._ones = None
        self._planner: Optional[AttentionPlanner] = None

    def sub_parts(self) -> Dict[str, Part]:
        return {"position": self.position}

    def param_decls(self) -> Dict[str, ParamDecl]:
        decls = {"down_weight": ParamDecl((self.q_rank + self.kv_rows + self.gate_rows, self.hidden_size)),
                 "q_norm_weight": ParamDecl((self.q_rank,), "vector", "norm"),
                 "uq_weight": ParamDecl((self.n_heads * self.q_head, self.q_rank)),
                 "uk_weight": ParamDecl((self.n_heads * self.head_dim, self.kv_rank)),
                 "uv_weight": ParamDecl((self.n_heads * self.value_dim, self.kv_rank)),
                 "o_weight": ParamDecl((self.hidden_size, self.n_heads * self.value_dim))}
        if self.own_latent:
            decls["kv_norm_weight"] = ParamDecl((self.kv_rank,), "vector", "norm")
        if self.has_sink:
            decls["sink"] = ParamDecl((self.n_heads,), "vector", "bias")
        return decls

    down_weight = property(lambda s: s.down.weight, lambda s, t: setattr(s.down, "weight", t))
    uq_weight = property(lambda s: s.uq.weight, lambda s, t: setattr(s.uq, "weight", t))
    o_weight = property(lambda s: s.o.weight, lambda s, t: setattr(s.o, "weight", t))

    def prepare(self, device, compute_dtype) -> None:
        copies = bool(self.options.get("weight_copies", True))
        self.down.prepare(copies)
        self.o.prepare(copies)
        # a matrix [outputs, inputs] for every head: W_uk,h^T (the plain query values to the latent's width)
        # and W_uv,h (the latent's width to the value)
        h = self.n_heads
        self._uk_by_head = self.uk_weight.view(h, self.head_dim, self.kv_rank).transpose(1, 2).contiguous()
        self._uv_by_head = self.uv_weight.view(h, self.value_dim, self.kv_rank).contiguous()

    def release_optional_memory(self) -> int:
        return self.down.drop_copy() + self.o.drop_copy()

    def cache_need(self) -> Optional[PagedNeed]:
        return PagedNeed(1, self.width, self.window) if self.own_latent else None

    def planner(self) -> AttentionPlanner:
        if self._planner is None:
            self._planner = AttentionPlanner(self.n_heads, 1, self.width, self.window)
        return self._planner

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        if cache is None or cache.writes != self.own_latent:
            raise RuntimeError("latent attention: a layer with a latent of its own writes its cache, one without reads "
                               "another layer's: the model's schedule says otherwise")
        h, t, width = self.n_heads, x.shape[0], self.width
        plan = ctx.plan(self.planner())
        table = self.position.table(ctx) if self.rot_pairs else None
        p = self.down(x)
        pools = dict(slots=cache.slots, k_pool=cache.k_pool, v_pool=cache.v_pool) if self.own_latent else {}
        cq, gate = ops.latent_prep(p, 0, self.q_rank, self.q_rank, self.kv_rank, self.rot_dim, self.kernel_pairs,
                                   self.q_rank + self.kv_rows, self.gate_rows, self.q_norm_weight, self.kv_norm_weight,
                                   self.norm_eps, table, **pools)
        q = self.uq(cq)
        # the queries as attention over the cached rows takes them: [W_uk,h^T q_h | turned part | zeros]
        qa = torch.empty((t, h * width), dtype=x.dtype, device=x.device)
        ops.head_gemm(q, 0, self.q_head, self._uk_by_head, qa, 0, width)
        ops.rope_pairs(q, self.head_dim, self.q_head, qa, self.kv_rank, width, h, self.rot_dim, self.kernel_pairs,
                       width - self.kv_rank, table)
        mixed = paged_attention(qa, h * width, cache, plan, h, 1, width, self.window, self.scale, t, sinks=self.sink)
        y = torch.empty((t, h * self.value_dim), dtype=x.dtype, device=x.device)
        ops.head_gemm(mixed, 0, width, self._uv_by_head, y, 0, self.value_dim, gate=gate if self.has_gate else None)
        return self.o.for_residual(y, ctx)
