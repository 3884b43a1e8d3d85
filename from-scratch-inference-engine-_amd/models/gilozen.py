"""Gilozen: a decoder whose layers mix tokens either by attention through a latent or by gated linear
attention, each sublayer between two norms; which parts, in which order, from which checkpoint tensors."""

from __future__ import annotations

from typing import List

from ..config.base import ConfigError
from ..config.gilozen import GLA, LATENT, GilozenConfig
from ..parts.base import make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import ParamBinding, TensorSpec
from .registry import register_architecture
from .spec import LayerCall, ModelSpec, bind


def build_gilozen(cfg: GilozenConfig) -> ModelSpec:
    """Layer i: x += norm1b(mixer(norm1(x))), then, if it has a feed-forward, x += norm2b(ff(norm2(x))); every norm
    is an RMS norm whose checkpoint tensor holds the factor less one (the factor is 1 + w).  The feed-forward is gated with GELU in its
    tanh form.  After the last layer the model's norm, the head, and the logits' soft cap.  Tensor names:
    ``embed``, ``l<i>.norm1`` ..., ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.  A latent-attention
    layer with ``kv_from`` reads the cache that the named layer's call fills."""
    w, eps = cfg.width, cfg.norm_eps
    bindings: List[ParamBinding] = []

    def norm(name: str):
        part = make_part("norm", "rms_norm", hidden_size=w, eps=eps, unit_offset=True)
        bind(bindings, part, "weight", [TensorSpec(name, (w,), "bias")])
        return part

    embedding = TokenEmbedding(cfg.vocab, w)
    bind(bindings, embedding, "weight", [TensorSpec("embed", (cfg.vocab, w))])

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", layer.mixer
        if layer.kind == LATENT:
            position = make_part("position", "rope", head_dim=m.rot_dim, theta=m.rot_base, rotary_dim=m.rot_dims,
                                 layout="interleaved") if m.rot_dims else make_part("position", "none")
            own = m.kv_from is None
            mixer = make_part("mixer", "latent_attention", hidden_size=w, n_heads=m.heads, head_dim=m.dim,
                              rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank, q_rank=m.q_rank, scale=m.scale,
                              norm_eps=eps, position=position, own_latent=own, sink=True, gate=True)
            down = [TensorSpec(p + "dq", (m.q_rank, w))]
            if own:
                down.append(TensorSpec(p + "dkv", (m.kv_rank + m.rot_dim, w)))
                bind(bindings, mixer, "kv_norm_weight", [TensorSpec(p + "dkv.norm", (m.kv_rank,), "norm")])
            down.append(TensorSpec(p + "g", (m.heads, w)))
            bind(bindings, mixer, "down_weight", down)
            bind(bindings, mixer, "q_norm_weight", [TensorSpec(p + "dq.norm", (m.q_rank,), "norm")])
            bind(bindings, mixer, "uq_weight", [TensorSpec(p + "uq", (m.heads * (m.dim + m.rot_dim), m.q_rank))])
            bind(bindings, mixer, "uk_weight", [TensorSpec(p + "uk", (m.heads * m.dim, m.kv_rank))])
            bind(bindings, mixer, "uv_weight", [TensorSpec(p + "uv", (m.heads * m.vdim, m.kv_rank))])
            bind(bindings, mixer, "sink", [TensorSpec(p + "sink", (m.heads,), "bias")])
            bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, m.heads * m.vdim))])
            schedule.append(LayerCall(i, cache_of=m.kv_from))
        elif layer.kind == GLA:
            kw, vw = m.heads * m.dim, m.heads * m.vdim
            # the rank of the decays' bottleneck is not in config.json: the tensor's shape gives it
            rank = m.decay_rank
            if rank is None:
                raise ConfigError(f"layer {i}: the rank of the decays' bottleneck is neither in config.json (a_rank) nor "
                                  f"known from the checkpoint's tensor {p}a1: load the configuration from the model folder")
            mixer = make_part("mixer", "gated_linear_attention", hidden_size=w, n_heads=m.heads, key_dim=m.dim,
                              value_dim=m.vdim, decay_rank=rank, tau=m.tau, norm_eps=eps, gate_activation="silu")
            bind(bindings, mixer, "qkvg_weight", [TensorSpec(p + "q", (kw, w)), TensorSpec(p + "k", (kw, w)),
                                                  TensorSpec(p + "v", (vw, w)), TensorSpec(p + "g", (vw, w))])
            bind(bindings, mixer, "a1_weight", [TensorSpec(p + "a1", (rank, w))])
            bind(bindings, mixer, "a2_weight", [TensorSpec(p + "a2", (kw, rank))])
            bind(bindings, mixer, "a2_bias", [TensorSpec(p + "a2.b", (kw,), "bias")])
            bind(bindings, mixer, "norm_weight", [TensorSpec(p + "norm", (m.vdim,), "norm")])
            bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, vw))])
            schedule.append(LayerCall(i))
        else:  # pragma: no cover - the configuration has refused it
            raise ValueError(layer.kind)
        parts = dict(mixer_norm=norm(f"l{i}.norm1"), mixer=mixer, mixer_post_norm=norm(f"l{i}.norm1b"))
        if layer.ff is not None:
            ffn = make_part("feed_forward", "gated", hidden_size=w, intermediate_size=layer.ff, activation="gelu_tanh")
            bind(bindings, ffn, "gate_up_weight", [TensorSpec(f"l{i}.mlp.gate", (layer.ff, w)),
                                                   TensorSpec(f"l{i}.mlp.up", (layer.ff, w))])
            bind(bindings, ffn, "down_weight", [TensorSpec(f"l{i}.mlp.down", (w, layer.ff))])
            parts.update(ffn_norm=norm(f"l{i}.norm2"), ffn=ffn, ffn_post_norm=norm(f"l{i}.norm2b"))
        layers.append(make_part("block", "sandwich_norm", **parts))

    final_norm = norm("final.norm")
    lm_head = LMHead(w, cfg.vocab, softcap=cfg.logit_softcap)
    bind(bindings, lm_head, "weight", [TensorSpec("head", (cfg.vocab, w))])
    return ModelSpec(config=cfg, embedding=embedding, layers=layers, schedule=schedule, final_norm=final_norm,
                     lm_head=lm_head, bindings=bindings)


register_architecture("Gilozen", GilozenConfig, build_gilozen)
