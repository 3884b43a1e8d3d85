"""Botulorn: a decoder whose layers run their mixer and their gated feed-forward side by side on the same
layer-normed stream; which parts, in which order, from which checkpoint tensors."""

from __future__ import annotations

from typing import List

from ..config.botulorn import ATTENTION, LATENT, BotulornConfig
from ..parts.base import make_part
from ..parts.embedding import LMHead, PairHashEmbedding
from ..weights.loader import ParamBinding, TensorSpec
from .registry import register_architecture
from .spec import LayerCall, ModelSpec, bind


def build_botulorn(cfg: BotulornConfig) -> ModelSpec:
    """Layer i: x += mixer(norm1(x)) + ff(norm2(x)), both layer norms (weight and bias) of the same x; a layer
    without feed-forward has no second norm.  The embedding is the token's row times a constant plus the hashed
    row of (previous token, token).  After the last layer the model's layer norm and the head.  Tensor names:
    ``embed``, ``bigram``, ``l<i>.norm1`` (+ ``.b``) ..., ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm`` (+ ``.b``),
    ``head``.  Of the attention layers that mix values, the first publishes its values and the later ones blend
    theirs with them."""
    w, eps = cfg.width, cfg.norm_eps
    bindings: List[ParamBinding] = []

    def norm(name: str):
        part = make_part("norm", "layer_norm", hidden_size=w, eps=eps)
        bind(bindings, part, "weight", [TensorSpec(name, (w,), "norm")])
        bind(bindings, part, "bias", [TensorSpec(name + ".b", (w,), "bias")])
        return part

    def head_norm(name: str, dim: int):
        part = make_part("norm", "rms_norm", hidden_size=dim, eps=eps)
        bind(bindings, part, "weight", [TensorSpec(name, (dim,), "norm")])
        return part

    def rotation(rot, head_dim: int):
        if not rot.dims:
            return make_part("position", "none")
        return make_part("position", "rope", head_dim=head_dim, theta=rot.base, rotary_dim=rot.dims, layout="half",
                         stretch=rot.stretch)

    embedding = PairHashEmbedding(cfg.vocab, w, cfg.pair_buckets, cfg.pair_mul_prev, cfg.pair_mul_cur, cfg.embedding_scale)
    bind(bindings, embedding, "weight", [TensorSpec("embed", (cfg.vocab, w))])
    bind(bindings, embedding, "pair_weight", [TensorSpec("bigram", (cfg.pair_buckets + 1, w))])

    layers, schedule = [], []
    values_published = False
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", layer.mixer
        if layer.kind == ATTENTION:
            mix = None
            if m.v_mix:
                mix = "mixed" if values_published else "source"
                values_published = True
            mixer = make_part("mixer", "gqa_attention", hidden_size=w, n_heads=m.heads, n_kv_heads=m.kv_heads,
                              head_dim=m.dim, qkv_bias=False, position=rotation(m.rot, m.dim), window=m.window,
                              q_norm=head_norm(p + "q.norm", m.dim), k_norm=head_norm(p + "k.norm", m.dim),
                              keep_first=m.keep_first, scale=m.scale, value_dim=m.vdim, gate=True, value_mix=mix)
            bind(bindings, mixer, "qkv_weight", [TensorSpec(p + "q", (m.heads * m.dim, w)),
                                                 TensorSpec(p + "k", (m.kv_heads * m.dim, w)),
                                                 TensorSpec(p + "v", (m.kv_heads * m.vdim, w)),
                                                 TensorSpec(p + "g", (m.heads, w))])
            if mix is not None:
                bind(bindings, mixer, "value_mix_weight", [TensorSpec(p + "vmix", (), "bias")])
            bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, m.heads * m.vdim))])
        elif layer.kind == LATENT:
            mixer = make_part("mixer", "latent_attention", hidden_size=w, n_heads=m.heads, head_dim=m.dim,
                              rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank, q_rank=m.q_rank, scale=m.scale,
                              norm_eps=eps, position=rotation(m.rot, m.rot_dim), own_latent=True, sink=False, gate=False,
                              window=m.window)
            bind(bindings, mixer, "down_weight", [TensorSpec(p + "dq", (m.q_rank, w)),
                                                  TensorSpec(p + "dkv", (m.kv_rank + m.rot_dim, w))])
            bind(bindings, mixer, "kv_norm_weight", [TensorSpec(p + "dkv.norm", (m.kv_rank,), "norm")])
            bind(bindings, mixer, "q_norm_weight", [TensorSpec(p + "dq.norm", (m.q_rank,), "norm")])
            bind(bindings, mixer, "uq_weight", [TensorSpec(p + "uq", (m.heads * (m.dim + m.rot_dim), m.q_rank))])
            bind(bindings, mixer, "uk_weight", [TensorSpec(p + "uk", (m.heads * m.dim, m.kv_rank))])
            bind(bindings, mixer, "uv_weight", [TensorSpec(p + "uv", (m.heads * m.vdim, m.kv_rank))])
            bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, m.heads * m.vdim))])
        else:  # pragma: no cover - the configuration has refused it
            raise ValueError(layer.kind)
        parts = dict(mixer_norm=norm(f"l{i}.norm1"), mixer=mixer)
        if layer.ff is not None:
            ffn = make_part("feed_forward", "gated", hidden_size=w, intermediate_size=layer.ff, activation="gelu_tanh")
            bind(bindings, ffn, "gate_up_weight", [TensorSpec(f"l{i}.mlp.gate", (layer.ff, w)),
                                                   TensorSpec(f"l{i}.mlp.up", (layer.ff, w))])
            bind(bindings, ffn, "down_weight", [TensorSpec(f"l{i}.mlp.down", (w, layer.ff))])
            parts.update(ffn_norm=norm(f"l{i}.norm2"), ffn=ffn)
        layers.append(make_part("block", "parallel", **parts))
        schedule.append(LayerCall(i))

    final_norm = norm("final.norm")
    lm_head = LMHead(w, cfg.vocab)
    bind(bindings, lm_head, "weight", [TensorSpec("head", (cfg.vocab, w))])
    # (the first value-mixing layer's weight is in the checkpoint and is not used: it is bound and left alone; a
    # layer that mixes nothing may carry one too, which is not read)
    unused = tuple(f"l{i}.mix.vmix" for i, layer in enumerate(cfg.layers) if layer.kind == ATTENTION and not layer.mixer.v_mix)
    return ModelSpec(config=cfg, embedding=embedding, layers=layers, schedule=schedule, final_norm=final_norm,
                     lm_head=lm_head, bindings=bindings, ignore_unexpected=unused)


register_architecture("Botulorn", BotulornConfig, build_botulorn)
