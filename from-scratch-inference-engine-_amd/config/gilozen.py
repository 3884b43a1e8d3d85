"""Configuration of the Gilozen decoder (config.json ``"architecture": "Gilozen"``): a list of layers, each
with a mixer of one of two kinds (attention through a latent, gated linear attention) and an optional gated
feed-forward, a norm before and after every sublayer, and soft-capped logits."""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, checked_float, checked_int, end_token_of, required_int

LATENT, GLA = "latent_attention", "gla"


@dataclass(frozen=True)
class LatentAttentionConfig:
    """``dim`` unrotated and ``rot_dim`` rotated query/key values a head, values of ``vdim``, a key/value
    latent of ``kv_rank`` and a query latent of ``q_rank``; the first ``rot_dims`` of the rotated values turn
    (neighbouring pairs, base ``rot_base``); ``kv_from``: the layer whose cached latent this one reads."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    kv_from: Optional[int] = None

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "q_rank": self.q_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class GLAConfig:
    """``heads`` heads of ``dim`` key channels and ``vdim`` value columns; decays sigmoid(z)^(1/tau), made through
    a bottleneck of ``decay_rank`` values.  config.json need not state that rank (key ``a_rank``): the shape of
    the layer's ``mix.a1`` tensor gives it (``GilozenConfig.completed_from``)."""

    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int] = None

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.decay_rank is not None:
            d["a_rank"] = self.decay_rank
        return d


@dataclass(frozen=True)
class LayerConfig:
    kind: str          # LATENT or GLA
    mixer: object      # LatentAttentionConfig or GLAConfig
    ff: Optional[int]  # width of the gated feed-forward, None: the layer has none

    def to_dict(self) -> dict:
        return {"type": self.kind, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


def _mixer_int(m: Mapping, key: str, where: str, minimum: int = 1) -> int:
    if key not in m:
        raise ConfigError(f"config.json: {where} has no '{key}'")
    return checked_int(m[key], f"{where}.{key}", minimum)


@dataclass(frozen=True)
class GilozenConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 1e-5
    logit_softcap: Optional[float] = None
    layers: Tuple[LayerConfig, ...] = ()
    eos_token_id: int = -1

    @property
    def end_token(self) -> int:
        return self.eos_token_id

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "GilozenConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(layers_raw):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} must be an object with a 'mixer'")
            kind, m = entry.get("type"), entry["mixer"]
            if kind == LATENT:
                rot = m.get("rot")
                if not isinstance(rot, dict):
                    raise ConfigError(f"config.json: {where}.mixer has no 'rot'")
                rot_dim = _mixer_int(m, "rot_dim", where, 0)
                rot_dims = _mixer_int(rot, "dims", where + ".rot", 0)
                if rot_dims % 2 or rot_dims > rot_dim:
                    raise ConfigError(f"config.json: {where}: rot.dims {rot_dims} must be even and at most rot_dim {rot_dim}")
                kv_from = m.get("kv_from")
                if kv_from is not None:
                    kv_from = checked_int(kv_from, f"{where}.kv_from", 0)
                mixer = LatentAttentionConfig(
                    heads=_mixer_int(m, "heads", where), dim=_mixer_int(m, "dim", where), rot_dim=rot_dim,
                    vdim=_mixer_int(m, "vdim", where), kv_rank=_mixer_int(m, "kv_rank", where),
                    q_rank=_mixer_int(m, "q_rank", where), scale=checked_float(m.get("scale"), f"{where}.scale"),
                    rot_base=checked_float(rot.get("base"), f"{where}.rot.base"), rot_dims=rot_dims, kv_from=kv_from)
                if kv_from is not None:
                    src = layers[kv_from].mixer if kv_from < i and layers[kv_from].kind == LATENT else None
                    if src is None or src.kv_from is not None:
                        raise ConfigError(f"config.json: {where}.kv_from = {kv_from} must name an earlier latent-attention "
                                          f"layer that makes its own latent")
                    if (src.kv_rank, src.rot_dim, src.rot_base, src.rot_dims) != (mixer.kv_rank, mixer.rot_dim,
                                                                                 mixer.rot_base, mixer.rot_dims):
                        raise ConfigError(f"config.json: {where} and layer {kv_from} must agree in kv_rank, rot_dim and rot")
            elif kind == GLA:
                mixer = GLAConfig(heads=_mixer_int(m, "heads", where), dim=_mixer_int(m, "dim", where),
                                  vdim=_mixer_int(m, "vdim", where), tau=checked_float(m.get("tau"), f"{where}.tau"),
                                  decay_rank=_mixer_int(m, "a_rank", where) if m.get("a_rank") is not None else None)
            else:
                raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this architecture "
                                  f"({LATENT}, {GLA})")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp must be null or a dense feed-forward")
                ff = _mixer_int(mlp, "ff", where + ".mlp")
            layers.append(LayerConfig(kind, mixer, ff))
        norm = raw.get("norm") or {}
        cap = raw.get("logit_softcap")
        return cls(architecture="Gilozen", width=required_int(raw, "width"), vocab=required_int(raw, "vocab"),
                   norm_eps=checked_float(norm.get("eps", 1e-5), "norm.eps", positive=False),
                   logit_softcap=None if cap is None else checked_float(cap, "logit_softcap"),
                   layers=tuple(layers), eos_token_id=end_token_of(raw))

    def completed_from(self, tensor_shapes: Mapping[str, tuple]) -> "GilozenConfig":
        layers = []
        for i, layer in enumerate(self.layers):
            name = f"l{i}.mix.a1"
            if layer.kind == GLA and layer.mixer.decay_rank is None and name in tensor_shapes:
                shape = tuple(tensor_shapes[name])
                if len(shape) != 2 or shape[0] < 1:
                    raise ConfigError(f"tensor {name}: shape {shape} does not give the rank of the decays' bottleneck")
                layer = replace(layer, mixer=replace(layer.mixer, decay_rank=int(shape[0])))
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab, "norm": {"eps": self.norm_eps},
             "layers": [layer.to_dict() for layer in self.layers]}
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_id >= 0:
            d["eos_token_id"] = self.eos_token_id
        return d
