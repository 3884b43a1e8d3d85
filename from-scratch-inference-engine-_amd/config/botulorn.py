"""Configuration of the Botulorn decoder (config.json ``"architecture": "Botulorn"``): a token embedding with a
hashed embedding of neighbouring token pairs, a list of layers whose mixer (grouped-query attention with a window
that keeps a request's first tokens, or attention through a latent with a plain window) and gated feed-forward
read the same layer-normed stream side by side, rotations whose frequencies are stretched for long contexts."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, checked_float, checked_int, end_token_of, required_int

ATTENTION, LATENT = "attention", "latent_attention"


@dataclass(frozen=True)
class Rotation:
    """The first ``dims`` values of a head turn, value i with value i + dims / 2, at base^(-2i/dims) a position;
    ``stretch`` = (factor, original, fast, slow) rescales those frequencies (None: as they are)."""

    base: float
    dims: int
    stretch: Optional[Tuple[float, float, float, float]] = None

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.stretch is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.stretch))
        return d


@dataclass(frozen=True)
class AttentionConfig:
    """``heads`` query and ``kv_heads`` key/value heads, keys of ``dim`` and values of ``vdim``; a query sees the
    latest ``window`` positions and the first ``keep_first`` of its request; ``v_mix``: the layer takes part in the
    mixing of values with the first such layer's."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int
    rot: Rotation
    v_mix: bool = False

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "mask": {"size": self.window, "keep_first": self.keep_first}, "rot": self.rot.to_dict()}
        if self.v_mix:
            d["v_mix"] = True
        return d


@dataclass(frozen=True)
class LatentConfig:
    """``dim`` unrotated and ``rot_dim`` rotated query/key values a head, values of ``vdim``, latents of ``kv_rank``
    (keys and values) and ``q_rank`` (queries), a window of ``window`` positions."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    window: int
    rot: Rotation

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "q_rank": self.q_rank, "scale": self.scale, "mask": {"size": self.window}, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class LayerConfig:
    kind: str          # ATTENTION or LATENT
    mixer: object
    ff: Optional[int]  # width of the gated feed-forward, None: the layer has none

    def to_dict(self) -> dict:
        return {"type": self.kind, "mixer": self.mixer.to_dict(),
                "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


def _int(m: Mapping, key: str, where: str, minimum: int = 1) -> int:
    if not isinstance(m, Mapping) or key not in m:
        raise ConfigError(f"config.json: {where} has no '{key}'")
    return checked_int(m[key], f"{where}.{key}", minimum)


def _rotation(m: Mapping, where: str, dims_within: int) -> Rotation:
    rot = m.get("rot")
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where} has no 'rot'")
    dims = _int(rot, "dims", where + ".rot", 0)
    if dims % 2 or dims > dims_within:
        raise ConfigError(f"config.json: {where}.rot.dims {dims} must be even and at most {dims_within}")
    base = checked_float(rot.get("base"), f"{where}.rot.base")
    stretch = None
    sc = rot.get("scaling")
    if sc is not None:
        if not isinstance(sc, dict):
            raise ConfigError(f"config.json: {where}.rot.scaling must be an object")
        stretch = tuple(checked_float(sc.get(k), f"{where}.rot.scaling.{k}") for k in ("factor", "original", "fast", "slow"))
        if stretch[0] < 1.0 or base <= 1.0:
            raise ConfigError(f"config.json: {where}.rot.scaling needs a factor >= 1 and a base > 1")
    return Rotation(base, dims, stretch)


@dataclass(frozen=True)
class BotulornConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    pair_buckets: int = 1
    pair_mul_prev: int = 1
    pair_mul_cur: int = 1
    layers: Tuple[LayerConfig, ...] = ()
    eos_token_id: int = -1

    @property
    def end_token(self) -> int:
        return self.eos_token_id

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "BotulornConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        mixed_values = None  # (kv_heads, vdim) of the layers that mix values
        for i, entry in enumerate(layers_raw):
            where = f"layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} must be an object with a 'mixer'")
            kind, m = entry.get("type"), entry["mixer"]
            mask = m.get("mask")
            if not isinstance(mask, dict):
                raise ConfigError(f"config.json: {where}.mixer has no 'mask'")
            window = _int(mask, "size", where + ".mask")
            scale = checked_float(m.get("scale"), f"{where}.scale")
            if kind == ATTENTION:
                dim = _int(m, "dim", where)
                mixer = AttentionConfig(
                    heads=_int(m, "heads", where), kv_heads=_int(m, "kv_heads", where), dim=dim, vdim=_int(m, "vdim", where),
                    scale=scale, window=window, keep_first=checked_int(mask.get("keep_first", 0), f"{where}.mask.keep_first", 0),
                    rot=_rotation(m, where, dim), v_mix=bool(m.get("v_mix", False)))
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"config.json: {where}: heads {mixer.heads} must be a multiple of kv_heads {mixer.kv_heads}")
                if mixer.v_mix:
                    if mixed_values is not None and mixed_values != (mixer.kv_heads, mixer.vdim):
                        raise ConfigError(f"config.json: {where}: layers that mix values must agree in kv_heads and vdim")
                    mixed_values = (mixer.kv_heads, mixer.vdim)
            elif kind == LATENT:
                rot_dim = _int(m, "rot_dim", where, 0)
                rot = _rotation(m, where, max(rot_dim, 0)) if rot_dim else Rotation(10000.0, 0)
                if rot_dim % 2:
                    raise ConfigError(f"config.json: {where}: rot_dim {rot_dim} must be even")
                # (the rotated part turns as a whole: the rotation's size is the part's)
                rot = Rotation(rot.base, rot_dim, rot.stretch)
                mixer = LatentConfig(heads=_int(m, "heads", where), dim=_int(m, "dim", where), rot_dim=rot_dim,
                                     vdim=_int(m, "vdim", where), kv_rank=_int(m, "kv_rank", where),
                                     q_rank=_int(m, "q_rank", where), scale=scale, window=window, rot=rot)
            else:
                raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this architecture "
                                  f"({ATTENTION}, {LATENT})")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp must be null or a dense feed-forward")
                ff = _int(mlp, "ff", where + ".mlp")
            layers.append(LayerConfig(kind, mixer, ff))
        norm = raw.get("norm") or {}
        emb = raw.get("embedding") or {}
        pairs = emb.get("bigram")
        if not isinstance(pairs, dict):
            raise ConfigError("config.json: 'embedding.bigram' (buckets, mul_prev, mul_cur) is missing")
        return cls(architecture="Botulorn", width=required_int(raw, "width"), vocab=required_int(raw, "vocab"),
                   norm_eps=checked_float(norm.get("eps", 1e-5), "norm.eps", positive=False),
                   embedding_scale=checked_float(emb.get("scale", 1.0), "embedding.scale"),
                   pair_buckets=_int(pairs, "buckets", "embedding.bigram"),
                   pair_mul_prev=_int(pairs, "mul_prev", "embedding.bigram", 0),
                   pair_mul_cur=_int(pairs, "mul_cur", "embedding.bigram", 0),
                   layers=tuple(layers), eos_token_id=end_token_of(raw))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab, "norm": {"eps": self.norm_eps},
             "embedding": {"scale": self.embedding_scale,
                           "bigram": {"buckets": self.pair_buckets, "mul_prev": self.pair_mul_prev, "mul_cur": self.pair_mul_cur}},
             "layers": [layer.to_dict() for layer in self.layers]}
        if self.eos_token_id >= 0:
            d["eos_token_id"] = self.eos_token_id
        return d
