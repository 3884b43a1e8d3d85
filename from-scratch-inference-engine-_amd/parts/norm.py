"""RMSNorm and layer norm, fused with the residual sum."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import HiddenState, Norm, ParamDecl, register_part


def _no_second_delta(hidden: HiddenState, name: str) -> None:
    if hidden.delta2 is not None:
        raise RuntimeError(f"{name}: the stream has a second pending delta (a block whose sublayers read the same "
                           f"stream came before), which this norm does not add")


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """y = (x * rsqrt(mean(x^2) + eps)) * w with x = residual + pending delta, all in float32;
    eps inside the square root, the weight multiplied last, plain w (the reference's rms_norm,
    src/model/nn.cpp:45-72, which sums in float64).  ``unit_offset=True``: the checkpoint tensor is the
    factor less one, so the factor is 1 + w (the one is added in float32 when the weights are loaded).
    Where the pending delta has a norm of its own to go through first (``HiddenState.delta_norm``, another
    ``RMSNorm``), that norm, the sum and this norm are one kernel."""

    adds_partial_sums = True

    graph_safe = True

    def __init__(self, hidden_size: int, eps: float, unit_offset: bool = False):
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.unit_offset = bool(unit_offset)
        self.weight = None
        self._offset_added = False

    def param_decls(self) -> Dict[str, ParamDecl]:
        # (an offset from one is drawn like a bias by the random-weights mode: small, centred on zero)
        return {"weight": ParamDecl((self.hidden_size,), "vector", "bias" if self.unit_offset else "norm")}

    def prepare(self, device, compute_dtype) -> None:
        if self.unit_offset and not self._offset_added and self.weight is not None:
            self.weight = self.weight + 1.0
            self._offset_added = True

    def __call__(self, hidden: HiddenState, out_dtype: torch.dtype) -> torch.Tensor:
        _no_second_delta(hidden, "rms_norm")
        delta, post = hidden.delta, hidden.delta_norm
        hidden.delta = hidden.delta_norm = None
        if delta is not None and post is not None:
            return ops.sandwich_norm(hidden.residual, delta, post.weight, post.eps, self.weight, self.eps, out_dtype,
                                     write_back=True)
        return ops.rmsnorm(hidden.residual, self.weight, self.eps, out_dtype, delta=delta,
                           write_back=delta is not None)

    def rows(self, hidden: HiddenState, rows: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        _no_second_delta(hidden, "rms_norm")
        if hidden.delta is not None and hidden.delta_norm is not None:
            post = hidden.delta_norm
            return ops.sandwich_norm(hidden.residual, hidden.delta, post.weight, post.eps, self.weight, self.eps,
                                     out_dtype, rows=rows)
        return ops.rmsnorm(hidden.residual, self.weight, self.eps, out_dtype, delta=hidden.delta, rows=rows)

    def plain(self, x: torch.Tensor, out=None) -> torch.Tensor:
        return ops.rmsnorm_plain(x, self.weight, self.eps, out=out)


@register_part("norm", "layer_norm")
class LayerNorm(Norm):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * w + b with x = residual + pending deltas, the variance the mean of
    the squared deviations, everything in float32.  It adds up to two pending deltas (each whole or as float32
    partial sums), and ``pair`` gives this norm's and another layer norm's output of the same stream from one
    pass: they share mean and variance and differ in weight and bias only."""

    adds_partial_sums = True
    adds_two_deltas = True
    graph_safe = True

    def __init__(self, hidden_size: int, eps: float):
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.weight = None
        self.bias = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.hidden_size,), "vector", "norm"),
                "bias": ParamDecl((self.hidden_size,), "vector", "bias")}

    @staticmethod
    def _take(hidden: HiddenState, clear: bool):
        if hidden.delta_norm is not None:
            raise RuntimeError("layer_norm: a pending delta with a norm of its own is not taken")
        deltas = hidden.delta, hidden.delta2
        if clear:
            hidden.delta = hidden.delta2 = None
        return deltas

    def __call__(self, hidden: HiddenState, out_dtype: torch.dtype) -> torch.Tensor:
        d1, d2 = self._take(hidden, True)
        return ops.layer_norm(hidden.residual, self.weight, self.bias, self.eps, out_dtype, delta=d1, delta2=d2,
                              write_back=d1 is not None or d2 is not None)

    def pair(self, hidden: HiddenState, other: "LayerNorm", out_dtype: torch.dtype):
        if not isinstance(other, LayerNorm) or other.eps != self.eps or other.hidden_size != self.hidden_size:
            raise ValueError("layer_norm: a pair is two layer norms of one width and eps")
        d1, d2 = self._take(hidden, True)
        return ops.layer_norm(hidden.residual, self.weight, self.bias, self.eps, out_dtype, delta=d1, delta2=d2,
                              weight2=other.weight, bias2=other.bias, write_back=d1 is not None or d2 is not None)

    def rows(self, hidden: HiddenState, rows: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        d1, d2 = self._take(hidden, False)
        return ops.layer_norm(hidden.residual, self.weight, self.bias, self.eps, out_dtype, delta=d1, delta2=d2, rows=rows)
