"""RMSNorm and layer norm, fused with the residual sum."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import HiddenState, Norm, ParamDecl, register_part


def _no_second_delta(hidden: HiddenState, name: str) -> None:
    if hidden.delta_scale != 1.0:
        raise RuntimeError(f"{name}: the stream's pending delta carries a factor of {hidden.delta_scale}, which this norm "
                           f"does not apply")
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
        if hidden.delta_scale != 1.0:
            raise RuntimeError("layer_norm: a factor on the pending deltas is not applied")
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


@register_part("norm", "group_rms_norm")
class GroupRMSNorm(Norm):
    """RMS norm in groups: the row is cut into ``groups`` equal consecutive parts, each divided by its own
    sqrt(mean(part^2) + eps), and the whole multiplied by w; everything in float32.  The row is
    x = residual + delta_scale * (delta + delta2): up to two pending deltas (each in the compute type or float32)
    and the stream's factor on them, added in the pass that normalises.  ``pair`` gives this norm's and another
    one's output of the same stream from one pass (they differ in the weight only).  ``groups=1`` is the plain RMS
    norm with those additions."""

    adds_partial_sums = False  # (a delta cut into partial sums is not taken: the model then never makes one)
    adds_two_deltas = True
    scales_deltas = True
    graph_safe = True

    def __init__(self, hidden_size: int, eps: float, groups: int = 1):
        if groups < 1 or hidden_size % groups:
            raise ValueError(f"group_rms_norm: {hidden_size} values do not make {groups} equal groups")
        self.hidden_size, self.eps, self.groups = hidden_size, float(eps), int(groups)
        self.weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.hidden_size,), "vector", "norm")}

    @staticmethod
    def _take(hidden: HiddenState, clear: bool):
        if hidden.delta_norm is not None:
            raise RuntimeError("group_rms_norm: a pending delta with a norm of its own is not taken")
        taken = hidden.delta, hidden.delta2, hidden.delta_scale
        for d in taken[:2]:
            if d is not None and d.ndim != 2:
                raise RuntimeError("group_rms_norm: a pending delta of partial sums is not taken")
        if clear:
            hidden.delta = hidden.delta2 = None
            hidden.delta_scale = 1.0
        return taken

    def __call__(self, hidden: HiddenState, out_dtype: torch.dtype) -> torch.Tensor:
        d1, d2, scale = self._take(hidden, True)
        return ops.group_rmsnorm(hidden.residual, self.weight, self.eps, self.groups, out_dtype, delta=d1, delta2=d2,
                                 delta_scale=scale, write_back=d1 is not None or d2 is not None)

    def pair(self, hidden: HiddenState, other: "GroupRMSNorm", out_dtype: torch.dtype):
        if (not isinstance(other, GroupRMSNorm) or other.eps != self.eps or other.hidden_size != self.hidden_size
                or other.groups != self.groups):
            raise ValueError("group_rms_norm: a pair is two such norms of one width, eps and number of groups")
        d1, d2, scale = self._take(hidden, True)
        return ops.group_rmsnorm(hidden.residual, self.weight, self.eps, self.groups, out_dtype, delta=d1, delta2=d2,
                                 delta_scale=scale, weight2=other.weight, write_back=d1 is not None or d2 is not None)

    def rows(self, hidden: HiddenState, rows: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        d1, d2, scale = self._take(hidden, False)
        return ops.group_rmsnorm(hidden.residual, self.weight, self.eps, self.groups, out_dtype, delta=d1, delta2=d2,
                                 delta_scale=scale, rows=rows)


@register_part("norm", "stream")
class StreamReader(Norm):
    """No norm at all: the stream itself, x = residual + pending delta, in the type asked for.  It stands where a
    layer's sublayers read the stream as it is and only their outputs are normed: the pending delta then comes with
    a norm of its own (``HiddenState.delta_norm``, an ``RMSNorm``), and that norm, the float32 sum and the rounding of
    the result are one kernel."""

    adds_partial_sums = True
    graph_safe = True

    def __init__(self, hidden_size: int):
        self.hidden_size = hidden_size

    @staticmethod
    def _pending(hidden: HiddenState):
        _no_second_delta(hidden, "stream")
        delta, post = hidden.delta, hidden.delta_norm
        if delta is not None and post is None:
            raise RuntimeError("stream: a pending delta without a norm of its own is not taken (a pre-norm block came before)")
        return delta, post

    def __call__(self, hidden: HiddenState, out_dtype: torch.dtype) -> torch.Tensor:
        delta, post = self._pending(hidden)
        hidden.delta = hidden.delta_norm = None
        if delta is None:
            return hidden.residual if out_dtype == torch.float32 else ops.round_to(hidden.residual, out_dtype)
        return ops.sandwich_norm(hidden.residual, delta, post.weight, post.eps, None, 0.0, out_dtype, write_back=True)

    def rows(self, hidden: HiddenState, rows: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        delta, post = self._pending(hidden)
        if delta is None:
            raise RuntimeError("stream: chosen rows of a stream without a pending delta are not offered")
        return ops.sandwich_norm(hidden.residual, delta, post.weight, post.eps, None, 0.0, out_dtype, rows=rows)
