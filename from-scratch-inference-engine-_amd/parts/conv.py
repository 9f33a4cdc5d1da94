"""A short causal convolution over time that a layer puts in front of what a sublayer reads."""

from __future__ import annotations

from typing import Dict, Tuple

import torch

from .. import ops
from .base import Convolution, ParamDecl, register_part


@register_part("convolution", "causal_residual")
class CausalResidualConvolution(Convolution):
    """y_t = x_t + sum_j w[:, j] * x_(t - taps + 1 + j), channel by channel, zeros before a request's first token; no
    bias.  The last ``taps`` - 1 inputs of a request are its state, so a portion of a prompt or a single decoded
    token continues where the step before stopped.  The input is float32 (a norm's output before any rounding),
    the result has the compute type."""

    graph_safe = True

    def __init__(self, hidden_size: int, taps: int):
        if taps < 1:
            raise ValueError(f"convolution: {taps} taps")
        self.hidden_size, self.taps = hidden_size, int(taps)
        self.weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.hidden_size, self.taps), "vector", "weight")}

    def state_shape(self) -> Tuple[int, ...]:
        return (self.taps - 1, self.hidden_size)

    def forward(self, x: torch.Tensor, ctx, state: torch.Tensor) -> torch.Tensor:
        return ops.causal_conv(x, self.weight, state, ctx.q_starts, ctx.seq_slots, ctx.compute_dtype)

    def forward_pair(self, x: torch.Tensor, state: torch.Tensor, other: "CausalResidualConvolution", x2: torch.Tensor,
                     state2: torch.Tensor, ctx):
        """This convolution of ``x`` and ``other`` (of the same sizes) of ``x2`` in the same kernels."""
        return ops.causal_conv(x, self.weight, state, ctx.q_starts, ctx.seq_slots, ctx.compute_dtype, x2, other.weight, state2)
