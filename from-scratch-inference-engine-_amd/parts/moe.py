"""A feed-forward of routed experts."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import FeedForward, ParamDecl, register_part


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """``n_experts`` small feed-forward layers W_down act(W_up x) (no biases, act = the exact GELU) of which every
    token uses ``top``.  Router: z = W_router x in float32, s = sigmoid(z); the ``top`` experts with the largest
    s + correction are chosen (the correction only moves the choice), their weights are their s divided by the sum of
    the chosen s (+ 1e-20) times ``route_scale``, and the output is the weighted sum of their outputs, float32.

    A step: the router (a kernel), the (token, choice) pairs grouped by expert on the device (nothing waits for
    the host: the table of row tiles has its worst-case length and unused tiles are empty), one product per expert
    over its tiles for W_up with the GELU in its epilogue, one for W_down with the pair's weight in its epilogue,
    and the sum of a token's rows in the order of its choices.  The experts' matrices lie one after the other:
    ``up_weight`` [n_experts * ff, hidden], ``down_weight`` [n_experts * hidden, ff]."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, n_experts: int, top: int, route_scale: float = 1.0):
        if not 1 <= top <= n_experts:
            raise ValueError(f"routed experts: top {top} of {n_experts} experts")
        if n_experts > 256 or top > 16:
            raise ValueError(f"routed experts: {n_experts} experts / top {top} are more than the kernels take (256 / 16)")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.n_experts, self.top, self.route_scale = int(n_experts), int(top), float(route_scale)
        self.router_weight = self.correction = self.up_weight = self.down_weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        e, h, f = self.n_experts, self.hidden_size, self.intermediate_size
        return {"router_weight": ParamDecl((e, h)),
                "correction": ParamDecl((e,), "vector", "bias"),
                "up_weight": ParamDecl((e * f, h)),
                "down_weight": ParamDecl((e * h, f))}

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        e, h, f = self.n_experts, self.hidden_size, self.intermediate_size
        ids, weights = ops.moe_route(x, self.router_weight, self.correction, self.top, self.route_scale)
        order, slot_of, tiles = ops.moe_group(ids, e)
        act = ops.moe_gemm(x, self.up_weight.view(e, f, h), tiles, order, gather_div=self.top)
        rows = ops.moe_gemm(act, self.down_weight.view(e, h, f), tiles, order, pair_weight=weights.view(-1))
        return ops.moe_combine(rows, slot_of, x.shape[0], self.top)
