"""A feed-forward of routed experts."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import FeedForward, ParamDecl, register_part


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """``n_experts`` small feed-forward layers W_down act(W_up x) (no biases, act = the exact GELU) of which every
    token uses ``top``.  Router: z = W_router x in float32, s = sigmoid(z); the ``top`` experts with the largest
    s + correction are chosen (the correction only moves the choice), their weights are their s divided by the sum of
    the chosen s (+ 1e-20) times ``route_scale``, and the output is the weighted sum of their outputs, float32.

    ``scores="softmax"``: s is the softmax of z over all experts instead.  ``groups`` > 1: the experts form that many
    equal groups of neighbours, a group's score is the largest score in it, and only experts of the ``keep`` best groups
    can be chosen.  ``renorm=False``: the weights are the chosen scores themselves (times ``route_scale``).
    ``correction=False``: the choice goes by the scores alone (no parameter).  ``gated`` (a gate activation's name, or
    None): an expert is W_down (act(W_gate x) * (W_up x)); its gate and up rows lie in turn in ``up_weight``
    [n_experts * 2 ff, hidden], and the first product's epilogue is act(gate) * up.

    A step: the router (a kernel), the (token, choice) pairs grouped by expert on the device (nothing waits for
    the host: the table of row tiles has its worst-case length and unused tiles are empty), one product per expert
    over its tiles for W_up with the GELU in its epilogue, one for W_down with the pair's weight in its epilogue,
    and the sum of a token's rows in the order of its choices.  The experts' matrices lie one after the other:
    ``up_weight`` [n_experts * ff, hidden], ``down_weight`` [n_experts * hidden, ff]."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, n_experts: int, top: int, route_scale: float = 1.0,
                 scores: str = "sigmoid", groups: int = 1, keep: int = 1, renorm: bool = True, correction: bool = True,
                 gated: Optional[str] = None):
        if not 1 <= top <= n_experts:
            raise ValueError(f"routed experts: top {top} of {n_experts} experts")
        if scores not in ("sigmoid", "softmax"):
            raise ValueError(f"routed experts: unknown scores '{scores}' (sigmoid or softmax)")
        if groups < 1 or n_experts % groups or not 1 <= keep <= groups or (groups > 1 and top > keep * (n_experts // groups)):
            raise ValueError(f"routed experts: {n_experts} experts in {groups} groups of which {keep} are kept do not give "
                             f"{top} choices")
        if gated is not None:
            ops.gate_act_code(gated)
        self.scores, self.groups, self.keep, self.renorm = scores, int(groups), int(keep), bool(renorm)
        self.has_correction, self.gated = bool(correction), gated
        if n_experts > 256 or top > 16:
            raise ValueError(f"routed experts: {n_experts} experts / top {top} are more than the kernels take (256 / 16)")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.n_experts, self.top, self.route_scale = int(n_experts), int(top), float(route_scale)
        self.router_weight = self.correction = self.up_weight = self.down_weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        e, h, f = self.n_experts, self.hidden_size, self.intermediate_size
        decls = {"router_weight": ParamDecl((e, h)),
                 "up_weight": ParamDecl((e * 2 * f, h), layout="interleave_pairs") if self.gated else ParamDecl((e * f, h)),
                 "down_weight": ParamDecl((e * h, f))}
        if self.has_correction:
            decls["correction"] = ParamDecl((e,), "vector", "bias")
        return decls

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        e, h, f = self.n_experts, self.hidden_size, self.intermediate_size
        ids, weights = ops.moe_route(x, self.router_weight, self.correction if self.has_correction else None, self.top,
                                     self.route_scale, scores=self.scores, groups=self.groups, keep=self.keep,
                                     renorm=self.renorm)
        order, slot_of, tiles = ops.moe_group(ids, e)
        if self.gated:
            act = ops.moe_gemm(x, self.up_weight.view(e, 2 * f, h), tiles, order, gather_div=self.top, gated=self.gated)
        else:
            act = ops.moe_gemm(x, self.up_weight.view(e, f, h), tiles, order, gather_div=self.top)
        rows = ops.moe_gemm(act, self.down_weight.view(e, h, f), tiles, order, pair_weight=weights.view(-1))
        return ops.moe_combine(rows, slot_of, x.shape[0], self.top)
