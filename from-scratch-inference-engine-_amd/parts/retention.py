"""Retention: linear attention with a fixed decay per head, and mixers side by side."""

from __future__ import annotations

from typing import Dict, List, Sequence

import torch

from .. import ops
from ..cache.manager import StateNeed
from .base import Mixer, ParamDecl, Part, PositionEncoding, register_part
from .linear import Linear


@register_part("mixer", "retention")
class Retention(Mixer):
    """Per head a state S [key_dim, value_dim] in float32 with a fixed decay:

        S_t = decay_h S_(t-1) + k_t v_t^T,    o_t = S_t^T q_t,

    no softmax and no denominator.  q = W_q x and k = W_k x are turned by the position encoding (the pairs
    (i, i + rotary_dim / 2) of every head), and the product q . k carries the factor ``key_scale`` (default
    key_dim^(-1/2); it multiplies q in the kernel, which gives the same o as a scaled k).  Every head's o is divided
    by its root mean square over the value columns (eps inside the root, no weight), multiplied by act(W_g x) and
    projected by W_o.  The projections that read x are one matrix (q, k, v, g rows one after the other).

    The state lives in the cache manager's per-request slots, zero when a request starts; decays, state and sums
    are float32 whatever the activations' type.  The rotation happens in float32 inside the scan's first kernel.  The walk over a request's tokens is the one of gated linear
    attention (token by token, or chunk by chunk on the float32 matrix instruction for long portions) with the
    head's decay in the place of a decay per token and key channel."""

    graph_safe = True

    def __init__(self, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, decay: Sequence[float],
                 position: PositionEncoding, norm_eps: float, gate_activation: str = "silu", key_scale=None):
        if key_dim > 256:
            raise ValueError(f"retention: {key_dim} key channels a head are more than the kernel takes (256)")
        decay = [float(d) for d in decay]
        if len(decay) != n_heads or not all(0.0 < d <= 1.0 for d in decay):
            raise ValueError(f"retention: {n_heads} heads need as many decays in (0, 1], got {decay}")
        if position.rotates and getattr(position, "layout", None) != "half":
            raise ValueError("retention: the position encoding must be the rotation of the pairs (i, i + rotary_dim / 2), or none")
        ops.gate_act_code(gate_activation)
        self.hidden_size, self.n_heads, self.key_dim, self.value_dim = hidden_size, n_heads, key_dim, value_dim
        self.decay, self.position, self.norm_eps, self.gate_activation = decay, position, float(norm_eps), gate_activation
        self.key_scale = key_dim ** -0.5 if key_scale is None else float(key_scale)
        self.k_width, self.v_width = n_heads * key_dim, n_heads * value_dim
        self.qkvg = Linear(hidden_size, 2 * self.k_width + 2 * self.v_width)
        self.o = Linear(self.v_width, hidden_size)
        self._decay = self._ones = None

    def sub_parts(self) -> Dict[str, Part]:
        return {"position": self.position}

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"qkvg_weight": ParamDecl((2 * self.k_width + 2 * self.v_width, self.hidden_size)),
                "o_weight": ParamDecl((self.hidden_size, self.v_width))}

    qkvg_weight = property(lambda s: s.qkvg.weight, lambda s, t: setattr(s.qkvg, "weight", t))
    o_weight = property(lambda s: s.o.weight, lambda s, t: setattr(s.o, "weight", t))

    def prepare(self, device, compute_dtype) -> None:
        copies = bool(self.options.get("weight_copies", True))
        self.qkvg.prepare(copies)
        self.o.prepare(copies)
        self._decay = torch.tensor(self.decay, dtype=torch.float32, device=device)
        self._ones = torch.ones((self.value_dim,), dtype=torch.float32, device=device)

    def release_optional_memory(self) -> int:
        return self.qkvg.drop_copy() + self.o.drop_copy()

    def cache_need(self) -> StateNeed:
        return StateNeed((self.n_heads, self.key_dim, self.value_dim), "float32")

    @property
    def heads_width(self) -> int:
        """Values a token has behind the gate, in front of the output projection."""
        return self.v_width

    def forward_heads(self, x: torch.Tensor, ctx, cache, out: torch.Tensor, scale: float = 1.0) -> None:
        """``forward`` without the output projection: the gated heads times ``scale`` into ``out`` [T, heads_width]
        (columns of wider rows may do)."""
        self.forward(x, ctx, cache, heads_out=out, heads_scale=scale)

    def forward(self, x: torch.Tensor, ctx, cache, heads_out=None, heads_scale: float = 1.0):
        kw, vw = self.k_width, self.v_width
        p = self.qkvg(x)
        # (the scan's own first kernel turns q and k by the step's cosines and sines as it reads them)
        table = self.position.table(ctx) if self.position.rotates else None
        o = ops.gla_scan(p, 0, kw, 2 * kw, None, cache.state, ctx.q_starts, ctx.seq_slots, self.n_heads, self.key_dim,
                         self.value_dim, self.key_scale, 1.0, head_decay=self._decay, cos_sin=table)
        y = ops.gated_headnorm(o, p[:, 2 * kw + vw:], self._ones, self.norm_eps, self.n_heads, self.gate_activation,
                               out=heads_out, scale=heads_scale)
        return None if heads_out is not None else self.o.for_residual(y, ctx)


@register_part("mixer", "side_by_side")
class SideBySide(Mixer):
    """Two mixers that read the same input; the result is left_scale * left(x) + right_scale * right(x), summed in
    float32.  What the two keep for a request are two caches: ``cache_need`` names them ``left`` and ``right`` and
    ``forward`` gets the views under the same names.

    Where both mixers end in an output projection without bias and can hand over what stands in front of it
    (``forward_heads``, ``heads_width``, a ``Linear`` named ``o``), the two projections are one: the mixers write their
    heads, times their scales, side by side into one row a token, and one product with [W_o left | W_o right] gives the
    sum (the scales multiply the activations in float32, before their one rounding).  ``joint_output=False`` keeps two
    products and a kernel for the weighted sum."""

    def __init__(self, left: Mixer, right: Mixer, left_scale: float = 1.0, right_scale: float = 1.0, joint_output: bool = True):
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)

        def joins(m) -> bool:
            return (callable(getattr(m, "forward_heads", None)) and isinstance(getattr(m, "o", None), Linear) and not m.o.has_bias
                    and getattr(m, "prepared", True))
        self.joint = bool(joint_output) and joins(left) and joins(right) and left.o.out_features == right.o.out_features
        self.o = Linear(left.heads_width + right.heads_width, left.o.out_features) if self.joint else None

    def prepare(self, device, compute_dtype) -> None:
        if self.joint and self.o.weight is None:
            # (the mixers' own prepare runs after this one: they find their projections' weights gone and make no copies)
            self.o.weight = torch.cat([self.left.o.weight, self.right.o.weight], dim=1).contiguous()
            self.left.o.weight = self.right.o.weight = None
            self.o.prepare(bool(self.options.get("weight_copies", True)))

    def release_optional_memory(self) -> int:
        return self.o.drop_copy() if self.joint else 0

    @property
    def graph_safe(self) -> bool:
        return bool(self.left.graph_safe and self.right.graph_safe)

    def sub_parts(self) -> Dict[str, Part]:
        return {"left": self.left, "right": self.right}

    def cache_need(self):
        needs = {"left": self.left.cache_need(), "right": self.right.cache_need()}
        return {k: v for k, v in needs.items() if v is not None} or None

    def planners(self) -> List:
        out = []
        for side in (self.left, self.right):
            mine = side.planners() if callable(getattr(side, "planners", None)) else [side.planner()]
            out += [p for p in mine if p is not None]
        return out

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        cache = cache or {}
        if self.joint:
            wl = self.left.heads_width
            heads = torch.empty((x.shape[0], self.o.in_features), dtype=x.dtype, device=x.device)
            self.left.forward_heads(x, ctx, cache.get("left"), heads[:, :wl], self.left_scale)
            self.right.forward_heads(x, ctx, cache.get("right"), heads[:, wl:], self.right_scale)
            return self.o.for_residual(heads, ctx)
        whole = ctx.partial_sums_ok
        ctx.partial_sums_ok = False  # (both results are added here: each comes whole, not as partial sums)
        try:
            a = self.left.forward(x, ctx, cache.get("left"))
            b = self.right.forward(x, ctx, cache.get("right"))
        finally:
            ctx.partial_sums_ok = whole
        return ops.scaled_sum(a, self.left_scale, b, self.right_scale)
