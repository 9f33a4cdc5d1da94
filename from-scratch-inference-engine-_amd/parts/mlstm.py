"""mLSTM: a recurrent mixer whose cache is a matrix memory of fixed size per request."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..cache.manager import StateNeed
from .base import Mixer, ParamDecl, register_part
from .linear import Linear


@register_part("mixer", "mlstm")
class MLSTM(Mixer):
    """Per head a matrix memory S [key_dim, value_dim], a normaliser n [key_dim] and a running maximum m, all float32
    and zero when a request starts:

        i_t = cap tanh((W_i x + b_i) / cap),   f_t = logsigmoid(cap tanh((W_f x + b_f) / cap))
        m_t = max(f_t + m_(t-1), i_t)
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t likewise with k_t alone
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)

    with q = (W_q x) key_dim^(-1/2), k = W_k x, v = W_v x.  Every head's o is divided by its root mean square, the
    heads side by side are multiplied by a weight (all heads' size) and by sigmoid(W_g x), then projected by W_o.

    The projections that read x are two matrices: q, k, v, g in the compute type, and the two gates' rows with
    their biases, whose result is float32 (as everything from there to the norm).  The state lives in the cache
    manager's per-request slots and is carried from step to step; a portion of a prompt and a single decoded token
    go through the same kernels, which walk a request's tokens in order."""

    graph_safe = True  # the step's requests and slots are read from the device tables

    def __init__(self, hidden_size: int, n_heads: int, key_dim: int, value_dim: int, gate_cap: float, norm_eps: float):
        if key_dim > 512:
            raise ValueError(f"mlstm: {key_dim} key channels a head are more than the kernel takes (512)")
        if not gate_cap > 0:
            raise ValueError(f"mlstm: gate_cap {gate_cap} must be positive")
        self.hidden_size, self.n_heads, self.key_dim, self.value_dim = hidden_size, n_heads, key_dim, value_dim
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        self.k_width, self.v_width = n_heads * key_dim, n_heads * value_dim
        self.qkvg = Linear(hidden_size, 2 * self.k_width + 2 * self.v_width)
        self.gates = Linear(hidden_size, 2 * n_heads, bias=True)
        self.o = Linear(self.v_width, hidden_size)
        self.norm_weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"qkvg_weight": ParamDecl((2 * self.k_width + 2 * self.v_width, self.hidden_size)),
                "gates_weight": ParamDecl((2 * self.n_heads, self.hidden_size)),
                "gates_bias": ParamDecl((2 * self.n_heads,), "vector", "bias"),
                "norm_weight": ParamDecl((self.v_width,), "vector", "norm"),
                "o_weight": ParamDecl((self.hidden_size, self.v_width))}

    qkvg_weight = property(lambda s: s.qkvg.weight, lambda s, t: setattr(s.qkvg, "weight", t))
    gates_weight = property(lambda s: s.gates.weight, lambda s, t: setattr(s.gates, "weight", t))
    gates_bias = property(lambda s: s.gates.bias, lambda s, t: setattr(s.gates, "bias", t))
    o_weight = property(lambda s: s.o.weight, lambda s, t: setattr(s.o, "weight", t))

    def prepare(self, device, compute_dtype) -> None:
        copies = bool(self.options.get("weight_copies", True))
        self.qkvg.prepare(copies)
        self.o.prepare(copies)

    def release_optional_memory(self) -> int:
        return self.qkvg.drop_copy() + self.o.drop_copy()

    def state_floats(self) -> int:
        """float32 numbers of a head's record: S, n, m and three unused ones (what the kernels lay out)."""
        return self.key_dim * self.value_dim + self.key_dim + 4

    def cache_need(self) -> StateNeed:
        return StateNeed((self.n_heads, self.state_floats()), "float32")

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        p = self.qkvg(x)
        gates = self.gates(x, out_dtype=torch.float32)  # float32 from here on
        num, den, coef = ops.mlstm_scan(p, 0, self.k_width, 2 * self.k_width, gates, self.gate_cap, self.key_dim ** -0.5,
                                        cache.state, ctx.q_starts, ctx.seq_slots, self.n_heads, self.key_dim, self.value_dim)
        y = ops.mlstm_out(num, den, coef, p[:, 2 * self.k_width + self.v_width:], self.norm_weight, self.norm_eps, x.dtype)
        return self.o.for_residual(y, ctx)
