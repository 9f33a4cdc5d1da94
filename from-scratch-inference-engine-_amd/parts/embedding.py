"""Token embedding and the LM head."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import ParamDecl, Part
from .linear import Linear


class TokenEmbedding(Part):
    """x[t] = table[ids[t]] (src/model/nn.cpp:90-108, which does not scale) times ``scale``, written as
    the float32 residual stream.  ``norm`` (a norm part as wide as the stream, or None): the rows go through it, in
    float32, before they become the stream."""

    kind = "embedding"
    graph_safe = True  # reads the step's token ids from the device

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, norm=None):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.scale = float(scale)
        self.norm = norm
        self.weight = None

    def sub_parts(self):
        return {} if self.norm is None else {"norm": self.norm}

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size))}

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        x = ops.embedding(self.weight, ids, scale=self.scale)
        return x if self.norm is None else self.norm.plain(x, out=x)

    def cache_need(self):
        """What the embedding keeps for a request between steps (a need of ``cache.needs``), or None."""
        return None

    def embed(self, ctx, cache) -> torch.Tensor:
        """The float32 stream of the step's tokens; ``cache`` is the view of what ``cache_need`` asked for."""
        return self.forward(ctx.token_ids)


class PairHashEmbedding(TokenEmbedding):
    """x[t] = table[id_t] * scale + pairs[(id_{t-1} * mul_prev + id_t * mul_cur) mod buckets]: a second table of
    ``buckets`` + 1 rows, addressed by a hash of the token and the one before it; a request's first token takes the
    last row.  The token before a portion's first one comes from the request's state slot (one int32: the latest
    id + 1, zero when the request starts), which the step brings up to date, so portions, single tokens and
    sampled ids that only the device knows all see the right neighbour."""

    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int, mul_cur: int, scale: float = 1.0):
        super().__init__(vocab_size, hidden_size, scale)
        if buckets < 1:
            raise ValueError(f"pair embedding: buckets {buckets} must be positive")
        self.buckets, self.mul_prev, self.mul_cur, self.scale = int(buckets), int(mul_prev), int(mul_cur), float(scale)
        self.pair_weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size)),
                "pair_weight": ParamDecl((self.buckets + 1, self.hidden_size))}

    def cache_need(self):
        from ..cache.needs import StateNeed

        return StateNeed((1,), "int32")

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        raise RuntimeError("pair embedding: the step's tables and the requests' state are needed (embed)")

    def embed(self, ctx, cache) -> torch.Tensor:
        if cache is None or cache.state is None:
            raise RuntimeError("pair embedding: no state slots (the model did not ask for the embedding's cache need)")
        return ops.pair_embedding(self.weight, self.pair_weight, ctx.token_ids, ctx.q_starts, ctx.seq_slots, cache.state,
                                  self.mul_prev, self.mul_cur, self.scale)

class LMHead(Part):
    """logits = x . W^T in float32, no bias (src/model/model.cpp:144-148).  With tied embeddings
    its weight is bound to the embedding table.  ``softcap`` (a positive number): the logits become
    softcap * tanh(logits / softcap)."""

    kind = "lm_head"
    graph_safe = True

    def __init__(self, hidden_size: int, vocab_size: int, softcap: Optional[float] = None):
        if softcap is not None and not softcap > 0:
            raise ValueError(f"lm head: softcap {softcap} must be positive")
        self.softcap = None if softcap is None else float(softcap)
        self.linear = Linear(hidden_size, vocab_size)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size))}

    @property
    def weight(self):
        return self.linear.weight

    @weight.setter
    def weight(self, t):
        self.linear.weight = t

    def prepare(self, device, compute_dtype) -> None:
        self.linear.prepare(bool(self.options.get("weight_copies", True)))

    def release_optional_memory(self) -> int:
        return self.linear.drop_copy()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = self.linear(x, out_dtype=torch.float32)
        return logits if self.softcap is None else ops.softcap(logits, self.softcap)
