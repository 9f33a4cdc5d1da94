"""The arrangement of a layer's parts."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Block, Convolution, FeedForward, HiddenState, Mixer, Norm, Part, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += ffn(norm2(x))  (src/model/model.cpp:106-139).  The sums are
    left pending in the hidden state, so the next norm (this block's second, the next block's
    first, or the model's last) adds them in the same pass that normalises."""

    graph_safe = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def sub_parts(self) -> Dict[str, Part]:
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def forward(self, hidden: HiddenState, ctx, cache) -> None:
        x = self.mixer_norm(hidden, ctx.compute_dtype)
        hidden.delta = self.mixer.forward(x, ctx, cache)
        x = self.ffn_norm(hidden, ctx.compute_dtype)
        hidden.delta = self.ffn.forward(x, ctx)


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    """A norm before and after every sublayer: x += post1(mixer(norm1(x))); x += post2(ffn(norm2(x))).
    A sublayer's output stays pending in the hidden state together with its post norm; the norm that reads
    the stream next (this block's second, the next block's first, the model's last) runs the post norm,
    the sum and itself in one pass.  ``ffn=None``: the layer has no feed-forward (and no norms for it)."""

    graph_safe = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, mixer_post_norm: Norm, ffn_norm: Optional[Norm] = None,
                 ffn: Optional[FeedForward] = None, ffn_post_norm: Optional[Norm] = None):
        if (ffn is None) != (ffn_norm is None) or (ffn is None) != (ffn_post_norm is None):
            raise ValueError("sandwich_norm block: a feed-forward comes with both of its norms, or none of the three")
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.ffn_norm, self.ffn, self.ffn_post_norm = ffn_norm, ffn, ffn_post_norm

    def sub_parts(self) -> Dict[str, Part]:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "mixer_post_norm": self.mixer_post_norm}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn, ffn_post_norm=self.ffn_post_norm)
        return parts

    def forward(self, hidden: HiddenState, ctx, cache) -> None:
        x = self.mixer_norm(hidden, ctx.compute_dtype)
        hidden.delta, hidden.delta_norm = self.mixer.forward(x, ctx, cache), self.mixer_post_norm
        if self.ffn is not None:
            x = self.ffn_norm(hidden, ctx.compute_dtype)
            hidden.delta, hidden.delta_norm = self.ffn.forward(x, ctx), self.ffn_post_norm


@register_part("block", "branch_norm")
class BranchNormBlock(Block):
    """Norms on the sublayers' outputs only: x += post1(mixer(x)); x += post2(ffn(x)).  The sublayers read the stream
    itself (``reader``: a norm part that returns the stream as it is, ``stream``).  A sublayer's output stays pending
    with its norm; whoever reads the stream next (this block's reader, the next block's, the model's last norm) runs
    that norm and the sum in its own pass.  ``ffn=None``: the layer has no feed-forward."""

    graph_safe = True

    def __init__(self, reader: Norm, mixer: Mixer, mixer_post_norm: Norm, ffn: Optional[FeedForward] = None,
                 ffn_post_norm: Optional[Norm] = None):
        if (ffn is None) != (ffn_post_norm is None):
            raise ValueError("branch_norm block: a feed-forward comes with the norm of its output, or neither")
        self.reader, self.mixer, self.mixer_post_norm = reader, mixer, mixer_post_norm
        self.ffn, self.ffn_post_norm = ffn, ffn_post_norm

    def sub_parts(self) -> Dict[str, Part]:
        parts = {"reader": self.reader, "mixer": self.mixer, "mixer_post_norm": self.mixer_post_norm}
        if self.ffn is not None:
            parts.update(ffn=self.ffn, ffn_post_norm=self.ffn_post_norm)
        return parts

    def forward(self, hidden: HiddenState, ctx, cache) -> None:
        x = self.reader(hidden, ctx.compute_dtype)
        hidden.delta, hidden.delta_norm = self.mixer.forward(x, ctx, cache), self.mixer_post_norm
        if self.ffn is not None:
            x = self.reader(hidden, ctx.compute_dtype)
            hidden.delta, hidden.delta_norm = self.ffn.forward(x, ctx), self.ffn_post_norm


@register_part("block", "parallel")
class ParallelBlock(Block):
    """Mixer and feed-forward side by side: x += mixer(norm1(x)) + ffn(norm2(x)), both norms of the same x.  The two
    outputs stay pending in the hidden state as two deltas, and the norm that reads the stream next adds both in
    the pass that normalises; this block's two norms are one pass as well (``Norm.pair``).  ``ffn=None``: the layer
    has no feed-forward (and no second norm).  ``residual_scale`` = m: x += m * (mixer(..) + ffn(..)); the factor
    travels with the pending deltas (norms that set ``scales_deltas``).  ``mixer_conv`` / ``ffn_conv``: a short causal
    convolution between a norm and its sublayer; what they keep per request is the block's own state."""

    graph_safe = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Optional[Norm] = None, ffn: Optional[FeedForward] = None,
                 residual_scale: float = 1.0, mixer_conv: Optional[Convolution] = None,
                 ffn_conv: Optional[Convolution] = None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("parallel block: a feed-forward comes with its norm, or neither")
        if ffn is None and ffn_conv is not None:
            raise ValueError("parallel block: a convolution in front of a feed-forward that is not there")
        if not mixer_norm.adds_two_deltas or (ffn_norm is not None and not ffn_norm.adds_two_deltas):
            raise ValueError("parallel block: its norms must add two pending deltas and come as a pair (layer_norm does)")
        self.residual_scale = float(residual_scale)
        if self.residual_scale != 1.0 and not (mixer_norm.scales_deltas and (ffn_norm is None or ffn_norm.scales_deltas)):
            raise ValueError("parallel block: a factor on the sublayers' sum needs norms that apply it (group_rms_norm does)")
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.mixer_conv, self.ffn_conv = mixer_conv, ffn_conv
        self._convs = [c for c in (mixer_conv, ffn_conv) if c is not None]
        if len({c.state_shape() for c in self._convs}) > 1:
            raise ValueError("parallel block: its convolutions must keep states of one shape")

    def sub_parts(self) -> Dict[str, Part]:
        parts = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            parts.update(ffn_norm=self.ffn_norm, ffn=self.ffn)
        if self.mixer_conv is not None:
            parts["mixer_conv"] = self.mixer_conv
        if self.ffn_conv is not None:
            parts["ffn_conv"] = self.ffn_conv
        return parts

    def state_need(self):
        if not self._convs or 0 in self._convs[0].state_shape():
            return None  # (a convolution of one tap keeps nothing)
        from ..cache.needs import StateNeed

        return StateNeed((len(self._convs), *self._convs[0].state_shape()), "float32")

    def _conv(self, conv: Optional[Convolution], x: torch.Tensor, ctx, state) -> torch.Tensor:
        if conv is None:
            return x
        if 0 in conv.state_shape():
            return conv.forward(x, ctx, None)
        if state is None or state.state is None:
            raise RuntimeError("parallel block: no state for its convolutions (the model did not ask for the block's need)")
        return conv.forward(x, ctx, state.state[:, self._convs.index(conv)])

    def forward(self, hidden: HiddenState, ctx, cache, state=None) -> None:
        # a convolution reads the norm's output before any rounding and rounds once itself
        a_type = torch.float32 if self.mixer_conv is not None else ctx.compute_dtype
        if self.ffn is None:
            a = self._conv(self.mixer_conv, self.mixer_norm(hidden, a_type), ctx, state)
            hidden.delta = self.mixer.forward(a, ctx, cache)
            hidden.delta_scale = self.residual_scale
            return
        b_type = torch.float32 if self.ffn_conv is not None else ctx.compute_dtype
        if a_type == b_type:
            a, b = self.mixer_norm.pair(hidden, self.ffn_norm, a_type)
        else:
            a = self.mixer_norm(hidden, a_type)  # (adds the pending deltas; the second norm then finds none)
            b = self.ffn_norm(hidden, b_type)
        pair = getattr(self.mixer_conv, "forward_pair", None)
        if (pair is not None and type(self.ffn_conv) is type(self.mixer_conv) and 0 not in self.mixer_conv.state_shape()
                and self.mixer_conv.state_shape() == self.ffn_conv.state_shape()):
            if state is None or state.state is None:
                raise RuntimeError("parallel block: no state for its convolutions (the model did not ask for the block's need)")
            a, b = pair(a, state.state[:, 0], self.ffn_conv, b, state.state[:, 1], ctx)  # two convolutions, one pass
        else:
            a = self._conv(self.mixer_conv, a, ctx, state)
            b = self._conv(self.ffn_conv, b, ctx, state)
        hidden.delta = self.mixer.forward(a, ctx, cache)
        hidden.delta2 = self.ffn.forward(b, ctx)
        hidden.delta_scale = self.residual_scale
