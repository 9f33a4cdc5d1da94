"""Fiterax: a decoder whose layers run a mixer (grouped-query attention or an mLSTM) and a feed-forward of routed
experts side by side on the same stream; which parts, in which order, from which checkpoint tensors."""

from __future__ import annotations

from typing import List

from ..config.fiterax import ATTENTION, MLSTM, FiteraxConfig
from ..parts.base import make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import ParamBinding, TensorSpec
from .registry import register_architecture
from .spec import LayerCall, ModelSpec, bind


def build_fiterax(cfg: FiteraxConfig) -> ModelSpec:
    """Layer i: x += m * (mixer(conv1(norm1(x))) + ff(conv2(norm2(x)))), both norms RMS norms in groups of the same
    x, each followed by a short causal convolution that is added to its input; a layer without feed-forward has no
    second norm.  The embedding is the token's row times a constant.  After the last layer the model's norm and the
    head.  Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``,
    ``head``; an expert's matrices are ``l<i>.mlp.e<j>.up`` and ``.down``."""
    w, eps, groups = cfg.width, cfg.norm_eps, cfg.norm_groups
    bindings: List[ParamBinding] = []

    def norm(name: str):
        part = make_part("norm", "group_rms_norm", hidden_size=w, eps=eps, groups=groups)
        bind(bindings, part, "weight", [TensorSpec(name, (w,), "norm")])
        return part

    def convolution(name: str):
        part = make_part("convolution", "causal_residual", hidden_size=w, taps=cfg.canon_taps)
        bind(bindings, part, "weight", [TensorSpec(name, (w, cfg.canon_taps), "weight")])
        return part

    embedding = TokenEmbedding(cfg.vocab, w, scale=cfg.embedding_scale)
    bind(bindings, embedding, "weight", [TensorSpec("embed", (cfg.vocab, w))])

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", layer.mixer
        if layer.kind == ATTENTION:
            position = (make_part("position", "rope", head_dim=m.dim, theta=m.rot_base, rotary_dim=m.rot_dims, layout="half")
                        if m.rot_dims else make_part("position", "none"))
            mixer = make_part("mixer", "gqa_attention", hidden_size=w, n_heads=m.heads, n_kv_heads=m.kv_heads,
                              head_dim=m.dim, qkv_bias=True, position=position, scale=m.scale, value_dim=m.vdim, gate=True,
                              o_bias=True, unit_norm_eps=eps, head_temperature=True, softcap=m.softcap)
            bind(bindings, mixer, "qkv_weight", [TensorSpec(p + "q", (m.heads * m.dim, w)),
                                                 TensorSpec(p + "k", (m.kv_heads * m.dim, w)),
                                                 TensorSpec(p + "v", (m.kv_heads * m.vdim, w)),
                                                 TensorSpec(p + "g", (m.heads, w))])
            bind(bindings, mixer, "qkv_bias", [TensorSpec(p + "q.b", (m.heads * m.dim,), "bias"),
                                               TensorSpec(p + "k.b", (m.kv_heads * m.dim,), "bias"),
                                               TensorSpec(p + "v.b", (m.kv_heads * m.vdim,), "bias")])
            bind(bindings, mixer, "temperature", [TensorSpec(p + "temp", (m.heads,), "norm")])
            bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, m.heads * m.vdim))])
            bind(bindings, mixer, "o_bias", [TensorSpec(p + "o.b", (w,), "bias")])
        elif layer.kind == MLSTM:
            mixer = make_part("mixer", "mlstm", hidden_size=w, n_heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                              gate_cap=m.gate_cap, norm_eps=eps)
            bind(bindings, mixer, "qkvg_weight", [TensorSpec(p + "q", (m.heads * m.dim, w)),
                                                  TensorSpec(p + "k", (m.heads * m.dim, w)),
                                                  TensorSpec(p + "v", (m.heads * m.vdim, w)),
                                                  TensorSpec(p + "g", (m.heads * m.vdim, w))])
            bind(bindings, mixer, "gates_weight", [TensorSpec(p + "i", (m.heads, w)), TensorSpec(p + "f", (m.heads, w))])
            bind(bindings, mixer, "gates_bias", [TensorSpec(p + "i.b", (m.heads,), "bias"),
                                                 TensorSpec(p + "f.b", (m.heads,), "bias")])
            bind(bindings, mixer, "norm_weight", [TensorSpec(p + "norm", (m.heads * m.vdim,), "norm")])
            bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, m.heads * m.vdim))])
        else:  # pragma: no cover - the configuration has refused it
            raise ValueError(layer.kind)
        parts = dict(mixer_norm=norm(f"l{i}.norm1"), mixer=mixer, residual_scale=cfg.residual_mult,
                     mixer_conv=convolution(f"l{i}.canon1"))
        if layer.mlp is not None:
            e, q = layer.mlp, f"l{i}.mlp."
            ffn = make_part("feed_forward", "routed_experts", hidden_size=w, intermediate_size=e.ff, n_experts=e.experts,
                            top=e.top, route_scale=e.scale)
            bind(bindings, ffn, "router_weight", [TensorSpec(q + "router", (e.experts, w))])
            bind(bindings, ffn, "correction", [TensorSpec(q + "correction", (e.experts,), "bias")])
            bind(bindings, ffn, "up_weight", [TensorSpec(f"{q}e{j}.up", (e.ff, w)) for j in range(e.experts)])
            bind(bindings, ffn, "down_weight", [TensorSpec(f"{q}e{j}.down", (w, e.ff)) for j in range(e.experts)])
            parts.update(ffn_norm=norm(f"l{i}.norm2"), ffn=ffn, ffn_conv=convolution(f"l{i}.canon2"))
        layers.append(make_part("block", "parallel", **parts))
        schedule.append(LayerCall(i))

    final_norm = norm("final.norm")
    lm_head = LMHead(w, cfg.vocab)
    bind(bindings, lm_head, "weight", [TensorSpec("head", (cfg.vocab, w))])
    # a layer without feed-forward may still carry the norm and the convolution in front of one: not read
    unused = tuple(f"l{i}.{name}" for i, layer in enumerate(cfg.layers) if layer.mlp is None for name in ("norm2", "canon2"))
    return ModelSpec(config=cfg, embedding=embedding, layers=layers, schedule=schedule, final_norm=final_norm,
                     lm_head=lm_head, bindings=bindings, ignore_unexpected=unused)


register_architecture("Fiterax", FiteraxConfig, build_fiterax)
