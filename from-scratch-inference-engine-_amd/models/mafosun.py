"""Mafosun: a decoder whose sublayers read the stream itself and whose outputs alone are normed; which parts, in which
order, from which checkpoint tensors."""

from __future__ import annotations

from typing import List

from ..config.mafosun import ATTENTION, DENSE, PARALLEL, AttentionConfig, MafosunConfig, RotationConfig
from ..parts.base import make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import ParamBinding, TensorSpec
from .registry import register_architecture
from .spec import LayerCall, ModelSpec, bind


def build_mafosun(cfg: MafosunConfig) -> ModelSpec:
    """x = norm(embed[token]); layer i: x += norm1(mixer(x)), x += norm2(ff(x)), all RMS norms with a plain weight; after
    the last layer the model's norm and the head, which is the embedding table.  Mixers: attention over a window with
    pooled blocks of older positions, interleaved rotation with rescaled frequencies, capped scores and a sink of score
    0; or chunked attention with normed values beside retention.  Tensor names: ``embed``, ``embed.norm``,
    ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*`` (``.left.*`` and ``.right.*`` for two mixers side by side),
    ``l<i>.mlp.*`` (an expert's matrices are ``l<i>.mlp.e<j>.gate``, ``.up`` and ``.down``), ``final.norm``."""
    w, eps = cfg.width, cfg.norm_eps
    bindings: List[ParamBinding] = []

    def norm(name: str, size: int = w):
        part = make_part("norm", "rms_norm", hidden_size=size, eps=eps)
        bind(bindings, part, "weight", [TensorSpec(name, (size,), "norm")])
        return part

    def rotation(rot: RotationConfig, dim: int):
        if rot is None:
            return make_part("position", "none")
        return make_part("position", "rope", head_dim=dim, theta=rot.base, rotary_dim=rot.dims, layout="half",
                         bands=rot.scaling)

    def attention(m: AttentionConfig, p: str, chunked: bool):
        mixer = make_part("mixer", "gqa_attention", hidden_size=w, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                          qkv_bias=False, position=rotation(m.rot, m.dim), scale=m.scale, value_dim=m.vdim,
                          q_norm=norm(p + "q.norm", m.dim), k_norm=norm(p + "k.norm", m.dim), softcap=m.softcap,
                          fused_prep=True,
                          **(dict(chunk=m.mask_size, value_unit_norm_eps=eps) if chunked else
                             dict(window=m.mask_size, pool=m.pool, unit_sink=True, interleaved_pairs=m.rot is not None)))
        bind(bindings, mixer, "qkv_weight", [TensorSpec(p + "q", (m.heads * m.dim, w)),
                                             TensorSpec(p + "k", (m.kv_heads * m.dim, w)),
                                             TensorSpec(p + "v", (m.kv_heads * m.vdim, w))])
        bind(bindings, mixer, "o_weight", [TensorSpec(p + "o", (w, m.heads * m.vdim))])
        return mixer

    embedding = TokenEmbedding(cfg.vocab, w, norm=norm("embed.norm"))
    embed_spec = TensorSpec("embed", (cfg.vocab, w))
    bind(bindings, embedding, "weight", [embed_spec])

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", layer.mixer
        if layer.kind == ATTENTION:
            mixer = attention(m, p, chunked=False)
        elif layer.kind == PARALLEL:
            r, q = m.right, p + "right."
            right = make_part("mixer", "retention", hidden_size=w, n_heads=r.heads, key_dim=r.dim, value_dim=r.vdim,
                              decay=r.decay, position=rotation(r.rot, r.dim), norm_eps=eps, gate_activation="silu")
            bind(bindings, right, "qkvg_weight", [TensorSpec(q + "q", (r.heads * r.dim, w)), TensorSpec(q + "k", (r.heads * r.dim, w)),
                                                  TensorSpec(q + "v", (r.heads * r.vdim, w)), TensorSpec(q + "g", (r.heads * r.vdim, w))])
            bind(bindings, right, "o_weight", [TensorSpec(q + "o", (w, r.heads * r.vdim))])
            mixer = make_part("mixer", "side_by_side", left=attention(m.left, p + "left.", chunked=True), right=right,
                              left_scale=m.left_scale, right_scale=m.right_scale)
        else:  # pragma: no cover - the configuration has refused it
            raise ValueError(layer.kind)
        parts = dict(reader=make_part("norm", "stream", hidden_size=w), mixer=mixer, mixer_post_norm=norm(f"l{i}.norm1"))
        if layer.mlp is not None:
            e, q = layer.mlp, f"l{i}.mlp."
            if e.kind == DENSE:
                ffn = make_part("feed_forward", "gated", hidden_size=w, intermediate_size=e.ff, activation="relu")
                bind(bindings, ffn, "gate_up_weight", [TensorSpec(q + "gate", (e.ff, w)), TensorSpec(q + "up", (e.ff, w))])
                bind(bindings, ffn, "down_weight", [TensorSpec(q + "down", (w, e.ff))])
            else:
                ffn = make_part("feed_forward", "routed_experts", hidden_size=w, intermediate_size=e.ff, n_experts=e.experts,
                                top=e.top, scores="softmax", groups=e.groups, keep=e.keep, renorm=False, correction=False,
                                gated="silu")
                bind(bindings, ffn, "router_weight", [TensorSpec(q + "router", (e.experts, w))])
                bind(bindings, ffn, "up_weight", [TensorSpec(f"{q}e{j}.{name}", (e.ff, w))
                                                  for j in range(e.experts) for name in ("gate", "up")])
                bind(bindings, ffn, "down_weight", [TensorSpec(f"{q}e{j}.down", (w, e.ff)) for j in range(e.experts)])
            parts.update(ffn=ffn, ffn_post_norm=norm(f"l{i}.norm2"))
        layers.append(make_part("block", "branch_norm", **parts))
        schedule.append(LayerCall(i))

    final_norm = norm("final.norm")
    lm_head = LMHead(w, cfg.vocab)
    bind(bindings, lm_head, "weight", [embed_spec])
    # a layer without feed-forward may still carry the norm of one: not read
    unused = tuple(f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.mlp is None)
    return ModelSpec(config=cfg, embedding=embedding, layers=layers, schedule=schedule, final_norm=final_norm,
                     lm_head=lm_head, bindings=bindings, ignore_unexpected=unused)


register_architecture("Mafosun", MafosunConfig, build_mafosun)
