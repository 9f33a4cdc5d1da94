"""A plain, slow Fiterax: whole sequences, float64, no cache, one function per mechanism.

It shares nothing with the engine: it reads config.json and model.safetensors itself (numpy) and
computes every token of a sequence from scratch.  The tests compare the engine with it.
"""

from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np


# ----------------------------------------------------------------------------------- files
def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def read_weights(folder) -> dict:
    """name -> float64 array (int64 for integer tables) from model.safetensors."""
    data = (Path(folder) / "model.safetensors").read_bytes()
    (n,) = struct.unpack("<Q", data[:8])
    header = json.loads(data[8:8 + n])
    body = data[8 + n:]
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        raw, shape = body[lo:hi], meta["shape"]
        if meta["dtype"] == "BF16":
            bits = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            arr = bits.view(np.float32).astype(np.float64)
        elif meta["dtype"] == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif meta["dtype"] == "I32":
            arr = np.frombuffer(raw, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {meta['dtype']}")
        out[name] = arr.reshape(shape)
    return out


# ------------------------------------------------------------------------------ mechanisms
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def gelu_erf(z):
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def unit_rms(x, eps):
    """x divided by sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def group_rms_norm(x, w, eps, groups):
    """The last axis in ``groups`` equal consecutive parts, each divided by its own root mean square; then times w."""
    t, width = x.shape
    parts = x.reshape(t, groups, width // groups)
    return unit_rms(parts, eps).reshape(t, width) * w


def input_convolution(h, w):
    """h + causal convolution of h over time, channel by channel: w [width, taps], the last tap on the token itself,
    zeros before the sequence's start."""
    taps = w.shape[1]
    out = h.copy()
    for j in range(taps):
        back = taps - 1 - j
        if back < h.shape[0]:
            out[back:] += w[:, j] * h[:h.shape[0] - back]
    return out


def rotate_half(x, positions, base, dims):
    """x [T, heads, dim]: of every head's first ``dims`` values, value i turns with value i + dims/2 by the angle
    position * base^(-2i/dims); the other values stay."""
    if not dims:
        return x
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    a = positions[:, None].astype(np.float64) * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def capped_attention(q, k, v, scale, temps, cap, past=0):
    """q [n, heads, dim] at positions past .. past + n - 1 against k [total, kv, dim], v [total, kv, vdim]: scores times
    ``scale`` and the head's temperature, capped (cap * tanh(score / cap); None: not), causal softmax.  [n, heads, vdim]."""
    n, heads, _ = q.shape
    total, kv, vdim = v.shape
    out = np.zeros((n, heads, vdim))
    seen = np.arange(total)[None, :] <= (past + np.arange(n))[:, None]
    for hd in range(heads):
        g = hd // (heads // kv)
        s = (q[:, hd] @ k[:, g].T) * scale * (1.0 if temps is None else temps[hd])
        if cap:
            s = cap * np.tanh(s / cap)
        s = np.where(seen, s, -np.inf)
        e = np.exp(s - s.max(-1, keepdims=True))
        out[:, hd] = (e / e.sum(-1, keepdims=True)) @ v[:, g]
    return out


def attention_mixer(h, w, p, m, eps):
    """Grouped-query attention with biases, partly rotated and unit-normed q and k, a temperature a head, capped
    scores, and a sigmoid gate a head on the result."""
    t = h.shape[0]
    heads, kv, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(t, heads, dim)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(t, kv, dim)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(t, kv, vdim)
    pos = np.arange(t)
    rot = m.get("rot") or {}
    q = unit_rms(rotate_half(q, pos, rot.get("base", 1.0), rot.get("dims", 0)), eps)
    k = unit_rms(rotate_half(k, pos, rot.get("base", 1.0), rot.get("dims", 0)), eps)
    gate = sigmoid(h @ w[p + "g"].T)  # [T, heads]
    out = capped_attention(q, k, v, m["scale"], w[p + "temp"], m.get("softcap"))
    out = out * gate[:, :, None]
    return out.reshape(t, heads * vdim) @ w[p + "o"].T + w[p + "o.b"]


def matrix_memory(q, k, v, gi, gf, pieces=False):
    """q, k [T, heads, dim], v [T, heads, vdim], log input gates gi and log forget gates gf [T, heads]: per head
    S [dim, vdim], n [dim] and a running maximum that all start at zero; token by token.  [T, heads, vdim].
    ``pieces``: also what the quotient is made of, (S^T q [T, heads, vdim], n . q [T, heads], the maximum [T, heads])."""
    t, heads, dim = q.shape
    vdim = v.shape[2]
    out = np.zeros((t, heads, vdim))
    num, den, top = np.zeros((t, heads, vdim)), np.zeros((t, heads)), np.zeros((t, heads))
    for hd in range(heads):
        S, n, mx = np.zeros((dim, vdim)), np.zeros(dim), 0.0
        for i in range(t):
            new = max(gf[i, hd] + mx, gi[i, hd])
            keep, take = math.exp(gf[i, hd] + mx - new), math.exp(gi[i, hd] - new)
            S = keep * S + take * np.outer(k[i, hd], v[i, hd])
            n = keep * n + take * k[i, hd]
            mx = new
            num[i, hd], den[i, hd], top[i, hd] = S.T @ q[i, hd], n @ q[i, hd], mx
            out[i, hd] = num[i, hd] / (max(abs(den[i, hd]), math.exp(-mx)) + 1e-6)
    return (out, num, den, top) if pieces else out


def capped_gates(zi, zf, cap):
    """(log input gate, log forget gate) from the gates' logits."""
    return cap * np.tanh(zi / cap), log_sigmoid(cap * np.tanh(zf / cap))


def mlstm_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(t, heads, dim) * dim ** -0.5
    k = (h @ w[p + "k"].T).reshape(t, heads, dim)
    v = (h @ w[p + "v"].T).reshape(t, heads, vdim)
    gi, gf = capped_gates(h @ w[p + "i"].T + w[p + "i.b"], h @ w[p + "f"].T + w[p + "f.b"], m["gate_cap"])
    out = matrix_memory(q, k, v, gi, gf)
    out = unit_rms(out, eps).reshape(t, heads * vdim) * w[p + "norm"]
    out = out * sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def route(h, router_w, correction, top, scale):
    """(chosen experts [T, top], their weights [T, top]): sigmoid scores; the choice by score + correction, the
    weights from the scores alone, normalised over the chosen ones, times ``scale``."""
    s = sigmoid(h @ router_w.T)
    order = np.argsort(-(s + correction), axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(s, order, axis=-1)
    return order, chosen / (chosen.sum(-1, keepdims=True) + 1e-20) * scale


def moe_feed_forward(h, w, p, mlp):
    r = mlp["router"]
    experts, weights = route(h, w[p + "router"], w[p + "correction"], r["top"], r["scale"])
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, a in zip(experts[t], weights[t]):
            out[t] += a * (w[f"{p}e{e}.down"] @ gelu_erf(w[f"{p}e{e}.up"] @ h[t]))
    return out


# ------------------------------------------------------------------------------ the model
def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer)."""
    tokens = np.asarray(tokens, dtype=np.int64)
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    mult = cfg.get("residual_mult", 1.0)
    x = w["embed"][tokens] * cfg["embedding"]["scale"]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = input_convolution(group_rms_norm(x, w[p + "norm1"], eps, groups), w[p + "canon1"])
        if layer["type"] == "attention":
            y = attention_mixer(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "mlstm":
            y = mlstm_mixer(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            h2 = input_convolution(group_rms_norm(x, w[p + "norm2"], eps, groups), w[p + "canon2"])
            y = y + moe_feed_forward(h2, w, p + "mlp.", layer["mlp"])
        x = x + mult * y
        after.append(x.copy())
    logits = group_rms_norm(x, w["final.norm"], eps, groups) @ w["head"].T
    return (logits, np.stack(after)) if return_layers else logits
