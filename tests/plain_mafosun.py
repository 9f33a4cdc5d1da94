"""A plain, slow Mafosun: whole sequences, float64, no cache, one function per mechanism.

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
def unit_rms(x, eps):
    """x divided by sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def value_norm(v, eps):
    """Every head's values divided by their root mean square (no weight)."""
    return unit_rms(v, eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims); with ``scaling`` (factor, low, high, original) frequencies whose wavelength is beyond
    original/low are divided by the factor, those below original/high stay, and the ones between are blended."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.copy()
    for n, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            out[n] = fi
        elif wavelength > original / low:
            out[n] = fi / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[n] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate(x, positions, freqs, dims, layout):
    """x [T, heads, dim]: the first ``dims`` values of every head rotated; pairs (2i, 2i+1) ('interleaved') or
    (i, i + dims/2) ('half')."""
    out = x.copy()
    ang = positions[:, None].astype(np.float64) * freqs[None, :]  # [T, dims/2]
    c, s = np.cos(ang)[:, None, :].astype(x.dtype), np.sin(ang)[:, None, :].astype(x.dtype)  # (the inputs' type: float64 here)
    if layout == "interleaved":
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    else:
        half = dims // 2
        a, b = x[..., :half], x[..., half:dims]
        out[..., :half] = a * c - b * s
        out[..., half:dims] = b * c + a * s
    return out


def window_pool_attention(q, k, v, scale, window, pool, softcap, sink):
    """q [T, H, d], k [T, G, d], v [T, G, e].  Query i sees keys j with 0 <= i - j < window and, if ``pool``, the mean
    key and mean value of every block of ``pool`` positions that ends at or before i - window.  ``sink``: one added
    to the softmax's denominator."""
    t, heads, _ = q.shape
    group = heads // k.shape[1]
    out = np.zeros((t, heads, v.shape[2]), dtype=v.dtype)
    n_blocks = t // pool if pool else 0
    if n_blocks:
        kp = k[:n_blocks * pool].reshape(n_blocks, pool, *k.shape[1:]).mean(1)
        vp = v[:n_blocks * pool].reshape(n_blocks, pool, *v.shape[1:]).mean(1)
    for i in range(t):
        lo = max(0, i - window + 1)
        seen = max(0, (i - window + 1) // pool) if pool else 0
        for h in range(heads):
            g = h // group
            keys = [k[lo:i + 1, g]] + ([kp[:seen, g]] if seen else [])
            vals = [v[lo:i + 1, g]] + ([vp[:seen, g]] if seen else [])
            keys, vals = np.concatenate(keys), np.concatenate(vals)
            s = keys @ q[i, h] * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            m = max(s.max(), 0.0)
            e = np.exp(s - m)
            den = e.sum() + (math.exp(-m) if sink else 0.0)
            out[i, h] = (e / den) @ vals
    return out


def chunk_attention(q, k, v, scale, chunk):
    """Query i sees keys j <= i of its own chunk (floor(i / chunk) == floor(j / chunk)); ordinary softmax."""
    t, heads, _ = q.shape
    group = heads // k.shape[1]
    out = np.zeros((t, heads, v.shape[2]), dtype=v.dtype)
    for i in range(t):
        lo = i // chunk * chunk
        for h in range(heads):
            g = h // group
            s = k[lo:i + 1, g] @ q[i, h] * scale
            e = np.exp(s - s.max())
            out[i, h] = (e / e.sum()) @ v[lo:i + 1, g]
    return out


def retention(q, k, v, decay):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, per head; q, k [T, H, d], v [T, H, e]."""
    t, heads, d = q.shape
    out = np.zeros((t, heads, v.shape[2]), dtype=v.dtype)
    for h in range(heads):
        state = np.zeros((d, v.shape[2]), dtype=v.dtype)
        for i in range(t):
            state = decay[h] * state + np.outer(k[i, h], v[i, h])
            out[i, h] = state.T @ q[i, h]
    return out


def route(z, top, groups, keep, margins=None):
    """Softmax scores over all experts; only experts of the ``keep`` groups with the largest best score can be
    chosen; the ``top`` largest scores among them, and those scores as weights.  Returns (ids [T, top], weights).
    ``margins`` (a list) receives, per token, by how much of the logits' spread the choice was made: the smaller of the
    distance between the last group kept and the first one dropped and between the last expert chosen and the first
    one not (infinite where there is nothing to drop)."""
    s = np.exp(z - z.max(-1, keepdims=True))
    s /= s.sum(-1, keepdims=True)
    t, experts = s.shape
    per = experts // groups
    ids, weights = np.zeros((t, top), dtype=np.int64), np.zeros((t, top))
    for i in range(t):
        best = s[i].reshape(groups, per).max(1)
        kept = np.argsort(-best, kind="stable")[:keep]
        allowed = np.full(experts, -np.inf)
        for g in kept:
            allowed[g * per:(g + 1) * per] = s[i, g * per:(g + 1) * per]
        chosen = np.argsort(-allowed, kind="stable")[:top]
        ids[i], weights[i] = chosen, s[i, chosen]
        if margins is not None:
            by_group = np.sort(z[i].reshape(groups, per).max(1))[::-1]
            inside = np.sort(np.where(np.isfinite(allowed), z[i], -np.inf))[::-1]
            gap = min(by_group[keep - 1] - by_group[keep] if keep < groups else np.inf,
                      inside[top - 1] - inside[top] if top < keep * per else np.inf)
            margins.append(gap / max(z[i].max() - z[i].min(), 1e-30))
    return ids, weights


# ---------------------------------------------------------------------------------- layers
def attention_mixer(h, positions, w, p, m, eps):
    t = h.shape[0]
    heads, kv, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(t, heads, d)
    k = (h @ w[p + "k"].T).reshape(t, kv, d)
    v = (h @ w[p + "v"].T).reshape(t, kv, e)
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, positions, f, rot["dims"], "interleaved"), rotate(k, positions, f, rot["dims"], "interleaved")
    mask = m["mask"]
    o = window_pool_attention(q, k, v, m["scale"], mask["size"], mask.get("pool", 0), m.get("softcap"), True)
    return o.reshape(t, heads * e) @ w[p + "o"].T


def chunked_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, kv, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ w[p + "q"].T).reshape(t, heads, d), w[p + "q.norm"], eps)
    k = rms_norm((h @ w[p + "k"].T).reshape(t, kv, d), w[p + "k.norm"], eps)
    v = value_norm((h @ w[p + "v"].T).reshape(t, kv, e), eps)
    o = chunk_attention(q, k, v, m["scale"], m["mask"]["size"])
    return o.reshape(t, heads * e) @ w[p + "o"].T


def retention_mixer(h, positions, w, p, m, eps):
    t = h.shape[0]
    heads, d, e = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(t, heads, d)
    k = (h @ w[p + "k"].T).reshape(t, heads, d)
    v = (h @ w[p + "v"].T).reshape(t, heads, e)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, positions, f, rot["dims"], "half"), rotate(k, positions, f, rot["dims"], "half")
    k = k * d ** -0.5
    o = unit_rms(retention(q, k, v, m["decay"]), eps).reshape(t, heads * e)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel_mixer(h, positions, w, p, m, eps):
    left = chunked_mixer(h, w, p + "left.", m["left"], eps)
    right = retention_mixer(h, positions, w, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h, w, p):
    return (np.maximum(h @ w[p + "gate"].T, 0.0) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def expert_ff(h, w, p, mlp, margins=None):
    r = mlp["router"]
    ids, weights = route(h @ w[p + "router"].T, r["top"], r["groups"]["count"], r["groups"]["keep"], margins)
    out = np.zeros_like(h)
    for i in range(h.shape[0]):
        for e, a in zip(ids[i], weights[i]):
            q = f"{p}e{e}."
            out[i] += a * ((silu(h[i] @ w[q + "gate"].T) * (h[i] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out


def forward(cfg: dict, w: dict, tokens, streams=None, margins=None):
    """Logits [T, vocab] of the whole sequence ``tokens``; ``streams`` (a list) receives the stream after each layer,
    ``margins`` (a list) one array [T] for every layer of routed experts: how clear each token's choice was."""
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens, dtype=np.int64)
    positions = np.arange(tokens.shape[0])
    x = rms_norm(w["embed"][tokens], w["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] == "attention":
            y = attention_mixer(x, positions, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            y = parallel_mixer(x, positions, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[p + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = dense_ff(x, w, p + "mlp.")
            else:
                mine = [] if margins is not None else None
                y = expert_ff(x, w, p + "mlp.", mlp, mine)
                if margins is not None:
                    margins.append(np.asarray(mine))
            x = x + rms_norm(y, w[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def load(folder):
    return read_config(folder), read_weights(folder)
