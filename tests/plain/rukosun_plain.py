"""Plain Rukosun forward pass: whole sequences, no cache, one function per mechanism.

Written from the design's equations in float64 (rotation angles in float32, as the design computes
them).  Nothing from the product package is imported; the engine is held against this in both of its
precisions.

Notation: T tokens, W model width; a linear weight is stored [out, in] and applied as h @ W.T.
"""
from __future__ import annotations

import math

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def rms_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def layer_norm(x, gain, bias, eps):
    """(x - mean) / sqrt(var + eps) * gain + bias, var the mean of squared deviations."""
    d = x - x.mean(-1, keepdims=True)
    return d / np.sqrt((d * d).mean(-1, keepdims=True) + eps) * gain + bias


# --------------------------------------------------------------------------- embedding
def bigram_rows(tokens, buckets: int, mul_prev: int, mul_cur: int) -> np.ndarray:
    """Row of the bigram table for every token: (previous * mul_prev + token * mul_cur) mod buckets, and row
    `buckets` for a sequence's first token."""
    rows = np.empty(len(tokens), dtype=np.int64)
    for t, tok in enumerate(tokens):
        rows[t] = buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets
    return rows


def embedding(tokens, w, cfg) -> np.ndarray:
    """table row + bigram row + learned position row."""
    tokens = np.asarray(tokens, dtype=np.int64)
    x = w["embed"][tokens].astype(F64)
    big = (cfg.get("embedding") or {}).get("bigram")
    if big is not None:
        x = x + w["bigram"][bigram_rows(tokens, int(big["buckets"]), int(big["mul_prev"]), int(big["mul_cur"]))]
    if "pos" in w:
        x = x + w["pos"][np.arange(len(tokens))]
    return x


# --------------------------------------------------------------------------- rotation
def rotate(x, positions, base: float, dims: int, interleaved: bool) -> np.ndarray:
    """Rotates the first `dims` entries of the last axis of x [T, ..., n]; pairs (2i, 2i+1) when interleaved, else
    (i, i + dims/2); angle = float32(p) * float32(base^(-2i/dims))."""
    half = dims // 2
    i = np.arange(half, dtype=F64)
    freq = (float(base) ** (-2.0 * i / dims)).astype(np.float32)
    ang = (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32).astype(F64)
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (half,)
    cos, sin = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    out = x.astype(F64).copy()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- attention
def windowed_softmax_attention(q, k, v, scale: float, window, sink=None) -> np.ndarray:
    """q [T, H, dq], k [T, H, dq], v [T, H, dv] -> [T, H, dv].  Query i sees keys j with 0 <= i - j < window (all
    j <= i when window is None).  With `sink` [H] the softmax's denominator also holds exp(sink_h)."""
    T, H, _ = q.shape
    out = np.zeros((T, H, v.shape[-1]), dtype=F64)
    for h in range(H):
        s = (q[:, h] @ k[:, h].T) * scale
        i, j = np.arange(T)[:, None], np.arange(T)[None, :]
        seen = (j <= i) if window is None else ((j <= i) & (i - j < window))
        s = np.where(seen, s, -np.inf)
        m = s.max(-1, keepdims=True)
        if sink is not None:
            m = np.maximum(m, sink[h])
        e = np.exp(s - m)
        den = e.sum(-1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, h]
    return out


def latent_attention(h, w, pre: str, m, eps: float, positions, kind: str) -> np.ndarray:
    """Both latent-attention mixers.  `latent_attention`: queries through a normed latent, interleaved rotation, a
    sink in the softmax, a sigmoid output gate.  `latent_attention_2`: direct queries, rotate-half rotation, plain
    softmax, no gate."""
    H, D, R, V, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    T = h.shape[0]
    first = kind == "latent_attention"
    if first:
        cq = rms_norm(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps)
        q = cq @ w[pre + "uq"].T
    else:
        q = h @ w[pre + "q"].T
    q = q.reshape(T, H, D + R)
    dkv = h @ w[pre + "dkv"].T
    c = rms_norm(dkv[:, :C], w[pre + "dkv.norm"], eps)
    k_rot = dkv[:, C:C + R]
    rot = m.get("rot") or {}
    base, dims = float(rot["base"]), int(rot.get("dims", R))
    q_rot = rotate(q[:, :, D:], positions, base, dims, interleaved=first)
    k_rot = rotate(k_rot[:, None, :], positions, base, dims, interleaved=first)
    k_nope = (c @ w[pre + "uk"].T).reshape(T, H, D)
    v = (c @ w[pre + "uv"].T).reshape(T, H, V)
    qq = np.concatenate([q[:, :, :D], q_rot], axis=-1)
    kk = np.concatenate([k_nope, np.broadcast_to(k_rot, (T, H, R))], axis=-1)
    mask = m.get("mask") or {}
    window = mask.get("size")
    o = windowed_softmax_attention(qq, kk, v, float(m["scale"]), None if window is None else int(window),
                                   w[pre + "sink"].astype(F64) if first else None)
    o = o.reshape(T, H * V)
    if first:
        o = o * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


# --------------------------------------------------------------------------- feed-forward
def poly_norm(z, coef, eps: float) -> np.ndarray:
    """a N(z) + b N(z^2) + c N(z^3) + e, N = division by the root mean square over the last axis."""
    a, b, c, e = (float(t) for t in coef)
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def feed_forward(h, w, pre: str, eps: float) -> np.ndarray:
    return poly_norm(h @ w[pre + "up"].T, w[pre + "act"], eps) @ w[pre + "down"].T


# --------------------------------------------------------------------------- the model
def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def hyper_read(xs, coef):
    """u = sum_s coef[s] x_s; xs [S, T, W]."""
    return np.tensordot(coef.astype(F64), xs, axes=(0, 0))


def hyper_write(xs, mix, out, y):
    """x_t <- sum_s mix[s, t] x_s + out[t] y, all streams at once from the old ones."""
    new = np.tensordot(mix.astype(F64).T, xs, axes=(1, 0))
    return new + out.astype(F64)[:, None, None] * y[None]


def forward(cfg, w, tokens, layers_out=None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence.  `w`: name -> float64 array.  `layers_out`: a list that receives the
    residual stream (the sum of the streams) after every layer run."""
    eps = float(cfg["norm"]["eps"])
    T = len(tokens)
    positions = np.arange(T)
    x = embedding(tokens, w, cfg)
    streams = cfg.get("streams")
    xs = None if streams is None else np.stack([x] * int(streams))
    for i in run_order(cfg):
        layer = cfg["layers"][i]
        p = f"l{i}."

        def sub(q, fn):
            nonlocal x, xs
            g, b = w[f"{p}norm{q}"], w[f"{p}norm{q}.b"]
            if xs is None:
                x = x + fn(layer_norm(x, g, b, eps))
            else:
                u = hyper_read(xs, w[f"{p}hc{q}.in"])
                xs = hyper_write(xs, w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"], fn(layer_norm(u, g, b, eps)))

        sub(1, lambda hh: latent_attention(hh, w, p + "mix.", layer["mixer"], eps, positions, layer["type"]))
        if layer.get("mlp") is not None:
            sub(2, lambda hh: feed_forward(hh, w, p + "mlp.", eps))
        if layers_out is not None:
            layers_out.append(x.copy() if xs is None else xs.sum(0))
    if xs is not None:
        x = xs.sum(0)
    return layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
