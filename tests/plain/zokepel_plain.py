"""Plain Zokepel forward pass: whole sequences, no cache, one function per mechanism.

Written from the design's equations in float64 (positions' angles in float32, as the design
computes them), token by token where the design is a recurrence.  Nothing from the product
package is imported; the engine is held against this in both of its precisions.

Notation: T tokens, W model width; a linear weight is stored [out, in] and applied as h @ W.T.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def rms_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def unit_vector(x):
    """x / sqrt(sum(x^2) + 1e-6) over the last axis."""
    return x / np.sqrt((x * x).sum(-1, keepdims=True) + 1e-6)


# --------------------------------------------------------------------------- embedding
def sinusoid(positions, width: int) -> np.ndarray:
    """[T, width]: with f_i = 10000^(-2i/width) and a = p * f_i, out[p, 2i] = sin(a) and out[p, 2i+1] = cos(a); the
    angle a is a float32 product of the float32 position and the float32 frequency."""
    i = np.arange(width // 2, dtype=F64)
    freq = (10000.0 ** (-2.0 * i / width)).astype(np.float32)
    angle = (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32).astype(F64)
    out = np.zeros((len(positions), width), dtype=F64)
    out[:, 0:2 * (width // 2):2] = np.sin(angle)
    out[:, 1:2 * (width // 2):2] = np.cos(angle)
    return out


def embedding(table, ids, scale: float) -> np.ndarray:
    table = np.asarray(table, dtype=F64)
    ids = np.asarray(ids, dtype=np.int64)
    return table[ids] * scale + sinusoid(np.arange(len(ids)), table.shape[1])


# --------------------------------------------------------------------------- feed-forward
def clamped_glu(h, w_gate, w_up, w_down, limit: float) -> np.ndarray:
    g = np.minimum(h @ w_gate.T, limit)
    u = np.clip(h @ w_up.T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


# --------------------------------------------------------------------------- short convolution
def causal_conv(x, taps) -> np.ndarray:
    """x [T, C], taps [C, K] (the last column is the current token's): y[t, c] = sum_j taps[c, j] *
    x[t - (K - 1) + j, c] with zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C), dtype=F64), x], axis=0)
    y = np.zeros((T, C), dtype=F64)
    for j in range(K):
        y += padded[j:j + T] * taps[None, :, j]
    return y


# --------------------------------------------------------------------------- gated delta rule
def delta_rule(q, k, v, beta, g) -> np.ndarray:
    """One head.  q, k [T, D]; v [T, V]; beta [T]; g [T] (one decay for the head) or [T, D] (one per key
    channel, acting on the rows of the state).  The state M [D, V] starts at zero; per token, in this order:
    M = g * M;  w = beta * (v - M' k);  M = M + k w';  out = M' q  (the read-out sees the token's own write)."""
    T, D = q.shape
    V = v.shape[1]
    S = np.zeros((D, V), dtype=F64)
    out = np.zeros((T, V), dtype=F64)
    for t in range(T):
        gt = g[t]
        S = S * (gt[:, None] if np.ndim(gt) else gt)
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def delta_mixer(h, w, p, eps: float, channel: bool) -> np.ndarray:
    """The 'delta' (channel False) and 'channel_delta' (channel True) mixers; w: tensors by their short names."""
    T = h.shape[0]
    H, G, D, V = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = silu(causal_conv(h @ w["q"].T, w["q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ w["k"].T, w["k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ w["v"].T, w["v.conv"])).reshape(T, H, V)
    q = unit_vector(q) * D ** -0.5
    k = unit_vector(k)
    beta = sigmoid(h @ w["b"].T)                                   # [T, H]
    if channel:
        a = ((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).reshape(T, H, D)
        g = np.exp(-np.exp(w["A_log"])[None, :, None] * softplus(a))
        gate = sigmoid((h @ w["g1"].T) @ w["g2"].T).reshape(T, H, V)
    else:
        g = np.exp(-np.exp(w["A_log"])[None, :] * softplus(h @ w["a"].T + w["dt_bias"]))   # [T, H]
        gate = silu(h @ w["g"].T).reshape(T, H, V)
    out = np.zeros((T, H, V), dtype=F64)
    for head in range(H):
        kv = head // (H // G)
        out[:, head] = delta_rule(q[:, kv], k[:, kv], v[:, head], beta[:, head], g[:, head])
    y = unit_rms(out, eps) * w["norm"][None, None, :] * gate
    return y.reshape(T, H * V) @ w["o"].T


# --------------------------------------------------------------------------- attention with a distance bias
def distance_bucket(n: int, rows: int, reach: int) -> int:
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (rows - half))))


def biased_attention(h, w, p, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, G, D, V = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = unit_rms((h @ w["q"].T).reshape(T, H, D), eps)
    k = unit_rms((h @ w["k"].T).reshape(T, G, D), eps)
    v = (h @ w["v"].T).reshape(T, G, V)
    pos = np.arange(T)
    if p.get("q_temp") is not None:                     # a temperature on the queries that grows with the position
        temp = 1.0 + p["q_temp"]["coef"] * np.log(np.floor((pos + 1) / p["q_temp"]["every"]) + 1.0)
        q = q * temp[:, None, None]
    rel = w["rel"]
    buckets = np.array([distance_bucket(n, rel.shape[0], p["bias_max"]) for n in range(T)], dtype=np.int64)
    dist = pos[:, None] - pos[None, :]
    visible = dist >= 0
    out = np.zeros((T, H, V), dtype=F64)
    for head in range(H):
        kv = head // (H // G)
        s = (q[:, head] @ k[:, kv].T) * p["scale"] + rel[buckets[np.maximum(dist, 0)], head]
        s = np.where(visible, s, -np.inf)
        s = np.exp(s - s.max(-1, keepdims=True))
        out[:, head] = (s / s.sum(-1, keepdims=True)) @ v[:, kv]
    return out.reshape(T, H * V) @ w["o"].T


# --------------------------------------------------------------------------- time mixing with a decayed outer-product state
def time_mix(h, w, p, eps: float) -> np.ndarray:
    T, W = h.shape
    H, D = p["heads"], p["dim"]
    prev = np.concatenate([np.zeros((1, W), dtype=F64), h[:-1]], axis=0)
    mix = lambda s: h + (prev - h) * w["mu." + s][None, :]
    r = (mix("r") @ w["r"].T).reshape(T, H, D)
    k = (mix("k") @ w["k"].T).reshape(T, H, D)
    v = (mix("v") @ w["v"].T).reshape(T, H, D)
    gate = silu(mix("g") @ w["g"].T)
    decay = np.exp(-np.exp(np.tanh(mix("w") @ w["w1"].T) @ w["w2"].T + w["w0"])).reshape(T, H, D)
    out = np.zeros((T, H, D), dtype=F64)
    for head in range(H):
        S = np.zeros((D, D), dtype=F64)
        for t in range(T):
            kv = np.outer(k[t, head], v[t, head])
            out[t, head] = (S + w["u"][head][:, None] * kv).T @ r[t, head]
            S = decay[t, head][:, None] * S + kv
    y = unit_rms(out, eps).reshape(T, H * D) * w["norm"][None, :] * gate
    return y @ w["o"].T


def parallel_mixer(h, w, p, eps: float) -> np.ndarray:
    sub = lambda side: {n[len(side) + 1:]: t for n, t in w.items() if n.startswith(side + ".")}
    left = rms_norm(biased_attention(h, sub("left"), p["left"], eps), w["left.out"], eps)
    right = rms_norm(time_mix(h, sub("right"), p["right"], eps), w["right.out"], eps)
    return 0.5 * (left + right)


MIXERS = {
    "delta": lambda h, w, p, eps: delta_mixer(h, w, p, eps, channel=False),
    "channel_delta": lambda h, w, p, eps: delta_mixer(h, w, p, eps, channel=True),
    "parallel": parallel_mixer,
}


# --------------------------------------------------------------------------- the model
def run_order(cfg) -> list:
    """[(layer, first of a repeated pass)]: layers start .. stop-1 run `times` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(i, False) for i in range(loop["start"])]
    for rep in range(loop["times"]):
        order += [(i, rep > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def layer(x, cfg, weights, i: int) -> np.ndarray:
    spec, eps = cfg["layers"][i], cfg["norm"]["eps"]
    pre = f"l{i}."
    w = {n[len(pre) + 4:]: t for n, t in weights.items() if n.startswith(pre + "mix.")}
    delta = MIXERS[spec["type"]](rms_norm(x, weights[pre + "norm1"], eps), w, spec["mixer"], eps)
    if spec.get("mlp") is not None:
        m = spec["mlp"]
        assert m["kind"] == "dense"
        delta = delta + clamped_glu(rms_norm(x, weights[pre + "norm2"], eps), weights[pre + "mlp.gate"],
                                    weights[pre + "mlp.up"], weights[pre + "mlp.down"], m["limit"])
    return x + delta


def forward(weights, cfg, ids, layers_out: list | None = None) -> np.ndarray:
    """[T, vocab] logits of a whole sequence; `layers_out` collects the residual stream after every layer run."""
    e0 = embedding(weights["embed"], ids, cfg["embedding"]["scale"])
    x = e0.copy()
    for i, again in run_order(cfg):
        if again:
            x = x + e0
        x = layer(x, cfg, weights, i)
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, weights["final.norm"], cfg["norm"]["eps"]) @ weights["head"].T


# --------------------------------------------------------------------------- reading a model folder
def read_safetensors(path: str) -> dict:
    """name -> float64 (or int64) array: an 8-byte length, that many bytes of JSON, then the data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, e in header.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = np.frombuffer(data[lo:hi], dtype=np.uint8)
        if e["dtype"] == "BF16":
            arr = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(F64)
        elif e["dtype"] == "F32":
            arr = raw.view(np.float32).astype(F64)
        elif e["dtype"] == "I32":
            arr = raw.view(np.int32).astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {e['dtype']}")
        out[name] = arr.reshape(e["shape"])
    return out


def load_model_dir(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return read_safetensors(os.path.join(model_dir, "model.safetensors")), cfg
