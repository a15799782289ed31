"""Small Rukosun configurations that differ in every size and option, model folders made from them through the
framework's random-weights mode, and the plain implementation's logits for them."""
from __future__ import annotations

import copy
import json
import os

import numpy as np

from tests.plain import rukosun_plain as R


def _mix(kind, heads, dim, rot, vdim, rank, scale, window, base, q_rank=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": rot}}
    if window is not None:
        m["mask"] = {"size": window}
    if q_rank is not None:
        m["q_rank"] = q_rank
    return {"type": kind, "mixer": m}


def _layer(mixer, ff):
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


A1, A2 = "latent_attention", "latent_attention_2"
# P: no size a multiple of 8 where it can be avoided (the plain kernels in both precisions); two streams; a layer without a
# feed-forward; the middle layers run three times; windows of 1, 5 and 37 and a layer that sees everything.
RUKOSUN_P = {
    "architecture": "Rukosun", "vocab": 211, "width": 100, "max_positions": 400, "norm": {"eps": 1e-5}, "streams": 2,
    "embedding": {"bigram": {"buckets": 97, "mul_prev": 31, "mul_cur": 5}},
    "layers": [
        _layer(_mix(A1, 3, 12, 6, 20, 21, 0.3, 5, 1000.0, q_rank=30), 150),
        _layer(_mix(A2, 5, 10, 4, 6, 18, 0.25, 37, 300.0), None),
        _layer(_mix(A1, 2, 18, 10, 14, 33, 0.2, None, 50000.0, q_rank=11), 90),
        _layer(_mix(A2, 3, 6, 2, 10, 9, 0.4, 1, 10.0), 64),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
# Q: aligned sizes (in bfloat16 the matrix-core attention kernels and per-head products), cached rows of 64 and 128
# values, four streams, the whole model run twice, windows that end inside and at page borders.
RUKOSUN_Q = {
    "architecture": "Rukosun", "vocab": 256, "width": 128, "max_positions": 1024, "norm": {"eps": 1e-6}, "streams": 4,
    "embedding": {"bigram": {"buckets": 1021, "mul_prev": 3, "mul_cur": 257}},
    "layers": [
        _layer(_mix(A1, 4, 32, 16, 32, 48, 0.15, 48, 10000.0, q_rank=64), 256),
        _layer(_mix(A2, 8, 16, 32, 16, 96, 0.2, 33, 500000.0), 128),
        _layer(_mix(A1, 2, 64, 16, 64, 48, 0.1, 200, 10000.0, q_rank=32), 192),
    ],
    "loop": {"start": 0, "stop": 3, "times": 2},
}
# R: one residual stream without connections (plain residual sums), no pair table, no loop, odd head counts.
RUKOSUN_R = {
    "architecture": "Rukosun", "vocab": 97, "width": 72, "max_positions": 300, "norm": {"eps": 1e-5},
    "layers": [
        _layer(_mix(A2, 5, 8, 8, 8, 24, 0.25, 20, 100.0), 40),
        _layer(_mix(A1, 3, 16, 8, 24, 40, 0.2, 64, 2000.0, q_rank=24), 100),
        _layer(_mix(A1, 1, 24, 24, 16, 8, 0.3, 7, 2000.0, q_rank=8), None),
    ],
}
# S: hyper-connections over a single stream (`streams: 1`), a loop that runs once, a model of one head.
RUKOSUN_S = {
    "architecture": "Rukosun", "vocab": 64, "width": 48, "max_positions": 256, "norm": {"eps": 1e-6}, "streams": 1,
    "embedding": {"bigram": {"buckets": 13, "mul_prev": 1, "mul_cur": 1}},
    "layers": [
        _layer(_mix(A1, 1, 16, 16, 16, 16, 0.2, 16, 10000.0, q_rank=16), 48),
        _layer(_mix(A2, 1, 16, 16, 16, 16, 0.2, 17, 10000.0), 48),
    ],
    "loop": {"start": 0, "stop": 1, "times": 1},
}
MODELS = {"P": RUKOSUN_P, "Q": RUKOSUN_Q, "R": RUKOSUN_R, "S": RUKOSUN_S}


def single_layer(kind: str, ff=None, streams=3) -> dict:
    """A model of one layer of one mixer kind (and no feed-forward, or nothing but...): the mechanism alone."""
    layer = copy.deepcopy(RUKOSUN_P["layers"][0 if kind == A1 else 1])
    layer["mlp"] = None if ff is None else {"kind": "dense", "ff": ff}
    cfg = {"architecture": "Rukosun", "vocab": 131, "width": 100, "max_positions": 300, "norm": {"eps": 1e-5}, "layers": [layer]}
    if streams is not None:
        cfg["streams"] = streams
    return cfg


def make_model_dir(folder: str, cfg: dict, name: str, seed: int = 0, std: float = 0.1, bias_std: float = 0.7,
                   gain_std: float = 0.3) -> str:
    """Writes a model of configuration `cfg` through the framework's random-weights mode: matrices in bfloat16, so that
    both precisions of the engine and the plain implementation start from the same values; gains, biases, sinks and the
    connections' weights spread widely so that leaving one out shows."""
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    config = config_from_dict(cfg)
    decls = DecoderModel(config.model_spec()).tensor_decls()
    path = os.path.join(folder, f"rukosun_{name}_{seed}")
    write_random_model(path, config, decls, seed=seed, dtype="bfloat16", std=std, gain_std=gain_std, bias_std=bias_std)
    return path


def tokens(seed: int, n: int, vocab: int) -> list:
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


def load_model_dir(model_dir: str):
    """(config, name -> float64 array) of a model folder, read with the safetensors package."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, w


_models: dict = {}
_logits: dict = {}


def plain_logits(model_dir: str, ids) -> np.ndarray:
    key = (model_dir, tuple(ids))
    if key not in _logits:
        if model_dir not in _models:
            _models[model_dir] = load_model_dir(model_dir)
        cfg, w = _models[model_dir]
        _logits[key] = R.forward(cfg, w, list(ids))
    return _logits[key]
