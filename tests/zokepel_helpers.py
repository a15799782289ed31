"""Small Zokepel configurations that differ in every size and option, model folders made from them through the
framework's random-weights mode, and the plain implementation's logits for them."""
from __future__ import annotations

import copy
import os

import numpy as np

from tests.plain import zokepel_plain as Z


def _left(heads, kv_heads, dim, vdim, rows, reach, scale, temp=None):
    d = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_rows": rows, "bias_max": reach, "scale": scale}
    if temp is not None:
        d["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return d


def _mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


# P: no size is a power of two or a multiple of 8 where it can be avoided; grouped heads everywhere; a layer
# without a feed-forward; the middle two layers run three times.
ZOKEPEL_P = {
    "architecture": "Zokepel", "vocab": 211, "width": 100, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
    "layers": [
        {"type": "delta", "mixer": {"heads": 6, "kv_heads": 2, "dim": 12, "vdim": 20, "conv": 3}, "mlp": _mlp(150, 2.5)},
        {"type": "parallel", "mixer": {"left": _left(6, 3, 24, 40, 12, 50, 0.3, (0.7, 9)),
                                       "right": {"heads": 5, "dim": 12, "decay_rank": 6}}, "mlp": None},
        {"type": "channel_delta", "mixer": {"heads": 3, "kv_heads": 3, "dim": 20, "vdim": 36, "conv": 5, "decay_rank": 10,
                                            "gate_rank": 7}, "mlp": _mlp(90, 0.8)},
        {"type": "delta", "mixer": {"heads": 2, "kv_heads": 1, "dim": 36, "vdim": 12, "conv": 2}, "mlp": _mlp(64, 1.5)},
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}
# Q: aligned sizes (the matrix-core products), one kv head for all query heads, values wider than keys, a
# convolution of one tap (no inputs kept), the whole model run twice, a large head of 128 key channels.
ZOKEPEL_Q = {
    "architecture": "Zokepel", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
    "layers": [
        {"type": "parallel", "mixer": {"left": _left(4, 1, 32, 64, 8, 40, 0.18, (0.25, 16)),
                                       "right": {"heads": 2, "dim": 64, "decay_rank": 16}}, "mlp": _mlp(256, 1.0)},
        {"type": "channel_delta", "mixer": {"heads": 2, "kv_heads": 1, "dim": 128, "vdim": 64, "conv": 1, "decay_rank": 8,
                                            "gate_rank": 16}, "mlp": _mlp(128, 4.0)},
        {"type": "delta", "mixer": {"heads": 4, "kv_heads": 4, "dim": 64, "vdim": 32, "conv": 4}, "mlp": _mlp(192, 1.0)},
    ],
    "loop": {"start": 0, "stop": 3, "times": 2},
}
# R: no loop at all, no temperature on the queries, odd head counts, a distance table with an odd number of rows.
ZOKEPEL_R = {
    "architecture": "Zokepel", "vocab": 97, "width": 72, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
    "layers": [
        {"type": "channel_delta", "mixer": {"heads": 5, "kv_heads": 5, "dim": 8, "vdim": 8, "conv": 2, "decay_rank": 4,
                                            "gate_rank": 4}, "mlp": _mlp(40, 1.0)},
        {"type": "parallel", "mixer": {"left": _left(3, 3, 16, 16, 9, 30, 0.25), "right": {"heads": 3, "dim": 24, "decay_rank": 5}},
         "mlp": _mlp(100, 3.0)},
    ],
}
# S: heads of 64 in groups of four with keys and values of one size (in bfloat16 the matrix-core attention kernels, with
# the distance bias), a table whose reach is shorter than the sequences, delta-rule heads of 128 key channels.
ZOKEPEL_S = {
    "architecture": "Zokepel", "vocab": 512, "width": 256, "norm": {"eps": 1e-6}, "embedding": {"scale": 2.0},
    "layers": [
        {"type": "parallel", "mixer": {"left": _left(8, 2, 64, 64, 16, 100, 0.125, (0.5, 64)),
                                       "right": {"heads": 4, "dim": 64, "decay_rank": 32}}, "mlp": _mlp(512, 7.0)},
        {"type": "delta", "mixer": {"heads": 4, "kv_heads": 2, "dim": 128, "vdim": 64, "conv": 4}, "mlp": _mlp(512, 7.0)},
        {"type": "parallel", "mixer": {"left": _left(4, 4, 32, 32, 10, 64, 0.2, (0.3, 32)),
                                       "right": {"heads": 8, "dim": 32, "decay_rank": 8}}, "mlp": None},
    ],
    "loop": {"start": 0, "stop": 2, "times": 2},
}
MODELS = {"P": ZOKEPEL_P, "Q": ZOKEPEL_Q, "R": ZOKEPEL_R, "S": ZOKEPEL_S}


def single_layer(kind: str) -> dict:
    """A model of one layer of one mixer kind and no feed-forward: the mechanism alone between embedding and head."""
    layer = {"delta": ZOKEPEL_P["layers"][0], "parallel": ZOKEPEL_P["layers"][1], "channel_delta": ZOKEPEL_P["layers"][2]}[kind]
    layer = dict(copy.deepcopy(layer), mlp=None)
    return {"architecture": "Zokepel", "vocab": 131, "width": 100, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0}, "layers": [layer]}


def make_model_dir(folder: str, cfg: dict, name: str, seed: int = 0, std: float = 0.1, bias_std: float = 0.5,
                   gain_std: float = 0.3) -> str:
    """Writes a model of configuration `cfg` through the framework's random-weights mode: matrices in bfloat16, so
    that both precisions of the engine and the plain implementation start from the same values; biases (distance
    table, decay offsets, shift weights, bonus) spread widely so that leaving one out shows."""
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    config = config_from_dict(cfg)
    decls = DecoderModel(config.model_spec()).tensor_decls()
    path = os.path.join(folder, f"zokepel_{name}_{seed}")
    write_random_model(path, config, decls, seed=seed, dtype="bfloat16", std=std, gain_std=gain_std, bias_std=bias_std)
    return path


def tokens(seed: int, n: int, vocab: int) -> list:
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


_models: dict = {}
_logits: dict = {}


def plain_logits(model_dir: str, ids) -> np.ndarray:
    key = (model_dir, tuple(ids))
    if key not in _logits:
        if model_dir not in _models:
            _models[model_dir] = Z.load_model_dir(model_dir)
        weights, cfg = _models[model_dir]
        _logits[key] = Z.forward(weights, cfg, list(ids))
    return _logits[key]
