"""Typed configuration of Zokepel: a decoder whose layers run a mixer and a feed-forward side by side on
two norms of the same stream, x += mixer(norm1(x)) + ff(norm2(x)), with three kinds of mixer:

  delta          gated delta rule with short convolutions, one decay per head, silu gate
  channel_delta  the same with one decay per head and key channel and a sigmoid gate, both through low-rank pairs
  parallel       an attention without rotation (q/k divided by their root mean square, a temperature on q that
                 grows with the position, a learned bias over bucketed distances) beside an RWKV-style time
                 mixing; each side's result is RMS-normed over the width and the two are averaged

The table's rows are scaled and a sinusoidal position vector is added; a stretch of the layers may run
several times in a row with the same weights (each pass with caches and state of its own), the embedding's
output being added into the stream again before every pass but the first.

config.json gives every size and constant except those that only a tensor's shape gives (the rows of the
distance-bias table, the ranks of the low-rank pairs): with the checkpoint's table at hand those are read
from the shapes; a configuration written by `to_dict` carries them as `bias_rows`, `decay_rank`, `gate_rank`.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

from .base import ArchConfig, ConfigError, require
from .spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec

MIXER_KINDS = ("delta", "channel_delta", "parallel")
# constants that the design fixes
SINUSOID_BASE = 10000.0
UNIT_VECTOR_EPS = 1e-6
SWISH_ALPHA = 1.702
MAX_POSITION = 1 << 20        # the design names no limit; positions stay exact in float32 far beyond this


def _shape(tensors, name: str) -> Optional[Tuple[int, ...]]:
    return None if tensors is None or name not in tensors else tuple(int(s) for s in tensors[name])


class ZokepelConfig(ArchConfig):
    architecture = "Zokepel"

    def __init__(self, cfg: Dict[str, Any], extra_norm2: Sequence[int] = ()):
        self.cfg = cfg
        self.extra_norm2 = tuple(extra_norm2)   # layers without a feed-forward whose checkpoint holds a second norm all the same

    def __eq__(self, other) -> bool:
        return isinstance(other, ZokepelConfig) and self.cfg == other.cfg

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], tensors: Optional[Mapping[str, Sequence[int]]] = None) -> "ZokepelConfig":
        c = copy.deepcopy(dict(cfg))
        width, vocab = int(require(c, "width")), int(require(c, "vocab"))
        for name, want in (("embed", (vocab, width)), ("head", (vocab, width))):
            got = _shape(tensors, name)
            if got is not None and got != want:
                raise ConfigError(f"config.json says {name} is {list(want)}, the checkpoint holds {list(got)}")
        float(require(c, "norm.eps"))
        float(require(c, "embedding.scale"))
        layers = require(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        extra = []
        for i, layer in enumerate(layers):
            kind = layer.get("type")
            if kind not in MIXER_KINDS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is none of {list(MIXER_KINDS)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"layer {i}: no mixer sizes")
            pre = f"l{i}.mix."
            if kind == "parallel":
                left, right = require(m, "left"), require(m, "right")
                for key in ("heads", "kv_heads", "dim", "vdim", "scale", "bias_max"):
                    require(left, key)
                if int(left["heads"]) % int(left["kv_heads"]):
                    raise ConfigError(f"layer {i}: {left['heads']} heads are not a multiple of {left['kv_heads']} kv heads")
                for key in ("heads", "dim"):
                    require(right, key)
                cls._from_shape(left, "bias_rows", _shape(tensors, pre + "left.rel"), 0, i)
                cls._from_shape(right, "decay_rank", _shape(tensors, pre + "right.w1"), 0, i)
            else:
                for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    require(m, key)
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"layer {i}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv heads")
                if int(m["conv"]) < 1:
                    raise ConfigError(f"layer {i}: a convolution of {m['conv']} taps")
                if kind == "channel_delta":
                    cls._from_shape(m, "decay_rank", _shape(tensors, pre + "a1"), 0, i)
                    cls._from_shape(m, "gate_rank", _shape(tensors, pre + "g1"), 0, i)
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not 'dense'")
                require(mlp, "ff")
                require(mlp, "limit")
            elif _shape(tensors, f"l{i}.norm2") is not None:
                extra.append(i)
        loop = c.get("loop")
        if loop is not None:
            start, stop, times = int(require(loop, "start")), int(require(loop, "stop")), int(require(loop, "times"))
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"loop {loop} does not fit {len(layers)} layers")
        return cls(c, extra)

    @staticmethod
    def _from_shape(section: dict, key: str, shape, axis: int, layer: int) -> None:
        """A size that only a tensor's shape gives: the shape wins, else the configuration's own key."""
        if shape is not None:
            section[key] = int(shape[axis])
        elif section.get(key) is None:
            raise ConfigError(f"layer {layer}: {key} is given neither by the checkpoint's tensors nor by config.json")

    def to_dict(self) -> dict:
        return copy.deepcopy(self.cfg)

    def derived(self) -> dict:
        order, again = self.run_order()
        return {"order": list(order), "embedding_added_again_before_runs": list(again)}

    # ------------------------------------------------------------------ the model it describes
    def run_order(self) -> Tuple[Tuple[int, ...], Tuple[int, ...]]:
        """(the layers in the order they run, the runs right before which the embedding's output is added again)."""
        n = len(self.cfg["layers"])
        loop = self.cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
        start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        order, again = list(range(start)), []
        for rep in range(times):
            if rep > 0 and stop > start:
                again.append(len(order))
            order += list(range(start, stop))
        return tuple(order + list(range(stop, n))), tuple(again)

    def _delta(self, i: int, kind: str, m: Mapping[str, Any], eps: float) -> MixerSpec:
        p = f"l{i}.mix."
        params = {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
                  "taps": int(m["conv"]), "norm_eps": eps, "unit_eps": UNIT_VECTOR_EPS, "q_scale": float(int(m["dim"]) ** -0.5)}
        names = {r: p + r for r in ("q", "k", "v", "b", "A_log", "norm", "dt_bias", "o")}
        names.update({"q_taps": p + "q.conv", "k_taps": p + "k.conv", "v_taps": p + "v.conv"})
        if kind == "channel_delta":
            params.update(decay="channel", decay_rank=int(m["decay_rank"]), gate="sigmoid", gate_rank=int(m["gate_rank"]))
            names.update({r: p + r for r in ("a1", "a2", "g1", "g2")})
        else:
            params.update(decay="head", gate="silu")
            names.update({"a": p + "a", "g": p + "g"})
        return MixerSpec("gated_delta", params, names)

    def _attention(self, i: int, m: Mapping[str, Any], eps: float) -> MixerSpec:
        p = f"l{i}.mix.left."
        bias = PositionSpec("distance_buckets", {"rows": int(m["bias_rows"]), "reach": int(m["bias_max"])}, {"table": p + "rel"})
        params = {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]), "v_head_dim": int(m["vdim"]),
                  "scale": float(m["scale"]), "qk_norm": "unit", "qk_norm_eps": eps, "window": None}
        temp = m.get("q_temp")
        if temp is not None:
            params["q_temperature"] = {"coef": float(require(temp, "coef")), "every": int(require(temp, "every"))}
        return MixerSpec("attention", params, {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "out_proj": p + "o"},
                         position=bias)

    def _time_mix(self, i: int, m: Mapping[str, Any], eps: float) -> MixerSpec:
        p = f"l{i}.mix.right."
        names = {r: p + r for r in ("r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o")}
        names.update({"mu_" + s: p + "mu." + s for s in "rkvgw"})
        return MixerSpec("time_mix", {"heads": int(m["heads"]), "dim": int(m["dim"]), "decay_rank": int(m["decay_rank"]),
                                      "norm_eps": eps}, names)

    def model_spec(self) -> ModelSpec:
        c = self.cfg
        width, eps = int(c["width"]), float(c["norm"]["eps"])
        layers = []
        for i, layer in enumerate(c["layers"]):
            name, kind, m = f"l{i}", layer["type"], layer["mixer"]
            parts = [("norm1", NormSpec("rms", eps, f"{name}.norm1"))]
            if kind == "parallel":
                parts += [("left", self._attention(i, m["left"], eps)), ("right", self._time_mix(i, m["right"], eps)),
                          ("left_out", NormSpec("rms", eps, f"{name}.mix.left.out")),
                          ("right_out", NormSpec("rms", eps, f"{name}.mix.right.out"))]
            else:
                parts.append(("mixer", self._delta(i, kind, m, eps)))
            mlp = layer.get("mlp")
            if mlp is not None or i in self.extra_norm2:
                parts.append(("norm2", NormSpec("rms", eps, f"{name}.norm2")))
            if mlp is not None:
                parts.append(("ffn", FeedForwardSpec(
                    "glu", {"inter": int(mlp["ff"]), "activation": "clamped_swish", "limit": float(mlp["limit"]), "alpha": SWISH_ALPHA},
                    {"gate": f"{name}.mlp.gate", "up": f"{name}.mlp.up", "down": f"{name}.mlp.down"})))
            layers.append(LayerSpec(name, "parallel_norms", parts=parts))
        order, again = self.run_order()
        return ModelSpec(
            architecture=self.architecture, hidden=width, vocab=int(c["vocab"]), layers=tuple(layers), order=order,
            embedding="embed", final_norm=NormSpec("rms", eps, "final.norm"), head="head", max_position=MAX_POSITION,
            embedding_scale=float(c["embedding"]["scale"]),
            embedding_position=PositionSpec("sinusoidal", {"base": SINUSOID_BASE}), reinject_before=again)
