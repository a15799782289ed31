"""Typed configuration of Rukosun: a decoder of latent-attention layers over several residual streams.

  embedding   the token table's row, plus the row of a table over hashed pairs (previous token, token), plus the
              row of a learned table over positions
  layer       pre-norm sublayers, x += mixer(norm1(x)) and x += ff(norm2(x)), with layer norms (gain and bias); with
              `streams` the model keeps that many copies of x and every sublayer reads and writes them through a
              hyper-connection: it reads u = sum_s in[s] x_s and writes x_t <- sum_s mix[s, t] x_s + out[t] y
  mixers      `latent_attention`: queries through a normed latent, keys and values from a small normed latent and one
              rotated key part that all heads share, interleaved rotation, a window, a sink in the softmax, a sigmoid
              gate on the heads' outputs;  `latent_attention_2`: direct queries, rotate-half pairing, a plain softmax
              over the window, no gate
  feed-forward  down(act(up h)) with act(z) = a N(z) + b N(z^2) + c N(z^3) + e, N the division by the root mean square
  loop        a stretch of the layers may run several times in a row with the same weights, every pass with a cache
              of its own

config.json gives every size and constant; what the design fixes (which mixer has the sink, the gate, which pairing)
is written here.  A layer without a feed-forward whose checkpoint nevertheless holds a second norm or connection
has those tensors declared, so that loading accounts for every tensor, and never reads them.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

from .base import ArchConfig, ConfigError, require
from .spec import (ConnectionSpec, EmbeddingTablesSpec, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec,
                   PositionSpec)

MIXER_KINDS = ("latent_attention", "latent_attention_2")
# what the design fixes per kind of mixer: (queries through a latent, pairing of the rotation, sink, output gate)
MIXER_TRAITS = {"latent_attention": (True, "interleaved", True, True),
                "latent_attention_2": (False, "half_split", False, False)}


def _has(tensors, name: str) -> bool:
    return tensors is not None and name in tensors


class RukosunConfig(ArchConfig):
    architecture = "Rukosun"

    def __init__(self, cfg: Dict[str, Any], unread: Sequence[Tuple[str, Tuple[int, ...]]] = ()):
        self.cfg = cfg
        self.unread = tuple(unread)     # (name, shape) of checkpoint tensors of sublayers that a layer does not have

    def __eq__(self, other) -> bool:
        return isinstance(other, RukosunConfig) and self.cfg == other.cfg

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], tensors: Optional[Mapping[str, Sequence[int]]] = None) -> "RukosunConfig":
        c = copy.deepcopy(dict(cfg))
        width, vocab = int(require(c, "width")), int(require(c, "vocab"))
        for name, want in (("embed", (vocab, width)), ("head", (vocab, width))):
            if _has(tensors, name) and tuple(int(s) for s in tensors[name]) != want:
                raise ConfigError(f"config.json says {name} is {list(want)}, the checkpoint holds {list(tensors[name])}")
        float(require(c, "norm.eps"))
        int(require(c, "max_positions"))
        big = (c.get("embedding") or {}).get("bigram")
        if big is not None:
            for key in ("buckets", "mul_prev", "mul_cur"):
                int(require(big, key))
            if int(big["buckets"]) <= 0:
                raise ConfigError("embedding.bigram.buckets must be positive")
        streams = c.get("streams")
        if streams is not None and not 1 <= int(streams) <= 8:
            raise ConfigError(f"{streams} residual streams (1 to 8)")
        layers = require(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        unread = []
        for i, layer in enumerate(layers):
            kind = layer.get("type")
            if kind not in MIXER_KINDS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is none of {list(MIXER_KINDS)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"layer {i}: no mixer sizes")
            for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"):
                require(m, key)
            if MIXER_TRAITS[kind][0]:
                require(m, "q_rank")
            if int(m["rot_dim"]) > 0:
                require(m, "rot.base")
                dims = int((m.get("rot") or {}).get("dims", m["rot_dim"]))
                if dims % 2 or not 0 <= dims <= int(m["rot_dim"]):
                    raise ConfigError(f"layer {i}: {dims} rotated dimensions of a part of {m['rot_dim']}")
            size = (m.get("mask") or {}).get("size")
            if size is not None and int(size) <= 0:
                raise ConfigError(f"layer {i}: a window of {size}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not 'dense'")
                require(mlp, "ff")
            elif tensors is not None:
                unread += [(n, tuple(int(s) for s in tensors[n])) for n in sorted(tensors)
                           if n.startswith((f"l{i}.norm2", f"l{i}.hc2."))]
        loop = c.get("loop")
        if loop is not None:
            start, stop, times = int(require(loop, "start")), int(require(loop, "stop")), int(require(loop, "times"))
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"loop {loop} does not fit {len(layers)} layers")
        return cls(c, unread)

    def to_dict(self) -> dict:
        return copy.deepcopy(self.cfg)

    def derived(self) -> dict:
        return {"order": list(self.run_order())}

    # ------------------------------------------------------------------ the model it describes
    def run_order(self) -> Tuple[int, ...]:
        n = len(self.cfg["layers"])
        loop = self.cfg.get("loop")
        if not loop:
            return tuple(range(n))
        start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        return tuple(list(range(start)) + list(range(start, stop)) * times + list(range(stop, n)))

    def _mixer(self, i: int, kind: str, m: Mapping[str, Any], eps: float) -> MixerSpec:
        p = f"l{i}.mix."
        latent_q, pairing, sink, gate = MIXER_TRAITS[kind]
        rot_dim = int(m["rot_dim"])
        params = {"heads": int(m["heads"]), "dim": int(m["dim"]), "rot_dim": rot_dim, "vdim": int(m["vdim"]),
                  "kv_rank": int(m["kv_rank"]), "q_rank": int(m["q_rank"]) if latent_q else None, "scale": float(m["scale"]),
                  "window": (m.get("mask") or {}).get("size"), "sink": sink, "gate": gate, "norm_eps": eps}
        names = {"dkv": p + "dkv", "dkv_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv", "o": p + "o"}
        names.update({"dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq"} if latent_q else {"q": p + "q"})
        if sink:
            names["sink"] = p + "sink"
        if gate:
            names["g"] = p + "g"
        position = None
        if rot_dim > 0:
            rot = m["rot"]
            position = PositionSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot.get("dims", rot_dim)),
                                             "variant": pairing, "precision": "f64"})
        return MixerSpec("latent_attention", params, names, position=position)

    def model_spec(self) -> ModelSpec:
        c = self.cfg
        width, eps = int(c["width"]), float(c["norm"]["eps"])
        streams = c.get("streams")
        layers = []
        for i, layer in enumerate(c["layers"]):
            name = f"l{i}"
            parts = [("norm1", NormSpec("layer", eps, f"{name}.norm1", f"{name}.norm1.b")),
                     ("mixer", self._mixer(i, layer["type"], layer["mixer"], eps))]
            if streams is not None:
                parts.append(("connection1", ConnectionSpec("hyper", int(streams), {r: f"{name}.hc1.{r}" for r in ("in", "mix", "out")})))
            mlp = layer.get("mlp")
            if mlp is not None:
                parts += [("norm2", NormSpec("layer", eps, f"{name}.norm2", f"{name}.norm2.b")),
                          ("ffn", FeedForwardSpec("mlp", {"inter": int(mlp["ff"]), "activation": "poly_norm", "eps": eps},
                                                  {"up": f"{name}.mlp.up", "down": f"{name}.mlp.down", "act": f"{name}.mlp.act"}))]
                if streams is not None:
                    parts.append(("connection2", ConnectionSpec("hyper", int(streams), {r: f"{name}.hc2.{r}" for r in ("in", "mix", "out")})))
            layers.append(LayerSpec(name, "sublayers", parts=parts))
        big = (c.get("embedding") or {}).get("bigram")
        tables = EmbeddingTablesSpec(
            pair="bigram" if big is not None else None, buckets=int(big["buckets"]) if big is not None else 0,
            mul_prev=int(big["mul_prev"]) if big is not None else 0, mul_cur=int(big["mul_cur"]) if big is not None else 0,
            position="pos", positions=int(c["max_positions"]))
        return ModelSpec(
            architecture=self.architecture, hidden=width, vocab=int(c["vocab"]), layers=tuple(layers), order=self.run_order(),
            embedding="embed", final_norm=NormSpec("layer", eps, "final.norm", "final.norm.b"), head="head",
            max_position=int(c["max_positions"]), embedding_tables=tables, streams=1 if streams is None else int(streams),
            unread_tensors=self.unread)
