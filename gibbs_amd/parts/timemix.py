"""RWKV-style time mixing with a decayed outer-product state.

With h' the previous token's row (zeros for a sequence's first token), each of r, k, v, g, w reads its own
mix h + (h' - h) mu_s.  r, k, v = W_r, W_k, W_v of their mixes (heads x dim); gate = silu(W_g mix_g); the
decay is exp(-exp(z)) with z = w0 + W_2 tanh(W_1 mix_w), per head and key channel.  Per head, with the state M [dim,
dim] starting at zero, ' for transposed, .* along the key channels, and a bonus [dim] for the current token only:

    read = (M + (bonus .* k) v')' r;  M = decay .* M (row by row) + k v'

Each head's read-out is divided by its root mean square; the heads side by side are multiplied by a gain and the
gate, and projected by W_o.  The state M and the previous token's row live in the request's slot as
float32; the decay and the rule are float32 in both precisions of a run.  The kernels are
csrc/recurrent.hip's; the step lays them out in csrc/step_plan.hip.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..cache.needs import StateNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, register_mixer

SHIFT_STATE, RULE_STATE = "shift_row", "outer_rule"
MIXES = "rkvgw"


@register_mixer("time_mix")
class TimeMixMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.heads, self.dim, self.rank = int(p["heads"]), int(p["dim"]), int(p["decay_rank"])
        self.norm_eps = float(p["norm_eps"])
        if self.heads <= 0 or not 0 < self.dim <= 256 or self.rank <= 0:
            raise ValueError(f"time mixing with {self.heads} heads of {self.dim} (at most 256) and a decay of rank {self.rank}")

    def state_needs(self) -> Sequence[StateNeed]:
        return (StateNeed(RULE_STATE, (self.heads, self.dim, self.dim)), StateNeed(SHIFT_STATE, (self.hidden,)))

    def tensor_decls(self) -> List[TensorDecl]:
        t, W, C = self.spec.tensors, self.hidden, self.heads * self.dim
        decls = [TensorDecl(t["mu_" + s], (W,), FLOAT32, init="bias") for s in MIXES]
        decls += [TensorDecl(t[s], (C, W)) for s in ("r", "k", "v", "g")]
        decls += [TensorDecl(t["w1"], (self.rank, W)), TensorDecl(t["w2"], (C, self.rank)),
                  TensorDecl(t["w0"], (C,), FLOAT32, init="bias"), TensorDecl(t["u"], (self.heads, self.dim), FLOAT32, init="bias"),
                  TensorDecl(t["norm"], (C,), FLOAT32, init="gain"), TensorDecl(t["o"], (W, C))]
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.mu = torch.stack([weights[t["mu_" + s]] for s in MIXES], dim=0).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (weights[t[s]] for s in ("r", "k", "v", "g"))
        self.w_1, self.w_2, self.w_out = weights[t["w1"]], weights[t["w2"]], weights[t["o"]]
        self.w0, self.bonus, self.gain = weights[t["w0"]], weights[t["u"]].contiguous(), weights[t["norm"]]

    def matrices(self):
        return [self.w_r, self.w_k, self.w_v, self.w_g, self.w_1, self.w_2, self.w_out]

    def product_shapes(self):
        C = self.heads * self.dim
        return [(C, self.hidden)] * 4 + [(self.rank, self.hidden), (C, self.rank), (self.hidden, C)]

    def small_tensors(self):
        return [self.mu, self.w0, self.bonus, self.gain]

    def state_bytes(self) -> int:
        return 2 * 4 * (self.heads * self.dim * self.dim + self.hidden)

    def emit(self, plan, cache) -> int:
        return plan.time_mix(self, shift_state=cache.states[SHIFT_STATE], rule_state=cache.states[RULE_STATE])
