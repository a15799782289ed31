"""Gated delta-rule mixer with short convolutions.

q = W_q h, k = W_k h (kv_heads x dim), v = W_v h (heads x vdim); each passes a short causal convolution
per channel (taps [channels, K], the last one the current token's, zeros before a sequence's start) and
silu; every head of q and k becomes a unit vector x / sqrt(sum x^2 + unit_eps), q times q_scale.  Per head
(head h reads q/k head h // (heads / kv_heads)), with the state M [dim, vdim] starting at zero and ' for transposed:

    M = decay * M;  w = beta * (v - M' k);  M = M + k w';  read = M' q

beta = sigmoid(W_b h); the decay, exp(-rate softplus(a + dt_bias)) with rate = exp(A_log), is one per head (`decay:
"head"`, a = W_a h) or one per head and key channel, acting on the rows of M (`decay: "channel"`, a =
W_a2 (W_a1 h), a low-rank pair).  Each head's read-out is divided by its root mean square, multiplied by a gain
[vdim] shared by the heads and by a gate, silu(W_g h) (`gate: "silu"`) or sigmoid(W_g2 (W_g1 h)) (`gate:
"sigmoid"`), and projected by W_o.  The state M and the convolutions' last K - 1 inputs live in the
request's slot as float32; decays, beta, the unit vectors and the rule itself are float32 in both
precisions of a run.  The kernels are csrc/recurrent.hip's; the step lays them out in csrc/step_plan.hip.
"""
from __future__ import annotations

import ctypes
from typing import List, Sequence

import torch

from ..cache.needs import StateNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, register_mixer

CONV_STATE, RULE_STATE = "delta_conv", "delta_rule"


def _pad8(n: int) -> int:
    return -(-n // 8) * 8


@register_mixer("gated_delta")
class GatedDeltaMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.heads, self.kv_heads, self.dim, self.vdim = int(p["heads"]), int(p["kv_heads"]), int(p["dim"]), int(p["vdim"])
        self.taps = int(p["taps"])
        self.decay, self.gate = p.get("decay", "head"), p.get("gate", "silu")
        self.decay_rank, self.gate_rank = int(p.get("decay_rank", 0)), int(p.get("gate_rank", 0))
        self.norm_eps, self.unit_eps = float(p["norm_eps"]), float(p.get("unit_eps", 1e-6))
        self.q_scale = float(p.get("q_scale", self.dim ** -0.5))
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv heads")
        if self.decay not in ("head", "channel") or self.gate not in ("silu", "sigmoid"):
            raise ValueError(f"decay {self.decay!r} / gate {self.gate!r}: 'head' or 'channel', 'silu' or 'sigmoid'")
        if (self.decay == "channel" and self.decay_rank <= 0) or (self.gate == "sigmoid" and self.gate_rank <= 0):
            raise ValueError("a low-rank pair needs its rank")
        if self.taps < 1 or self.dim > 256:
            raise ValueError(f"taps {self.taps} must be at least 1 and the key size {self.dim} at most 256")
        self.conv_channels = 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def state_needs(self) -> Sequence[StateNeed]:
        needs = [StateNeed(RULE_STATE, (self.heads, self.dim, self.vdim))]
        if self.taps > 1:
            needs.append(StateNeed(CONV_STATE, (self.taps - 1, self.conv_channels)))
        return tuple(needs)

    def tensor_decls(self) -> List[TensorDecl]:
        t, W = self.spec.tensors, self.hidden
        qk, hv = self.kv_heads * self.dim, self.heads * self.vdim
        decls = [TensorDecl(t["q"], (qk, W)), TensorDecl(t["k"], (qk, W)), TensorDecl(t["v"], (hv, W)),
                 TensorDecl(t["q_taps"], (qk, self.taps), FLOAT32), TensorDecl(t["k_taps"], (qk, self.taps), FLOAT32),
                 TensorDecl(t["v_taps"], (hv, self.taps), FLOAT32),
                 TensorDecl(t["b"], (self.heads, W)), TensorDecl(t["A_log"], (self.heads,), FLOAT32, init="bias"),
                 TensorDecl(t["norm"], (self.vdim,), FLOAT32, init="gain"), TensorDecl(t["o"], (W, hv))]
        if self.decay == "channel":
            decls += [TensorDecl(t["a1"], (self.decay_rank, W)), TensorDecl(t["a2"], (self.heads * self.dim, self.decay_rank)),
                      TensorDecl(t["dt_bias"], (self.heads * self.dim,), FLOAT32, init="bias")]
        else:
            decls += [TensorDecl(t["a"], (self.heads, W)), TensorDecl(t["dt_bias"], (self.heads,), FLOAT32, init="bias")]
        if self.gate == "sigmoid":
            decls += [TensorDecl(t["g1"], (self.gate_rank, W)), TensorDecl(t["g2"], (hv, self.gate_rank))]
        else:
            decls.append(TensorDecl(t["g"], (hv, W)))
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        # one product for everything that reads the normed rows: [q; k; v | b | a or a1 | g or g1], every segment
        # starting at a multiple of 8 rows (zero rows between), so that slices of the result stay 16-byte aligned
        segments = [torch.cat([weights[t["q"]], weights[t["k"]], weights[t["v"]]], dim=0), weights[t["b"]],
                    weights[t["a1"] if self.decay == "channel" else t["a"]], weights[t["g1"] if self.gate == "sigmoid" else t["g"]]]
        rows, offsets = [], []
        for seg in segments:
            offsets.append(sum(r.shape[0] for r in rows))
            rows.append(seg)
            pad = _pad8(seg.shape[0]) - seg.shape[0]
            if pad:
                rows.append(torch.zeros((pad, seg.shape[1]), dtype=seg.dtype, device=seg.device))
        self.w_in = torch.cat(rows, dim=0).contiguous()
        _, self.off_b, self.off_a, self.off_g = offsets
        self.w_a2 = weights[t["a2"]] if self.decay == "channel" else None
        self.w_g2 = weights[t["g2"]] if self.gate == "sigmoid" else None
        self.w_out = weights[t["o"]]
        self.conv_taps = torch.cat([weights[t["q_taps"]], weights[t["k_taps"]], weights[t["v_taps"]]], dim=0).contiguous()
        self.a_log, self.dt_bias, self.gain = weights[t["A_log"]], weights[t["dt_bias"]], weights[t["norm"]]

    def matrices(self):
        return [m for m in (self.w_in, self.w_a2, self.w_g2, self.w_out) if m is not None]

    def product_shapes(self):
        qk, hv = self.kv_heads * self.dim, self.heads * self.vdim
        shapes = [(2 * qk + hv + self.heads, self.hidden), (self.hidden, hv)]
        shapes += [(self.decay_rank, self.hidden), (self.heads * self.dim, self.decay_rank)] if self.decay == "channel" else [(self.heads, self.hidden)]
        shapes += [(self.gate_rank, self.hidden), (hv, self.gate_rank)] if self.gate == "sigmoid" else [(hv, self.hidden)]
        return shapes

    def small_tensors(self):
        return [self.conv_taps, self.a_log, self.dt_bias, self.gain]

    def state_bytes(self) -> int:
        """Bytes of state that a decoded token reads and writes."""
        return 2 * 4 * (self.heads * self.dim * self.vdim + (self.taps - 1) * self.conv_channels)

    def emit(self, plan, cache) -> int:
        rule = cache.states[RULE_STATE]
        conv = cache.states[CONV_STATE] if self.taps > 1 else rule      # (one tap: no inputs are kept)
        return plan.gated_delta(self, conv_state=conv, rule_state=rule)
