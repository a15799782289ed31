"""Arrangements of a layer's parts.

`pre_norm` is LFM2's (arch/families/lfm2.json5:77-88):
    x = x + mixer(norm(x));   x = x + ffn(norm(x))
The residual stream x is float32.  In the native step each residual add is fused into the norm that
follows it, so a half of the block hands its delta on instead of adding it.

In bfloat16 the block folds each norm's gain into the matrices that read the normed rows (the
reference's graph passes fold norm gains into weights too, src/graph/passes/mod.rs).
A step of single decoded tokens (up to `Runtime.fused_decode_rows` rows) then takes the parts' fused
decode kernels: the product itself computes 1/rms of its input rows, and the last product of each
half adds its result into the stream, so a half of a layer is two or three kernels.  Whether a step
does is decided where the step runs (csrc/step_plan.hip), per half, from the step's shape, the
norm (its gain folded) and the part (sizes that its fused kernels take).
"""
from __future__ import annotations

import torch

from .base import Block, Runtime, register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock(Block):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        missing = [r for r in spec.PRE_NORM_ROLES if r not in self.named]
        if missing:
            raise ValueError(f"a pre-norm block needs the parts {list(spec.PRE_NORM_ROLES)}; layer {spec.name!r} lacks {missing}")

    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        self._fold(self.mixer_norm, self.mixer)
        self._fold(self.ffn_norm, self.ffn)
        if self.rt.act_dtype == torch.bfloat16:
            self.mixer.pack_matrices()
            self.ffn.pack_matrices()

    def _fold(self, norm, part) -> bool:
        if self.rt.act_dtype != torch.bfloat16 or not self.rt.fold_gains:
            return False
        if not (hasattr(norm, "fold_gain") and hasattr(part, "fold_input_gain")):
            return False
        part.fold_input_gain(norm.fold_gain())
        return True

    def emit(self, plan, caches) -> None:
        plan.half(self.mixer_norm.emit(plan), self.mixer.emit(plan, caches["mixer"]))
        plan.half(self.ffn_norm.emit(plan), self.ffn.emit(plan))


@register_arrangement("parallel_norms")
class ParallelNormsBlock(Block):
    """Mixer and feed-forward side by side, each on a norm of its own of the same stream:

        x = x + mixer(norm1(x)) + ffn(norm2(x))

    Roles: `norm1`, then either `mixer`, or a pair of mixers `left` and `right` that read the same normed rows,
    each result normed over the width by `left_out` / `right_out` and the two averaged; `norm2` and `ffn` may
    be missing (a layer without a feed-forward).  The average's half is multiplied into the two out-norms'
    gains when the weights are bound (exact: a power of two).

    The feed-forward is laid down as a half of its own, x += ffn(norm2(x)), between the mixer's norm and the
    mixer itself: the mixer's rows were normed before that half touched the stream, so both still read the
    same x, and in bfloat16 the half takes the fused few-row kernels (norm2's gain folded into the gate and up
    matrices) as a pre-norm block's does.  The mixers run norm, body and add operations."""

    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        self.pair = "left" in self.named
        want = ["norm1"] + (["left", "right", "left_out", "right_out"] if self.pair else ["mixer"])
        want += ["norm2"] if "ffn" in self.named else []
        missing = [r for r in want if r not in self.named]
        if missing:
            raise ValueError(f"layer {spec.name!r} lacks the parts {missing}")

    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        if self.pair:
            for norm in (self.left_out, self.right_out):
                norm.gain = norm.gain * 0.5
        if "ffn" in self.named and rt.act_dtype == torch.bfloat16:
            if rt.fold_gains and hasattr(self.norm2, "fold_gain") and hasattr(self.ffn, "fold_input_gain"):
                self.ffn.fold_input_gain(self.norm2.fold_gain())
            self.ffn.pack_matrices()

    def emit(self, plan, caches) -> None:
        h = plan.normed(self.norm1.emit(plan))
        if "ffn" in self.named:
            plan.half(self.norm2.emit(plan), self.ffn.emit(plan))
        if self.pair:
            left = plan.apply(self.left.emit(plan, caches["left"]), h)
            right = plan.apply(self.right.emit(plan, caches["right"]), h)
            plan.drop(h)
            plan.add_normed(self.left_out.emit(plan), left)      # (normed and added in float32, in one pass each)
            plan.add_normed(self.right_out.emit(plan), right)
        else:
            delta = plan.apply(self.mixer.emit(plan, caches["mixer"]), h)
            plan.drop(h)
            plan.add(delta)
