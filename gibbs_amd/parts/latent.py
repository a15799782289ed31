"""Latent attention: keys and values of all heads come from one small latent per token.

With h the mixer's input, H heads, per head `dim` unrotated and `rot_dim` rotated query/key entries, values of size
`vdim`, a latent of size `kv_rank`:

    queries   q = W_uq rms_norm(W_dq h) (`q_rank` given: through a latent of their own), or q = W_q h; a head of q is
              [dim unrotated | rot_dim rotated]
    latent    W_dkv h has kv_rank + rot_dim rows: c = rms_norm(first kv_rank), k_r = the last rot_dim (not normed), one
              rotated key part for all heads
    per head  key [W_uk,i c | rotate(k_r)], value W_uv,i c, score = (q_i . W_uk,i c + rotate(q_r,i) . rotate(k_r)) * scale
    softmax   over the last `window` positions (None: all), optionally with a sink: a learned number per head whose
              exponential joins the denominator, with no key and no value
    output    the heads' results, optionally times sigmoid(W_g h) (`gate`), through W_o

Only [c | rotate(k_r)] is cached: one row of kv_rank + rot_dim values per token and layer, whatever the number of
heads.  The kernels work on those rows directly: since q_i . W_uk,i c = (W_uk,i' q_i) . c, every head's query becomes
[W_uk,i' q_i | rotate(q_r,i)] and all heads attend over the same cached rows (one kv head whose values are the rows
themselves); the weighted sum of latents then passes W_uv,i.  Norms, angles, scores and the softmax are float32.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..cache.needs import CacheNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, build_position, register_mixer


def _pad8(n: int) -> int:
    return -(-n // 8) * 8


@register_mixer("latent_attention")
class LatentAttentionMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.heads, self.dim, self.rot_dim, self.vdim = int(p["heads"]), int(p["dim"]), int(p["rot_dim"]), int(p["vdim"])
        self.kv_rank = int(p["kv_rank"])
        self.q_rank = int(p["q_rank"]) if p.get("q_rank") else 0
        self.scale = float(p["scale"])
        self.window = None if p.get("window") is None else int(p["window"])
        self.sink, self.gate = bool(p.get("sink", False)), bool(p.get("gate", False))
        self.norm_eps = float(p["norm_eps"])
        if self.window is not None and self.window <= 0:
            raise ValueError(f"attention window {self.window} must be positive")
        if min(self.heads, self.dim, self.vdim, self.kv_rank) <= 0 or self.rot_dim < 0:
            raise ValueError("latent attention: heads, dim, vdim and kv_rank must be positive")
        if self.kv_rank + self.rot_dim > 512:
            raise ValueError(f"a cached row of {self.kv_rank + self.rot_dim} values is more than the attention kernels take (512)")
        self.position = build_position(spec.position, self.rot_dim) if self.rot_dim > 0 else None

    # ------------------------------------------------------------------ what it asks for
    def cache_need(self) -> Optional[CacheNeed]:
        # one "kv head" whose keys are the cached rows; the values are read from the same rows (no pages of their own)
        return CacheNeed(1, self.kv_rank + self.rot_dim, self.window, 0)

    def attention_flops(self, keys: float) -> float:
        return 2.0 * keys * self.heads * (2 * self.kv_rank + self.rot_dim)

    def tensor_decls(self) -> List[TensorDecl]:
        t, W, H = self.spec.tensors, self.hidden, self.heads
        qk = H * (self.dim + self.rot_dim)
        decls = [TensorDecl(t["dkv"], (self.kv_rank + self.rot_dim, W)), TensorDecl(t["dkv_norm"], (self.kv_rank,), FLOAT32, init="gain"),
                 TensorDecl(t["uk"], (H * self.dim, self.kv_rank)), TensorDecl(t["uv"], (H * self.vdim, self.kv_rank)),
                 TensorDecl(t["o"], (W, H * self.vdim))]
        if self.q_rank:
            decls += [TensorDecl(t["dq"], (self.q_rank, W)), TensorDecl(t["dq_norm"], (self.q_rank,), FLOAT32, init="gain"),
                      TensorDecl(t["uq"], (qk, self.q_rank))]
        else:
            decls.append(TensorDecl(t["q"], (qk, W)))
        if self.sink:
            decls.append(TensorDecl(t["sink"], (H,), FLOAT32, init="bias"))
        if self.gate:
            decls.append(TensorDecl(t["g"], (H * self.vdim, W)))
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        # one product for everything that reads the normed rows: [W_dq or W_q | W_dkv | W_g], every segment starting at
        # a multiple of 8 rows (zero rows between), so that slices of the result stay 16-byte aligned
        segments = [weights[t["dq"]] if self.q_rank else weights[t["q"]], weights[t["dkv"]]]
        if self.gate:
            segments.append(weights[t["g"]])
        rows, offsets = [], []
        for seg in segments:
            offsets.append(sum(r.shape[0] for r in rows))
            rows.append(seg)
            pad = _pad8(seg.shape[0]) - seg.shape[0]
            if pad:
                rows.append(torch.zeros((pad, seg.shape[1]), dtype=seg.dtype, device=seg.device))
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.off_kv = offsets[1]
        self.off_g = offsets[2] if self.gate else -1
        self.w_uq = weights[t["uq"]] if self.q_rank else None
        self.q_gain = weights[t["dq_norm"]] if self.q_rank else None
        if self.q_rank and rt.act_dtype == torch.bfloat16 and rt.fold_gains:
            # the queries' latent is read by W_uq alone: its norm's gain goes into that matrix's columns (as the layer
            # norms' gains of the other models do), and steps of few rows take the product that norms its rows itself
            self.w_uq = (self.w_uq.float() * self.q_gain[None, :]).to(self.w_uq.dtype)
            self.q_gain = None
        self.kv_gain = weights[t["dkv_norm"]]
        # every head's key up-projection transposed, [heads, kv_rank, dim]: the product that takes a head's unrotated
        # query part to the latent's size reads it as a matrix [out, in]
        self.w_uk_t = weights[t["uk"]].view(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = weights[t["uv"]].contiguous()
        self.w_out = weights[t["o"]]
        self.sinks = weights[t["sink"]] if self.sink else None
        self.rot = None
        if self.position is not None:
            self.position.bind(weights, rt)
            self.rot = self.position.rotation()
            if self.rot is None:
                raise ValueError("latent attention takes a rotation as its position encoding")

    def matrices(self):
        return [m for m in (self.w_in, self.w_uq, self.w_uk_t, self.w_uv, self.w_out) if m is not None]

    def product_shapes(self):
        H, W = self.heads, self.hidden
        qk = H * (self.dim + self.rot_dim)
        shapes = [((self.q_rank or qk) + self.kv_rank + self.rot_dim + (H * self.vdim if self.gate else 0), W), (W, H * self.vdim)]
        if self.q_rank:
            shapes.append((qk, self.q_rank))
        shapes += [(H * self.kv_rank, self.dim), (H * self.vdim, self.kv_rank)]     # per head: flops of [kv_rank, dim] and [vdim, kv_rank]
        return shapes

    def small_tensors(self):
        own = [t for t in (self.q_gain, self.kv_gain, self.sinks) if t is not None]
        return own + ([] if self.position is None else list(self.position.small_tensors()))

    def emit(self, plan, cache) -> int:
        if cache.kpages is None or cache.kpages.shape[-1] != self.kv_rank + self.rot_dim or cache.kpages.shape[1] != 1:
            raise ValueError("the latent attention's pages do not have its row size")
        return plan.latent_attention(self, pages=cache.kpages, group=cache.group)
