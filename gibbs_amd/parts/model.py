"""A decoder put together from a `ModelSpec`: token table, blocks in the spec's run order, final
norm and head (arch/families/lfm2.json5:66-95,
arch/lib/transformer.json5:170-198).

The model owns structure and weights; its step is the native plan that its blocks lay down
(parts/native.py).  Only the rows whose logits are wanted go through the final norm and the head:
the gather comes before the norm, as in the reference's `last_row` (transformer.json5:177-192).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from .. import ops
from ..cache.needs import CacheNeed, StateNeed
from ..config.spec import ModelSpec
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Block, Part, Runtime, build_block, build_norm


class DecoderModel(Part):
    PREV_TOKEN = "previous_token"      # state the model itself keeps per request: its last token (for a table over token pairs)

    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.blocks: List[Block] = [build_block(ls, spec.hidden, i) for i, ls in enumerate(spec.layers)]
        self.final_norm = build_norm(spec.final_norm, spec.hidden)
        if any(not 0 < r < len(spec.order) for r in spec.reinject_before):
            raise ValueError(f"the embedding's output is added again before runs {list(spec.reinject_before)}; the order has {len(spec.order)}")
        for i in spec.order:
            if not 0 <= i < len(self.blocks):
                raise ValueError(f"layer order names layer {i}; the model has {len(self.blocks)}")
        for i, b in enumerate(self.blocks):
            for mixer in b.mixers().values():
                src = mixer.kv_source()
                if src is None:
                    continue
                if not 0 <= src < len(self.blocks) or self._cache_owner_role(src) is None:
                    raise ValueError(f"layer {i} reads the cache of layer {src}, which owns none")
                first_use = spec.order.index(i) if i in spec.order else -1
                if first_use >= 0 and src not in spec.order[:first_use]:
                    raise ValueError(f"layer {i} runs before layer {src}, whose cache it reads")

    def _cache_owner_role(self, layer: int) -> Optional[str]:
        """The role of the first mixer of `layer` that owns cache pages."""
        return next((role for role, m in self.blocks[layer].mixers().items() if m.cache_need() is not None), None)

    # ------------------------------------------------------------------ what the model asks for
    def tensor_decls(self) -> List[TensorDecl]:
        s = self.spec
        decls = [TensorDecl(s.embedding, (s.vocab, s.hidden))]
        decls += self.final_norm.tensor_decls()
        for b in self.blocks:
            decls += b.tensor_decls()
        if s.head is not None:
            decls.append(TensorDecl(s.head, (s.vocab, s.hidden)))
        tables = s.embedding_tables
        if tables is not None and tables.pair is not None:
            decls.append(TensorDecl(tables.pair, (tables.buckets + 1, s.hidden)))
        if tables is not None and tables.position is not None:
            decls.append(TensorDecl(tables.position, (tables.positions, s.hidden)))
        decls += [TensorDecl(name, tuple(shape), FLOAT32 if len(shape) <= 2 else "compute") for name, shape in s.unread_tensors]
        return decls

    def model_state_needs(self) -> Sequence[StateNeed]:
        """Per-request state of fixed size that the model itself keeps, beside its mixers'."""
        tables = self.spec.embedding_tables
        if tables is not None and tables.pair is not None:
            return (StateNeed(self.PREV_TOKEN, (), "int32"),)
        return ()

    # Caches belong to the mixers of runs (entries of the run order), not to layers: a layer that the
    # order names twice shares its weights between both runs, but each run caches its own keys,
    # values and state.  `cache_owners` lists them, (run, role) in the order they run; what the cache
    # manager calls a layer is an entry of this list.
    def cache_owners(self) -> List[Tuple[int, str]]:
        return [(run, role) for run, i in enumerate(self.spec.order) for role in self.blocks[i].mixers()]

    def _mixer(self, owner: Tuple[int, str]):
        return self.blocks[self.spec.order[owner[0]]].mixers()[owner[1]]

    # What the cache manager is asked for: one entry per cache owner and, when the model itself keeps state per
    # request, one more entry behind them (no pages, the model's states): entry `model_state_owner()`.
    def cache_needs(self) -> List[Optional[CacheNeed]]:
        own = [None] if self.model_state_needs() else []
        return [self._mixer(o).cache_need() for o in self.cache_owners()] + own

    def state_needs(self) -> List[Sequence[StateNeed]]:
        own = [tuple(self.model_state_needs())] if self.model_state_needs() else []
        return [tuple(self._mixer(o).state_needs()) for o in self.cache_owners()] + own

    def model_state_owner(self) -> Optional[int]:
        return len(self.cache_owners()) if self.model_state_needs() else None

    def kv_sources(self) -> List[Optional[int]]:
        """For each cache owner, the earlier owner whose pages it reads (the page-owning mixer of the
        latest run of the layer that its mixer names as `kv_source`), or None."""
        owners = self.cache_owners()
        out: List[Optional[int]] = []
        for run, role in owners:
            src = self._mixer((run, role)).kv_source()
            if src is None:
                out.append(None)
                continue
            src_run = max(j for j in range(run) if self.spec.order[j] == src)
            out.append(owners.index((src_run, self._cache_owner_role(src))))
        return out

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.table = weights[self.spec.embedding]
        self.head = weights[self.spec.head] if self.spec.head is not None else self.table
        self.head_packed = ops.PackedWeight(self.head) if rt.act_dtype == torch.bfloat16 else None
        self.embedding_inv_freq = None
        pos = self.spec.embedding_position
        if pos is not None and pos.kind != "none":
            if pos.kind != "sinusoidal":
                raise ValueError(f"position vector of kind {pos.kind!r} on the embedding is not implemented ('sinusoidal')")
            # frequencies f_i = base^(-2i / width), rounded to float32 once; the kernel puts sin(p f_i) at 2i and cos(p f_i) at 2i + 1
            width = self.spec.hidden
            i = torch.arange(width // 2, dtype=torch.float64)
            self.embedding_inv_freq = (float(pos.params.get("base", 10000.0)) ** (-2.0 * i / width)).to(torch.float32).to(rt.device)
        tables = self.spec.embedding_tables
        self.pair_table = weights[tables.pair] if tables is not None and tables.pair is not None else None
        self.position_table = weights[tables.position] if tables is not None and tables.position is not None else None
        streams = {b.streams() for b in self.blocks if hasattr(b, "streams")}
        if streams - {self.spec.streams} or (self.spec.streams != 1 and len(streams) != 1):
            raise ValueError(f"the model has {self.spec.streams} residual streams, its layers are connected for {sorted(streams)}")
        self.final_norm.bind(weights, rt)
        for b in self.blocks:
            b.bind(weights, rt)
