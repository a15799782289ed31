"""A learned bias on attention scores by bucketed distance.

The table has B rows (one per bucket) and a column per head; a query at position i adds table[bucket(i - j), h]
to its score with the key at position j.  With D the reach of the buckets:

    bucket(n) = n                                                     for n < h,      h = B // 2
              = min(B - 1, h + floor((B - h) * log(n / h) / log(D / h)))   from h on

so near distances have a bucket each, farther ones share buckets whose width grows with the distance, and
every distance from D on has the last one.  The attention kernels get the bias as a table over the distance
itself, [D + 1, heads] (row n for distance n, the last row for everything beyond), made once when the
weights are bound; the score's scale does not multiply it.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import PositionEncoding, Runtime, register_position


def distance_buckets(rows: int, reach: int) -> List[int]:
    """bucket(n) for n = 0 .. reach (the last entry stands for every longer distance)."""
    half = rows // 2
    out = []
    for n in range(reach + 1):
        if n < half:
            out.append(n)
        elif n >= reach:
            out.append(rows - 1)
        else:
            out.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (rows - half)))))
    return out


@register_position("distance_buckets")
class DistanceBuckets(PositionEncoding):
    def __init__(self, spec, head_dim):
        super().__init__(spec, head_dim)
        self.rows, self.reach = int(spec.params["rows"]), int(spec.params["reach"])
        if self.rows < 2 or self.reach <= self.rows // 2:
            raise ValueError(f"{self.rows} distance buckets with a reach of {self.reach}")
        self.heads: Optional[int] = None

    def for_heads(self, heads: int) -> "DistanceBuckets":
        self.heads = heads
        return self

    def tensor_decls(self) -> List[TensorDecl]:
        return [TensorDecl(self.spec.tensors["table"], (self.rows, self.heads), FLOAT32, init="bias")]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        table = weights[self.spec.tensors["table"]]
        index = torch.tensor(distance_buckets(self.rows, self.reach), dtype=torch.long, device=table.device)
        self.by_distance = table[index].contiguous()            # [reach + 1, heads]

    def score_table(self, heads: int) -> torch.Tensor:
        """float32 [distances, heads]: what is added to the score at each distance (the last row beyond)."""
        assert self.by_distance.shape[1] == heads
        return self.by_distance

    def small_tensors(self):
        return [self.by_distance]
