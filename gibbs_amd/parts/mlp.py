"""Dense feed-forward without a gate: down(act(up(h))).

`activation: "poly_norm"`: act(z) = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N the division of
a token's vector of values by its root mean square (`eps` inside the root), and [a, b, c, e] a tensor of the
checkpoint (`act`).  The three mean squares are float32 sums in either precision of a run."""
from __future__ import annotations

from typing import List

from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import FeedForward, Runtime, register_feed_forward


@register_feed_forward("mlp")
class MlpFeedForward(FeedForward):
    def __init__(self, spec, hidden):
        super().__init__(spec, hidden)
        self.inter = int(spec.params["inter"])
        self.activation = spec.params.get("activation", "poly_norm")
        self.eps = float(spec.params.get("eps", 0.0))
        if self.activation != "poly_norm":
            raise ValueError(f"feed-forward activation {self.activation!r} is not implemented ('poly_norm')")

    def tensor_decls(self) -> List[TensorDecl]:
        t = self.spec.tensors
        return [TensorDecl(t["up"], (self.inter, self.hidden)), TensorDecl(t["down"], (self.hidden, self.inter)),
                TensorDecl(t["act"], (4,), FLOAT32, init="gain")]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.w_up, self.w_down, self.coef = weights[t["up"]], weights[t["down"]], weights[t["act"]]

    def matrices(self):
        return [self.w_up, self.w_down]

    def product_shapes(self):
        return [(self.inter, self.hidden), (self.hidden, self.inter)]

    def small_tensors(self):
        return [self.coef]

    def emit(self, plan) -> int:
        return plan.mlp(w_up=self.w_up, w_down=self.w_down, inter=self.inter, coef=self.coef, eps=self.eps)
