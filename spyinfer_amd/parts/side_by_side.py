"""Two token mixers side by side on one input: each result is divided by its root mean square over the model width and
multiplied by a weight of its own, and the mixer's result is half their sum.  Each of the two keeps what it needs per
request (pages, a state slot) under a cache of its own."""
from __future__ import annotations

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Mixer


class SideBySide(Mixer):
    def __init__(self, hidden_size: int, left: Mixer, right: Mixer, norm_eps: float, names=("left", "right"), out_suffix: str = ".out"):
        self.hidden_size, self.left, self.right, self.norm_eps = hidden_size, left, right, float(norm_eps)
        self.names, self.out_suffix = names, out_suffix
        self.w_left = self.w_right = None

    def _sides(self, prefix):
        return [(self.left, prefix + "." + self.names[0]), (self.right, prefix + "." + self.names[1])]

    def weight_specs(self, prefix):
        specs = [s for part, p in self._sides(prefix) for s in part.weight_specs(p)]
        return specs + [WeightSpec(p + self.out_suffix, (self.hidden_size,), "norm") for _, p in self._sides(prefix)]

    def bind(self, prefix, weights):
        for part, p in self._sides(prefix):
            part.bind(p, weights)
        self.w_left, self.w_right = (weights[p + self.out_suffix] for _, p in self._sides(prefix))
        if self.w_left.dtype != self.w_right.dtype:
            self.w_left, self.w_right = self.w_left.float(), self.w_right.float()

    def cache_spec(self):
        """A list: one need per side (None where a side keeps nothing)."""
        return [self.left.cache_spec(), self.right.cache_spec()]

    def plan(self, batch) -> None:
        self.left.plan(batch)
        self.right.plan(batch)

    def plan_arrays(self, entries):
        out = dict(self.left.plan_arrays(entries))
        out.update(self.right.plan_arrays(entries))
        return out

    def capturable(self, batch):
        return self.left.capturable(batch) and self.right.capturable(batch)

    def forward(self, x, batch, cache, store=True):
        left_cache, right_cache = cache
        a = self.left.forward(x, batch, left_cache, store)
        b = self.right.forward(x, batch, right_cache, store)
        return ops.norm_pair_mean(a, b, self.w_left, self.w_right, self.norm_eps)
