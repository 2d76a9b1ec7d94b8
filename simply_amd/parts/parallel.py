"""Two mixers side by side: both read the same input, the result is a weighted sum of theirs.  Each keeps its own
cache or state (`CompositeNeed`); their tensors are the parts' own, under the prefixes 'left.' and 'right.'."""
from __future__ import annotations

from ..config.spec import PartSpec
from ..kernels import ops
from ..registry import MIXERS
from .base import CompositeNeed, Mixer


@MIXERS.register("parallel")
class ParallelMixers(Mixer):
    SIDES = ("left", "right")

    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0):
        self.parts = {"left": MIXERS.build(left.kind, **left.params), "right": MIXERS.build(right.kind, **right.params)}
        self.scales = {"left": float(left_scale), "right": float(right_scale)}

    def param_specs(self):
        return {f"{side}.{name}": spec for side in self.SIDES for name, spec in self.parts[side].param_specs().items()}

    def load(self, tensors):
        for side in self.SIDES:
            prefix = side + "."
            self.parts[side].load({n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)})

    def cache_need(self):
        return CompositeNeed(tuple(self.parts[side].cache_need() for side in self.SIDES))

    def forward(self, x, ctx, cache):
        left = self.parts["left"].forward(x, ctx, cache.parts[0])
        right = self.parts["right"].forward(x, ctx, cache.parts[1])
        return ops.weighted_sum(left, self.scales["left"], right, self.scales["right"])
