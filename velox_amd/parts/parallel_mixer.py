"""Two mixers side by side: both read the same input, the result is ``left_scale * left(x) + right_scale * right(x)``.

The two are parts of any registered mixer kinds, built from their ``PartSpec`` under ``<prefix><left_prefix>`` and
``<prefix><right_prefix>``; each keeps the cache or state its own kind asks for (the pair's need is the
``CompositeNeed`` of theirs).  The weighted sum is not a pass of its own: it is handed on as a ``ScaledSum``, which the
kernel that adds a sub-layer's output to the residual forms in float32.
"""
from __future__ import annotations

from typing import Tuple

from .base import CompositeNeed, Mixer, Part, PartSpec, ScaledSum, make_part, register_part


class ParallelMixer(Mixer):
    def __init__(self, prefix: str, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0,
                 left_prefix: str = "left.", right_prefix: str = "right.", position=None, position_to: Tuple[bool, bool] = (True, False)) -> None:
        """``position``: the layer's position encoding (a part); ``position_to`` says which of the two mixers takes it."""
        super().__init__(prefix)
        self.scales = (float(left_scale), float(right_scale))
        self.mixers = []
        for spec, below, takes in ((left, left_prefix, position_to[0]), (right, right_prefix, position_to[1])):
            kwargs = spec.kwargs()
            if position is not None and takes:
                kwargs["position"] = position
            self.mixers.append(make_part("mixer", spec.kind, prefix=prefix + below, **kwargs))

    def children(self) -> Tuple[Part, ...]:
        return tuple(self.mixers)

    def cache_need(self):
        return CompositeNeed(tuple(mixer.cache_need() for mixer in self.mixers))

    def forward(self, x, ctx, cache, owns_cache: bool = True):
        outputs = []
        for mixer, view in zip(self.mixers, cache.views):
            y = mixer.forward(x, ctx, view, owns_cache)
            outputs.append(y.sum(0) if y.dim() == 3 else y)
        return ScaledSum(tuple(outputs), self.scales)


register_part("mixer", "parallel_mixers", ParallelMixer)
