"""Sinusoidal positions added to the embedded tokens.

Channel 2i of the vector for position p is sin(p * base^(-2i/width)), channel 2i + 1 the
cosine of the same angle; angles are worked out in double.  Parameters: ``base`` (default
10000).  No tensors.  Named by the embedding's ``position`` parameter.
"""

from __future__ import annotations

from .. import kernels as K
from .base import Part, register_part


@register_part("position", "sinusoidal")
class SinusoidalPositions(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.base = float(self.param("base", 10000.0))
        if not self.base > 0:
            raise ValueError(f"sinusoidal: base {self.base} must be positive")

    def on_embedding(self, ctx, x):
        K.add_sinusoid(x, ctx.positions, self.base)
