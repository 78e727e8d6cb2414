"""Position encodings.

``RotaryEncoding`` builds the float32 cos/sin tables the way the reference does
(``src/rope.py:45-56``): ``inv_freq[i] = 1 / theta^(2i/d)``, positions divided by a
linear scaling factor, ``cos/sin(pos * inv_freq)``, kept in float32 whatever the
run dtype (``src/rope.py:58-63``).  The rotation itself (halves paired ``(i, i + d/2)``,
``src/rope_inplace.py:25-47``) is fused into the attention mixer's cache-write kernel.
The tables are built on the host so that every run, on any device, rotates by
bit-identical angles.

Two options beyond the reference's: ``layout`` says which channels are a pair (``halves``:
``(i, i + d/2)``; ``interleaved``: ``(2i, 2i + 1)``; the mixer's rotation kernel reads it), and
``stretch = (factor, original, fast, slow)`` stretches the slow frequencies for contexts beyond the
``original`` length (YaRN): with ``dim(t) = d ln(original / (2 pi t)) / (2 ln theta)``,
``lo = max(floor(dim(fast)), 0)``, ``hi = min(ceil(dim(slow)), d - 1)`` and
``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)`` the frequency becomes
``f_i / factor * r_i + f_i (1 - r_i)``, and cos and sin are both multiplied by
``0.1 ln(factor) + 1``, which the tables hold already.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch

from .base import PositionEncoding, register_part


class RotaryEncoding(PositionEncoding):
    def __init__(self, rotary_dim: int, theta: float, max_position: int, scaling_factor: float = 1.0, layout: str = "halves",
                 stretch: Optional[Sequence[float]] = None, exact_angles: bool = False) -> None:
        """``exact_angles``: frequencies ``theta^(-2i/d) / scaling_factor`` and the angles ``p * f_i`` are worked out in
        float64 and only cosine and sine are rounded to float32 (the tables then do not carry the float32 error of the
        angle, which grows with the position)."""
        super().__init__("")
        self.exact_angles = bool(exact_angles)
        if rotary_dim % 2 != 0:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        if layout not in ("halves", "interleaved"):
            raise ValueError(f"layout must be 'halves' or 'interleaved', got {layout!r}")
        if stretch is not None and (len(stretch) != 4 or not stretch[0] > 0 or not stretch[1] > 0 or not stretch[2] > 0 or not stretch[3] > 0):
            raise ValueError(f"stretch must be four positive numbers (factor, original, fast, slow), got {stretch!r}")
        self.layout = layout
        self.stretch = tuple(float(v) for v in stretch) if stretch is not None else None
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        self.max_position = int(max_position)
        self.scaling_factor = float(scaling_factor)
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def frequencies(self) -> Tuple[torch.Tensor, float]:
        """float32 ``[rotary_dim / 2]`` and the factor that cos and sin are multiplied with."""
        if self.stretch is None:
            exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
            return 1.0 / (self.theta ** exponent), 1.0
        factor, original, fast, slow = self.stretch
        d = self.rotary_dim
        index = torch.arange(d // 2, dtype=torch.float64)
        plain = self.theta ** (-2.0 * index / d)

        def dim_of(turns: float) -> float:
            return d * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

        lo = max(math.floor(dim_of(fast)), 0)
        hi = min(math.ceil(dim_of(slow)), d - 1)
        ramp = ((index - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return (plain / factor * ramp + plain * (1.0 - ramp)).float(), 0.1 * math.log(factor) + 1.0

    def finalize(self, device, dtype) -> None:
        if self.exact_angles and self.stretch is None:
            index = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
            freq = self.theta ** (-2.0 * index / self.rotary_dim) / self.scaling_factor
            angles = torch.outer(torch.arange(self.max_position, dtype=torch.float64), freq)
            self.cos = angles.cos().float().contiguous().to(device)
            self.sin = angles.sin().float().contiguous().to(device)
            return
        inv_freq, magnitude = self.frequencies()
        positions = torch.arange(self.max_position, dtype=torch.float32)
        if self.scaling_factor != 1.0:
            positions = positions / self.scaling_factor
        angles = torch.outer(positions, inv_freq)
        cos, sin = angles.cos(), angles.sin()
        if magnitude != 1.0:
            cos, sin = cos * magnitude, sin * magnitude
        self.cos = cos.contiguous().to(device)
        self.sin = sin.contiguous().to(device)

    def rotary_tables(self) -> Optional[Tuple[torch.Tensor, torch.Tensor]]:
        return self.cos, self.sin


class SinusoidalEncoding(PositionEncoding):
    """An absolute encoding added to the embeddings: entry ``2i`` of position ``p`` is ``sin(p * base^(-2i/width))`` and
    entry ``2i + 1`` the cosine of the same angle.  Nothing is stored per position: the kernel takes the frequencies
    (float64, built on the host) and works the angle out for each of the step's tokens, so there is no limit on
    positions and no table of ``max_position x width``."""

    def __init__(self, width: int, base: float = 10000.0) -> None:
        super().__init__("")
        if width < 1 or not base > 0:
            raise ValueError("width and base must be positive")
        self.width = int(width)
        self.base = float(base)
        self.frequencies: Optional[torch.Tensor] = None

    def finalize(self, device, dtype) -> None:
        pairs = (self.width + 1) // 2
        self.frequencies = torch.tensor([self.base ** (-2.0 * i / self.width) for i in range(pairs)], dtype=torch.float64).to(device)

    def on_embeddings(self, hidden: torch.Tensor, ctx) -> torch.Tensor:
        return ctx.ops.add_sinusoid(hidden, ctx.positions, self.frequencies)


class NoPositionEncoding(PositionEncoding):
    def __init__(self) -> None:
        super().__init__("")


register_part("position", "rotary", RotaryEncoding)
register_part("position", "sinusoidal", SinusoidalEncoding)
register_part("position", "none", NoPositionEncoding)
