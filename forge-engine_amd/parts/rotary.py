"""Rotary position encoding: the table of inverse frequencies that attention
rotates q and k with.

``inv_freq[j] = 1 / theta^(2j / R)``, j < R/2, in float32, computed with the
same expression as the reference (src/forge_engine/qwen3.py:352-360) so that the
angles ``float(position) * inv_freq[j]`` are bit-equal to its own.  R is the
number of rotated dims (the whole head unless ``rotary_dim`` says less); the
partner of dim j is j + R/2 (rotate-half pairing, qwen3.py:366-381).
"""

from __future__ import annotations

import math

import torch

from ..registry import register_part
from .base import BuildContext, PositionEncoding


class RotaryPosition(PositionEncoding):
    def __init__(self, ctx: BuildContext, prefix: str = "", *, head_dim: int, theta: float,
                 rotary_dim: int | None = None, precise: bool = False) -> None:
        """``precise``: the table is computed in 64-bit and rounded once, instead of with the
        reference's float32 expression."""
        super().__init__(ctx, prefix)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {head_dim}")
        exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        self.inv_freq = (1.0 / (float(theta) ** exponent)).to(ctx.device)
        if precise:
            table = [float(theta) ** (-2.0 * j / self.rotary_dim) for j in range(self.rotary_dim // 2)]
            self.inv_freq = torch.tensor(table, dtype=torch.float64).to(torch.float32).to(ctx.device)

    def rotary(self):
        return self.inv_freq, self.rotary_dim


class YarnRotaryPosition(RotaryPosition):
    """Rotary frequencies stretched for contexts beyond the trained one (YaRN).  With
    ``turning(t) = R ln(original / (2 pi t)) / (2 ln theta)`` (the pair index that makes t turns
    over the original context), ``lo = max(floor(turning(fast)), 0)``, ``hi = min(ceil(turning(slow)),
    R - 1)`` and ``ramp_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1)``, pair j turns at
    ``f_j / factor * ramp_j + f_j (1 - ramp_j)``: fast pairs keep their frequency, slow ones are
    divided by the factor.  Cosines and sines are multiplied by ``0.1 ln(factor) + 1``
    (``magnitude``)."""

    def __init__(self, ctx: BuildContext, prefix: str = "", *, head_dim: int, theta: float, factor: float,
                 original: float, fast: float, slow: float, rotary_dim: int | None = None) -> None:
        super().__init__(ctx, prefix, head_dim=head_dim, theta=theta, rotary_dim=rotary_dim)
        dims, half = self.rotary_dim, self.rotary_dim // 2

        def turning(turns: float) -> float:
            return dims * math.log(float(original) / (2.0 * math.pi * turns)) / (2.0 * math.log(float(theta)))

        lo = max(math.floor(turning(float(fast))), 0)
        hi = min(math.ceil(turning(float(slow))), dims - 1)
        plain = [float(theta) ** (-2.0 * j / dims) for j in range(half)]
        ramp = [min(max((j - lo) / max(hi - lo, 0.001), 0.0), 1.0) for j in range(half)]
        blended = [f / float(factor) * r + f * (1.0 - r) for f, r in zip(plain, ramp)]
        self.inv_freq = torch.tensor(blended, dtype=torch.float64).to(torch.float32).to(ctx.device)
        self._magnitude = 0.1 * math.log(float(factor)) + 1.0

    def magnitude(self) -> float:
        return self._magnitude


class NoPosition(PositionEncoding):
    """No position information inside the mixer."""

    def __init__(self, ctx: BuildContext, prefix: str = "") -> None:
        super().__init__(ctx, prefix)


register_part("position", "rotary", RotaryPosition)
register_part("position", "yarn_rotary", YarnRotaryPosition)
register_part("position", "none", NoPosition)
