"""Rotary position encoding; half-split pairing (i, i + rot_dim/2) unless told
`pairing="interleaved"` (neighbours 2i, 2i + 1).

f_i = theta^(-2i/rot_dim), evaluated in double and rounded once to 32-bit
(reference src/models/model.hip:635-642 builds the same table with std::pow);
the angle pos * f_i, its sine and cosine and the rotation are 32-bit in the
kernel (reference src/ops/kernels.hip:73-94). `rot_dim` may be smaller than
the head size (the rest of the head is left alone); 0 means no rotation.

`scaling` stretches the slow pairs for contexts beyond the trained one (the
NTK-by-parts rule known as YaRN): with d(t) = rot_dim ln(original / (2 pi t)) /
(2 ln theta), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), rot_dim - 1)
and r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at
f_i / factor * r_i + f_i * (1 - r_i), and cosine and sine are both multiplied by
`magnitude` = 0.1 ln(factor) + 1.

A `scaling` with the keys {factor, original, low, high} slows pairs down by their wavelength
l_i = 2 pi / f_i instead: f_i stays where l_i < original / high, becomes f_i / factor where
l_i > original / low, and between the two, with s = (original / l_i - low) / (high - low),
(1 - s) f_i / factor + s f_i; cosine and sine keep their size.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..registry import register_part
from .base import PositionEncoding, WeightBinder


class Rotary(PositionEncoding):
    def __init__(self, rot_dim: int, theta: float, pairing: str = "half",
                 scaling: Optional[Dict[str, float]] = None):
        """`scaling`: None, or {'factor', 'original', 'fast', 'slow'}: the stretch, the trained
        context, and the turns over that context above which a pair is left alone (`fast`)
        and below which it is stretched in full (`slow`); or {'factor', 'original', 'low',
        'high'}: the same bounds given as wavelengths, original / high and original / low, with
        the blend linear in the turns and cosine and sine left as they are."""
        if rot_dim % 2:
            raise ValueError(f"rotary dimension must be even, got {rot_dim}")
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"pairing must be 'half' or 'interleaved', got {pairing!r}")
        self.rot_dim = rot_dim
        self.pairing = pairing
        self.theta = float(theta)
        self.scaling = None
        self.magnitude = 1.0   # factor on cosine and sine
        self.bands = None
        if scaling is not None and "low" in scaling and "high" in scaling:
            missing = [k for k in ("factor", "original") if k not in scaling]
            if missing:
                raise ValueError(f"rotary scaling lacks {missing}")
            self.bands = {k: float(scaling[k]) for k in ("factor", "original", "low", "high")}
            if not self.bands["factor"] > 0 or not self.bands["high"] > self.bands["low"] > 0:
                raise ValueError("rotary scaling needs factor > 0 and high > low > 0")
        elif scaling is not None:
            missing = [k for k in ("factor", "original", "fast", "slow") if k not in scaling]
            if missing:
                raise ValueError(f"rotary scaling lacks {missing}")
            self.scaling = {k: float(scaling[k]) for k in ("factor", "original", "fast", "slow")}
            if not self.scaling["factor"] > 0 or not self.theta > 1:
                raise ValueError("rotary scaling needs factor > 0 and theta > 1")
            self.magnitude = 0.1 * math.log(self.scaling["factor"]) + 1.0
        self._table: Optional[torch.Tensor] = None

    def inv_freq(self) -> torch.Tensor:
        vals = [math.pow(self.theta, -(2.0 * i) / self.rot_dim)
                for i in range(self.rot_dim // 2)]
        if self.scaling is not None:
            sc, n = self.scaling, self.rot_dim

            def place(turns: float) -> float:
                return n * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
            lo = max(math.floor(place(sc["fast"])), 0)
            hi = min(math.ceil(place(sc["slow"])), n - 1)
            for i in range(n // 2):
                ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                vals[i] = vals[i] / sc["factor"] * ramp + vals[i] * (1.0 - ramp)
        if self.bands is not None:
            b = self.bands
            for i, f in enumerate(vals):
                wave = 2.0 * math.pi / f
                if wave < b["original"] / b["high"]:
                    continue
                if wave > b["original"] / b["low"]:
                    vals[i] = f / b["factor"]
                else:
                    s = (b["original"] / wave - b["low"]) / (b["high"] - b["low"])
                    vals[i] = (1.0 - s) * f / b["factor"] + s * f
        return torch.tensor(vals, dtype=torch.float64).to(torch.float32)

    def bind(self, w: WeightBinder) -> None:
        self._table = self.inv_freq().to(w.device)

    def table(self) -> Optional[torch.Tensor]:
        return self._table


class NoPosition(PositionEncoding):
    """Queries and keys are used as projected."""
    rot_dim = 0

    def table(self) -> Optional[torch.Tensor]:
        return None


register_part("position", "rotary", Rotary)
register_part("position", "none", NoPosition)
