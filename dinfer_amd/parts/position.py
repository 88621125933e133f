"""Position encodings. The mixer's kernel rotates q and k by a table this part builds.

Rotary: row p of the table is [cos(p f_i) | sin(p f_i)], f_i = theta^(-2i / rotary_dim),
i < rotary_dim / 2, computed in float64 on the host and stored in float32
(crates/layers/src/nn.rs:152-185). rotary_dim may be smaller than the head
size (the other dims are not rotated); style selects the pairing.

With `scaling` (factor s, original length L, fast, slow; "YaRN"): dimensions that turn often within L keep their
frequency, those that turn rarely are slowed by s, with a linear ramp between: for d(t) = D ln(L / (2 pi t)) / (2 ln theta),
lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), D - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the
frequency is f_i / s * r_i + f_i * (1 - r_i), and cos and sin are both multiplied by 0.1 ln(s) + 1.

With `scaling` of kind "wavelength_bands" (factor s, original length L, low, high): by the wavelength l_i = 2 pi / f_i a
frequency is kept (l_i < L / high), divided by s (l_i > L / low), or, between the two, blended with
t = (L / l_i - low) / (high - low) as (1 - t) f_i / s + t f_i; cos and sin keep their size.
"""
from __future__ import annotations

import torch

from .base import PositionEncoding
from .registry import POSITION_ENCODINGS

STYLES = {"neox": 0, "interleaved": 1}


@POSITION_ENCODINGS.register("none")
class NoPosition(PositionEncoding):
    def __init__(self, head_dim: int = 0, **_):
        self.rotary_dim, self.style = 0, 0

    def table(self):
        return None


@POSITION_ENCODINGS.register("rotary")
class Rotary(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, max_positions: int, rotary_dim: int | None = None,
                 style: str = "neox", scaling: dict | None = None):
        rd = head_dim if rotary_dim is None else rotary_dim
        if rd <= 0 or rd > head_dim or rd % 2:
            raise ValueError(f"rotary_dim {rd} must be even and in (0, head_dim={head_dim}]")
        if style not in STYLES:
            raise ValueError(f"rotary style {style!r} unknown; known: {sorted(STYLES)}")
        self.head_dim, self.theta, self.max_positions = head_dim, float(theta), max_positions
        self.rotary_dim, self.style = rd, STYLES[style]
        self.scaling = None
        self.scaling_kind = None
        if scaling:
            self.scaling_kind = scaling.get("kind", "ramp")
            if self.scaling_kind not in ("ramp", "wavelength_bands"):
                raise ValueError(f"rotary scaling kind {self.scaling_kind!r} unknown; known: 'ramp', 'wavelength_bands'")
            keys = ("factor", "original", "fast", "slow") if self.scaling_kind == "ramp" else ("factor", "original", "low", "high")
            sc = {k: float(scaling[k]) for k in keys}
            if not all(v > 0 for v in sc.values()):
                raise ValueError(f"rotary scaling needs positive {', '.join(keys)}, got {scaling!r}")
            if self.scaling_kind == "wavelength_bands" and not sc["high"] > sc["low"]:
                raise ValueError(f"rotary scaling by wavelength needs high > low, got {scaling!r}")
            self.scaling = sc
        self._table = None

    def bind(self, ctx):
        # one table for all layers with the same rotation, as long as the longest request the engine admits
        n = min(self.max_positions, ctx.max_seq_len or self.max_positions)
        sc = (self.scaling_kind,) + tuple(sorted(self.scaling.items())) if self.scaling else None
        self._table = ctx.share(("rotary", self.theta, self.rotary_dim, self.style, n, sc),
                                lambda: self.host_table(n).to(ctx.device).contiguous())

    def frequencies(self) -> tuple[torch.Tensor, float]:
        """(float64 frequency per pair, the factor on cos and sin)."""
        import math
        D = self.rotary_dim
        i = torch.arange(0, D // 2, dtype=torch.float64)
        freq = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / D)
        if self.scaling is None:
            return freq, 1.0
        sc = self.scaling
        if self.scaling_kind == "wavelength_bands":
            wavelength = 2 * math.pi / freq
            t = ((sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])).clamp(0, 1)
            # t is 0 where the wavelength exceeds original / low and 1 where it is below original / high
            return (1 - t) * freq / sc["factor"] + t * freq, 1.0

        def dim_of(turns: float) -> float:     # the (fractional) pair index that makes `turns` turns within the original length
            return D * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(self.theta))

        lo = max(math.floor(dim_of(sc["fast"])), 0)
        hi = min(math.ceil(dim_of(sc["slow"])), D - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        return freq / sc["factor"] * ramp + freq * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0

    def host_table(self, positions: int | None = None) -> torch.Tensor:
        freq, mag = self.frequencies()
        ang = torch.arange(positions or self.max_positions, dtype=torch.float64)[:, None] * freq[None, :]
        return (torch.cat([ang.cos(), ang.sin()], dim=1) * mag).to(torch.float32)

    def table(self):
        if self._table is None:
            raise RuntimeError("the rotation table is built in bind(); the part has not been bound")
        return self._table
