"""Rotary position encodings: tables of cos and sin for a step's positions; the mixer's kernel
rotates with them, pairing dimensions half-split or interleaved as the encoding says."""

from __future__ import annotations

import torch

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels import ops
from tokamak_amd.parts.base import PositionData, PositionEncoding


class RotaryHalf(PositionEncoding):
    """cos/sin tables for a step's positions.

    inv_freq[j] = 1 / theta^(2j / rotary_dim), float32, computed on the host
    exactly as written in reference: src/tokamak/model/layers.py:47; the angle
    float(pos) * inv_freq[j] and its cos/sin are float32 (layers.py:56-58).  The
    rotation itself pairs dim j with dim j + rotary_dim/2 (layers.py:61-63) and
    is applied by the mixer's fused kernel.

    ``scaling`` = (factor, low, high, original) rescales the frequencies by wavelength
    l = 2 pi / f: kept where l < original / high, divided by ``factor`` where l > original / low,
    and in between (1 - s) f / factor + s f with s = (original / l - low) / (high - low);
    computed on the host in double precision, then rounded to float32 once.

    ``yarn`` = (factor, original, fast, slow) stretches the slow frequencies with a ramp over the
    dimensions instead and multiplies both tables by 0.1 ln(factor) + 1 (``yarn_frequencies``).
    """

    capturable = True
    replayable = True

    def __init__(self, *, rotary_dim: int, theta: float, dtype, device, scaling: tuple | None = None,
                 yarn: tuple | None = None) -> None:
        super().__init__(dtype=dtype, device=device)
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        if scaling is not None and yarn is not None:
            raise ValueError("frequencies are rescaled by wavelength or stretched by a ramp, not both")
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        self.scaling = None if scaling is None else tuple(float(x) for x in scaling)
        self.yarn = None if yarn is None else tuple(float(x) for x in yarn)
        self.amplitude = 1.0
        if self.yarn is not None:
            freqs, self.amplitude = yarn_frequencies(self.rotary_dim, self.theta, self.yarn)
            inv_freq = torch.tensor(freqs, dtype=torch.float64).to(torch.float32)
        elif self.scaling is None:
            inv_freq = 1.0 / (self.theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
        else:
            inv_freq = torch.tensor(scaled_frequencies(self.rotary_dim, self.theta, *self.scaling), dtype=torch.float32)
        self.inv_freq = inv_freq.to(self.device)
        self.key = ("rotary_half", self.rotary_dim, self.theta, self.scaling, self.yarn)

    def prepare(self, batch) -> PositionData:
        """cos and sin, each float32 [N, rotary_dim/2]; computed once per step."""
        cached = batch.memo.get(self.key)
        if cached is None:
            n, half = batch.num_tokens, self.rotary_dim // 2
            cos = torch.empty((n, half), dtype=torch.float32, device=self.device)
            sin = torch.empty((n, half), dtype=torch.float32, device=self.device)
            ops.rope_tables(batch.positions, self.inv_freq, cos, sin, self.amplitude)
            cached = batch.memo[self.key] = PositionData(cos=cos, sin=sin, rotary_dim=self.rotary_dim)
        return cached


class RotaryInterleaved(PositionEncoding):
    """cos/sin tables for a rotation that pairs dimension 2j with 2j + 1.

    f_j = theta^(-2j / rotary_dim), computed on the host in double precision and rounded to float32
    once; the angle float(pos) * f_j and its cos/sin are float32.  The pair (u, v) becomes
    (u cos - v sin, v cos + u sin), applied by the mixer's kernel.

    ``yarn`` = (factor, original, fast, slow) stretches the slow frequencies for contexts beyond
    ``original`` positions: with d(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta),
    lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), rotary_dim - 1) and the ramp
    r_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1), the frequency is f_j / factor * r_j + f_j (1 - r_j),
    and both tables are multiplied by 0.1 ln(factor) + 1.
    """

    capturable = True
    replayable = True

    def __init__(self, *, rotary_dim: int, theta: float, dtype, device, yarn: tuple | None = None) -> None:
        super().__init__(dtype=dtype, device=device)
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        self.yarn = None if yarn is None else tuple(float(x) for x in yarn)
        freqs, self.amplitude = yarn_frequencies(self.rotary_dim, self.theta, self.yarn)
        self.inv_freq = torch.tensor(freqs, dtype=torch.float64).to(torch.float32).to(self.device)
        self.key = ("rotary_interleaved", self.rotary_dim, self.theta, self.yarn)

    def prepare(self, batch) -> PositionData:
        """cos and sin, each float32 [N, rotary_dim/2]; computed once per step."""
        cached = batch.memo.get(self.key)
        if cached is None:
            n, half = batch.num_tokens, self.rotary_dim // 2
            cos = torch.empty((n, half), dtype=torch.float32, device=self.device)
            sin = torch.empty((n, half), dtype=torch.float32, device=self.device)
            ops.rope_tables(batch.positions, self.inv_freq, cos, sin, self.amplitude)
            cached = batch.memo[self.key] = PositionData(cos=cos, sin=sin, rotary_dim=self.rotary_dim, interleaved=True)
        return cached


def yarn_frequencies(rotary_dim: int, theta: float, yarn: tuple | None) -> tuple[list[float], float]:
    """(theta^(-2j / rotary_dim) for j < rotary_dim / 2, stretched as ``RotaryInterleaved`` says; the
    amplitude of the tables), in double precision."""
    import math

    freqs = [theta ** (-2.0 * j / rotary_dim) for j in range(rotary_dim // 2)]
    if yarn is None:
        return freqs, 1.0
    factor, original, fast, slow = yarn
    if factor <= 0 or original <= 0 or fast <= 0 or slow <= 0 or theta <= 1:
        raise ValueError("yarn scaling needs positive factor, original, fast and slow, and a base above 1")

    def dim_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(dim_of(fast)), 0)
    hi = min(math.ceil(dim_of(slow)), rotary_dim - 1)
    span = max(hi - lo, 0.001)
    for j in range(len(freqs)):
        ramp = min(max((j - lo) / span, 0.0), 1.0)
        freqs[j] = freqs[j] / factor * ramp + freqs[j] * (1.0 - ramp)
    return freqs, 0.1 * math.log(factor) + 1.0


def scaled_frequencies(rotary_dim: int, theta: float, factor: float, low: float, high: float, original: float) -> list[float]:
    """theta^(-2j / rotary_dim) for j < rotary_dim / 2, rescaled by wavelength (see ``RotaryHalf``)."""
    import math

    if factor <= 0 or high <= low or original <= 0:
        raise ValueError("frequency scaling needs factor > 0, high > low and original > 0")
    out = []
    for j in range(rotary_dim // 2):
        f = theta ** (-2.0 * j / rotary_dim)
        turns = original * f / (2.0 * math.pi)      # original / wavelength
        if turns > high:
            pass
        elif turns < low:
            f /= factor
        else:
            s = (turns - low) / (high - low)
            f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


register_part("position", "rotary_half", RotaryHalf)
register_part("position", "rotary_interleaved", RotaryInterleaved)
