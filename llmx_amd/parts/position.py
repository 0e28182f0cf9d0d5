"""Position encodings.

Rotary tables follow the reference's float32 arithmetic (/root/reference/src/model/rope.hpp:25-28,203-210):
freq_i = 1.0f / powf(theta, 2.0f*i/R), angle = (float)pos * freq_i, cos and sin of that angle, one table for all
layers, pairs (i, i + R/2) of each head rotated (NeoX halves).
"""

from __future__ import annotations

import numpy as np
import torch

from .base import PositionEncoding, register

PAIRINGS = ("halves", "interleaved")


def neox_table(positions: int, rotary_dim: int, theta: float) -> np.ndarray:
    """[positions, rotary_dim] float32: cos of the rotary_dim/2 pairs, then sin.

    Every value is what correctly rounded float32 functions give: the power, the cosine and the sine are computed in
    float64 from their float32 arguments and rounded once (vectorised float32 routines lose bits in the range reduction
    of large angles, and a position of 65,536 is a large angle); products and the division are float32.
    """
    half = rotary_dim // 2
    if half == 0:
        return np.zeros((positions, 0), dtype=np.float32)
    i = np.arange(half, dtype=np.float32)
    exponent = (np.float32(2.0) * i / np.float32(rotary_dim)).astype(np.float32)
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
    freq = (np.float32(1.0) / power).astype(np.float32)
    pos = np.arange(positions, dtype=np.float32)[:, None]
    angle = (pos * freq[None, :]).astype(np.float32).astype(np.float64)
    return np.concatenate([np.cos(angle), np.sin(angle)], axis=1).astype(np.float32)


class PartialRotary(PositionEncoding):
    """params: rotary_dim (even, at most head_dim; 0 rotates nothing), theta, head_dim, pairing ("halves", the default:
    dims i and i + rotary_dim/2 rotate together; "interleaved": dims 2i and 2i + 1)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.pairing = str(params.get("pairing", "halves"))
        if self.pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {self.pairing!r} is not one of {sorted(PAIRINGS)}")
        self.rotary_dim = int(params["rotary_dim"])
        self.theta = float(params["theta"])
        head_dim = int(params["head_dim"])
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= head_dim:
            raise ValueError(f"rotary width {self.rotary_dim} must be even and at most the head width {head_dim}")
        table = neox_table(ctx.max_positions, self.rotary_dim, self.theta)
        self.cos_sin = torch.from_numpy(table).to(ctx.device)

    def rotation(self):
        return self.cos_sin, self.rotary_dim


def blended_frequencies(dims: int, base: float, scaling) -> tuple:
    """(frequencies [dims/2] float64, magnitude): f_i = base^(-2i/dims); with `scaling` = {factor, original, fast, slow}
    the YaRN blend: pairs that turn more than `fast` times over `original` positions keep f_i, pairs that turn fewer
    than `slow` times get f_i / factor, and between them a linear ramp over the pair index decides:
    pair(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(pair(fast)), 0), hi = min(ceil(pair(slow)),
    dims - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), f = f_i / factor * ramp_i + f_i (1 - ramp_i);
    cos and sin are then multiplied by magnitude = 0.1 ln(factor) + 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = np.power(float(base), -2.0 * i / float(dims)) if dims else i
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])
    fast, slow = float(scaling["fast"]), float(scaling["slow"])
    if not (factor > 0.0 and original > 0.0 and fast > 0.0 and slow > 0.0 and base > 1.0):
        raise ValueError("rotary scaling: factor, original, fast and slow must be positive and the base above 1")

    def pair_of(turns: float) -> float:
        return dims * np.log(original / (2.0 * np.pi * turns)) / (2.0 * np.log(float(base)))

    lo = max(int(np.floor(pair_of(fast))), 0)
    hi = min(int(np.ceil(pair_of(slow))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * float(np.log(factor)) + 1.0


def wavelength_scaled_frequencies(dims: int, base: float, scaling) -> np.ndarray:
    """Frequencies [dims/2] float64 rescaled by wavelength: f_i = base^(-2i/dims); with `scaling` = {factor, low, high,
    original} and a pair's wavelength l = 2 pi / f: l < original/high keeps f; l > original/low gives f / factor; between
    the two, s = (original/l - low) / (high - low) blends them, (1 - s) f / factor + s f.  No factor on cos and sin."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = np.power(float(base), -2.0 * i / float(dims)) if dims else i
    if not scaling:
        return f
    factor, original = float(scaling["factor"]), float(scaling["original"])
    low, high = float(scaling["low"]), float(scaling["high"])
    if not (factor > 0.0 and original > 0.0 and low > 0.0 and high > low):
        raise ValueError("rotary scaling: factor, original and low must be positive and high above low")
    wavelength = 2.0 * np.pi / f
    s = (original / wavelength - low) / (high - low)
    blended = (1.0 - s) * f / factor + s * f
    return np.where(wavelength < original / high, f, np.where(wavelength > original / low, f / factor, blended))


def scaled_table(positions: int, dims: int, base: float, scaling) -> np.ndarray:
    """[positions, dims] float32: magnitude * cos of the dims/2 pairs' angles, then magnitude * sin.  The angle is the
    float32 product of the position and the float32 frequency; cos and sin are evaluated in float64 on it and rounded
    once, as `neox_table` does."""
    if dims == 0:
        return np.zeros((positions, 0), dtype=np.float32)
    if scaling and "low" in scaling:           # {factor, low, high, original}: rescaled by wavelength
        # this form has no float32 recipe to follow: the angle is formed in float64 and only cos and sin are rounded
        f = wavelength_scaled_frequencies(dims, base, scaling)
        angle = np.arange(positions, dtype=np.float64)[:, None] * f[None, :]
        return np.concatenate([np.cos(angle), np.sin(angle)], axis=1).astype(np.float32)
    f, magnitude = blended_frequencies(dims, base, scaling)      # None, or {factor, original, fast, slow}
    pos = np.arange(positions, dtype=np.float32)[:, None]
    angle = (pos * f.astype(np.float32)[None, :]).astype(np.float32).astype(np.float64)
    return (np.concatenate([np.cos(angle), np.sin(angle)], axis=1) * magnitude).astype(np.float32)


class ScaledRotary(PositionEncoding):
    """Rotary pairs with optionally rescaled frequencies.  params: dims (even; the rotated dims), base, scaling (None;
    {factor, original, fast, slow}: the YaRN blend over the pair index with its factor on cos and sin; {factor, low, high,
    original}: frequencies rescaled by wavelength, see `wavelength_scaled_frequencies`), pairing ("interleaved", the default here: dims 2i and 2i + 1; "halves")."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.pairing = str(params.get("pairing", "interleaved"))
        if self.pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {self.pairing!r} is not one of {sorted(PAIRINGS)}")
        self.rotary_dim = int(params["dims"])
        if self.rotary_dim % 2 or self.rotary_dim < 0:
            raise ValueError(f"rotary width {self.rotary_dim} must be even")
        self.base = float(params["base"])
        self.scaling = dict(params["scaling"]) if params.get("scaling") else None
        self.cos_sin = torch.from_numpy(scaled_table(ctx.max_positions, self.rotary_dim, self.base, self.scaling)).to(ctx.device)

    def rotation(self):
        return self.cos_sin, self.rotary_dim


class NoPosition(PositionEncoding):
    """Leaves rows as they are."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.cos_sin = torch.zeros((max(1, ctx.max_positions), 0), dtype=torch.float32, device=ctx.device)

    def rotation(self):
        return self.cos_sin, 0


register("position", "rotary_neox_partial", PartialRotary)
register("position", "rotary_scaled", ScaledRotary)
register("position", "none", NoPosition)
