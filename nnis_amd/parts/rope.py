"""Rotate-half rotary position encoding.  The tables are built once on the
host in 32-bit as the reference builds them
(/root/reference/crates/nnis-model/src/runtime.rs:1166-1184):
exponent = (2*pair)/rot_dim, inv_freq = 1/theta**exponent, angle = pos*inv_freq.
``powf``, ``cos`` and ``sin`` of a 32-bit argument are evaluated in 64-bit and
rounded once, which is what a correctly rounded 32-bit routine returns.
"""

from __future__ import annotations

import math

import torch

from ..errors import InvalidInput
from .base import PositionEncoding, RotaryTables, register_part


def bend_frequencies(inv_freq: torch.Tensor, factor: float, low: float, high: float, original: float) -> torch.Tensor:
    """Frequencies bent by their wavelength l = 2 pi / f: f stays where l <
    original / high, becomes f / factor where l > original / low, and between
    the two (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    f = inv_freq.to(torch.float64)
    length = 2.0 * math.pi / f
    s = (original / length - low) / (high - low)
    blended = (1.0 - s) * f / factor + s * f
    return torch.where(length < original / high, f, torch.where(length > original / low, f / factor, blended))


def ramp_frequencies(inv_freq: torch.Tensor, theta: float, factor: float, original: float, fast: float, slow: float):
    """Frequencies scaled over a ramp of the pairs' indices, and the factor that goes with them on cosine and sine.
    A frequency that makes t turns within ``original`` positions belongs to the (fractional) pair index n(t) = dims
    ln(original / (2 pi t)) / (2 ln theta); with lo = max(floor(n(fast)), 0) and hi = min(ceil(n(slow)), dims - 1), pair
    i gets the share r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) of the scaled frequency: f_i / factor * r_i +
    f_i (1 - r_i).  Cosine and sine are multiplied by 0.1 ln(factor) + 1."""
    f = inv_freq.to(torch.float64)
    dims = 2 * f.shape[0]

    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), dims - 1)
    share = torch.clamp((torch.arange(f.shape[0], dtype=torch.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * share + f * (1.0 - share), 0.1 * math.log(factor) + 1.0


def rotary_tables(positions: int, rot_dim: int, theta: float, angles: str = "float32", scaling=None, ramp=None):
    """``angles``: "float32" rounds the frequencies and the angles to 32-bit as
    the reference does; "float64" takes frequency i as theta^(-2i / rot_dim) and
    the angle as position x frequency in 64-bit, and rounds cosine and sine only.
    ``scaling``: (factor, low, high, original) of ``bend_frequencies``; ``ramp``: (factor, original, fast, slow) of
    ``ramp_frequencies``; both with 64-bit angles only."""
    half = rot_dim // 2
    if (scaling is not None or ramp is not None) and angles != "float64":
        raise InvalidInput("scaled frequencies are made with 64-bit angles")
    if scaling is not None and ramp is not None:
        raise InvalidInput("frequencies are bent by their wavelength or scaled over a ramp, not both")
    if angles == "float64":
        pair = torch.arange(half, dtype=torch.float64)
        inv_freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * pair / float(rot_dim))
        magnitude = 1.0
        if scaling is not None:
            inv_freq = bend_frequencies(inv_freq, *[float(value) for value in scaling])
        if ramp is not None:
            inv_freq, magnitude = ramp_frequencies(inv_freq, float(theta), *[float(value) for value in ramp])
        angle = torch.arange(positions, dtype=torch.float64)[:, None] * inv_freq[None, :]
        return (torch.cos(angle) * magnitude).to(torch.float32), (torch.sin(angle) * magnitude).to(torch.float32)
    pair = torch.arange(half, dtype=torch.float32)
    exponent = (2.0 * pair) / torch.tensor(float(rot_dim), dtype=torch.float32)  # 32-bit quotient
    theta32 = torch.tensor(theta, dtype=torch.float32).to(torch.float64)
    power = torch.pow(theta32, exponent.to(torch.float64)).to(torch.float32)
    inv_freq = torch.tensor(1.0, dtype=torch.float32) / power
    pos = torch.arange(positions, dtype=torch.float32)[:, None]
    angle = pos * inv_freq[None, :]  # 32-bit product
    angle64 = angle.to(torch.float64)
    return torch.cos(angle64).to(torch.float32), torch.sin(angle64).to(torch.float32)


class RotaryHalf(PositionEncoding):
    graph_safe = True
    pairing = "halves"  # channel i turns with channel i + rot_dim / 2

    def __init__(self, rot_dim: int, theta: float, max_positions: int = None, angles: str = "float32", scaling=None, ramp=None):
        """``max_positions`` None: the model names no last position; the tables
        are made as long as the engine's cache lets a sequence grow (``reach``).
        ``scaling``: (factor, low, high, original), frequencies bent by their
        wavelength (``bend_frequencies``); ``ramp``: (factor, original, fast,
        slow), frequencies scaled over a ramp of the pairs (``ramp_frequencies``)."""
        if rot_dim <= 0 or rot_dim % 2 != 0:
            raise InvalidInput(f"rotary dimension must be even and positive; got {rot_dim}")
        if angles not in ("float32", "float64"):
            raise InvalidInput(f"rotary angles are made in float32 or float64, got {angles!r}")
        self.rot_dim = int(rot_dim)
        self.theta = float(theta)
        self.max_positions = None if max_positions is None else int(max_positions)
        self.angles = angles
        self.scaling = None if scaling is None else tuple(float(value) for value in scaling)
        if self.scaling is not None and len(self.scaling) != 4:
            raise InvalidInput(f"bent frequencies take (factor, low, high, original); got {scaling!r}")
        self.ramp = None if ramp is None else tuple(float(value) for value in ramp)
        if self.ramp is not None and len(self.ramp) != 4:
            raise InvalidInput(f"frequencies scaled over a ramp take (factor, original, fast, slow); got {ramp!r}")
        self._tables = None
        self._device = None
        self._kept = []

    def bind(self, weights, rt):
        self._device = rt.device
        self._make(self.max_positions or 64)

    def _make(self, positions: int) -> None:
        cos, sin = rotary_tables(positions, self.rot_dim, self.theta, self.angles, self.scaling, self.ramp)
        self._tables = RotaryTables(cos.to(self._device).contiguous(), sin.to(self._device).contiguous(), self.rot_dim)

    def reach(self, positions: int) -> None:
        """Makes the tables cover ``positions`` positions, if the model sets no end of its own.  Called when an
        engine is made, before any step is captured: captured steps hold the tables' addresses."""
        if self.max_positions is None and self._tables is not None and self._tables.cos.shape[0] < positions:
            self._kept.append(self._tables)  # (steps captured by an earlier engine of the same model go on reading these)
            self._make(positions)

    def rotary(self):
        return self._tables


register_part("position", "rotary_half", RotaryHalf)


class RotaryPairs(RotaryHalf):
    """The same tables (angle = position x frequency i) for consumers that
    turn channel 2i with channel 2i + 1.  Which channels make a pair is the
    consuming kernel's business: it asks for the ``pairing`` it implements."""

    pairing = "neighbours"


register_part("position", "rotary_pairs", RotaryPairs)
