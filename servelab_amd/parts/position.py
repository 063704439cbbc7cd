"""Position encodings, as parameters of a mixer.

Rotary: inv_freq[j] = theta^(-2j/D) built in float32 as
``1 / theta ** (arange(0, D, 2) / D)`` (servelab/parallel/tp_model.py:94-96);
angles, cos and sin are float32; the rotation pairs (j, j + D/2)
(docs/architecture.md:69).  ``rotary_dim`` (the leading channels that are
rotated) and ``pairing`` go beyond the reference, whose heads turn whole and in
halves, and so do ``frequencies`` (the angle per position of every pair, given
from outside instead of theta^(-2j/D)) and ``magnitude`` (cos and sin are both
multiplied by it); two rules that stretch frequencies for contexts beyond a
trained length are functions here.
"""
import math

import torch

from .base import PositionEncoding, RotaryLayout, RotaryTables


class RotaryPosition(PositionEncoding):
    graph_safe = True

    kind = "rotary"

    def __init__(self, head_dim: int, theta: float, rotary_dim=None, pairing: str = "half",
                 frequencies=None, magnitude: float = 1.0):
        self.head_dim = int(head_dim)
        self.rotary_dim = self.head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"the rotated width must be even and within head_dim {head_dim}, "
                             f"is {self.rotary_dim}")
        self.theta = float(theta)
        self.pairing = pairing
        self.frequencies = None if frequencies is None else tuple(float(f) for f in frequencies)
        if self.frequencies is not None and len(self.frequencies) != self.rotary_dim // 2:
            raise ValueError(f"{self.rotary_dim // 2} pairs turn, {len(self.frequencies)} frequencies are given")
        self.magnitude = float(magnitude)

    def layout(self):
        return RotaryLayout(self.rotary_dim, self.pairing)

    def load(self, tensors, rt):
        self.rt = rt
        if self.frequencies is not None:
            inv = torch.tensor(self.frequencies, dtype=torch.float64).to(torch.float32)
        else:
            inv = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32)
                                        / self.rotary_dim))
        self.inv_freq = inv.to(rt.device)

    def tables(self, batch, shared):
        key = ("rotary", self.rotary_dim, self.theta, self.frequencies, self.magnitude)
        if key not in shared:
            if self.magnitude != 1.0:
                tables = self.rt.ops.rope_tables(batch.positions, self.inv_freq, self.magnitude)
            else:
                tables = self.rt.ops.rope_tables(batch.positions, self.inv_freq)
            shared[key] = RotaryTables(*tables)
        return shared[key]


def plain_frequencies(rotary_dim: int, theta: float):
    """theta^(-2j / rotary_dim) for the rotary_dim / 2 pairs, in double precision."""
    return [theta ** (-2.0 * j / rotary_dim) for j in range(rotary_dim // 2)]


def blended_frequencies(rotary_dim: int, theta: float, factor: float, original: float, fast: float, slow: float):
    """Frequencies that go over from f (pairs that turn more than ``fast`` times within ``original``
    positions) to f / factor (pairs that turn fewer than ``slow`` times), linearly in the pair's
    number between the two: with n(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta), lo =
    max(floor(n(fast)), 0), hi = min(ceil(n(slow)), rotary_dim - 1) and ramp_j = clamp((j - lo) /
    max(hi - lo, 0.001), 0, 1), the result is f_j / factor ramp_j + f_j (1 - ramp_j).  The
    magnitude that goes with it is 0.1 ln(factor) + 1 (``blended_magnitude``)."""
    def pair_of(turns):
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), rotary_dim - 1)
    out = []
    for j, f in enumerate(plain_frequencies(rotary_dim, theta)):
        ramp = min(max((j - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out


def blended_magnitude(factor: float) -> float:
    return 0.1 * math.log(factor) + 1.0


def wavelength_frequencies(rotary_dim: int, theta: float, factor: float, low: float, high: float, original: float):
    """Frequencies stretched by wavelength l = 2 pi / f: kept where l < original / high, divided
    by ``factor`` where l > original / low, and between the two (1 - s) f / factor + s f with
    s = (original / l - low) / (high - low)."""
    out = []
    for f in plain_frequencies(rotary_dim, theta):
        wave = 2.0 * math.pi / f
        if wave < original / high:
            out.append(f)
        elif wave > original / low:
            out.append(f / factor)
        else:
            s = (original / wave - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


class NoPosition(PositionEncoding):
    graph_safe = True

    kind = "none"

    def tables(self, batch, shared):
        return None
