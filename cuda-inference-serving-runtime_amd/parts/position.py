"""Position encodings applied to queries and keys before keys are cached.

RotaryEmbedding is the split-half rotary embedding: coordinate pair
(i, i + rot/2) of a head turns by pos * theta^(-2i/rot)
(reference: runtime/reference.py:9-15, kernels/ops.cu:21-33).  Angles are
computed on the host in float64 and stored as float cosine/sine tables, so the
kernels do no transcendental arithmetic.  NoPosition turns nothing.

What a position part gives a mixer: `tables() -> (cos, sin)` float
[max_positions, pairs], and `pairing`: which two coordinates of a head pair i
is, "split_half" (i, i + pairs) or "interleaved" (2i, 2i + 1).  A part without
the attribute is split-half.
"""
import math

import numpy as np
import torch

from .base import Part, register_part


class RotaryEmbedding(Part):
    def __init__(self, head_dim, theta, max_positions, rotary_dim=None, pairing="split_half", scaling=None):
        """`scaling` (YaRN): {"factor", "original", "fast", "slow"}.  With turns(t) the index of the pair that makes t
        turns over `original` positions, rotary_dim * ln(original / (2 pi t)) / (2 ln theta), pairs up to
        lo = max(floor(turns(fast)), 0) keep their frequency, pairs from hi = min(ceil(turns(slow)), rotary_dim - 1) on
        turn `factor` times slower, those between go over linearly; cosines and sines are multiplied by
        0.1 ln(factor) + 1.
        `scaling` by wavelength (the rule of Llama 3.1): {"factor", "low", "high", "original"}.  A pair whose wavelength
        2 pi / f is shorter than original / high keeps its frequency, one longer than original / low turns `factor`
        times slower, one between goes over linearly in s = (original / wavelength - low) / (high - low):
        (1 - s) f / factor + s f; cosines and sines keep their size.
        `scaling` linear: {"factor"} alone: every frequency is divided by it (positions shrink), sizes kept."""
        if pairing not in ("split_half", "interleaved"):
            raise ValueError(f"pairing {pairing!r} is neither split_half nor interleaved")
        self.pairing = pairing
        self.head_dim, self.theta, self.max_positions = head_dim, float(theta), int(max_positions)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary size {self.rotary_dim} must be even and at most the head size {head_dim}")
        self.scaling = self.by_wavelength = self.linear = None
        if scaling is not None and set(scaling) == {"factor"}:
            self.linear = float(scaling["factor"])
            if not self.linear > 0:
                raise ValueError("linear rotary scaling: the factor must be positive")
        elif scaling is not None and ("low" in scaling or "high" in scaling):
            missing = [k for k in ("factor", "low", "high", "original") if k not in scaling]
            if missing:
                raise ValueError(f"rotary scaling by wavelength lacks {missing}")
            self.by_wavelength = {k: float(scaling[k]) for k in ("factor", "low", "high", "original")}
            w = self.by_wavelength
            if not (w["factor"] > 0 and w["original"] > 0 and 0 < w["low"] < w["high"]):
                raise ValueError("rotary scaling by wavelength: factor and original positive, 0 < low < high")
        elif scaling is not None:
            missing = [k for k in ("factor", "original", "fast", "slow") if k not in scaling]
            if missing:
                raise ValueError(f"rotary scaling lacks {missing}")
            self.scaling = {k: float(scaling[k]) for k in ("factor", "original", "fast", "slow")}
            if not (self.scaling["factor"] > 0 and self.scaling["original"] > 0 and self.scaling["fast"] > 0 and self.scaling["slow"] > 0):
                raise ValueError("rotary scaling: factor, original, fast and slow must be positive")
        self._tables = None

    def frequencies(self):
        """Radians a position of each pair (float64 [rotary_dim / 2])."""
        half, dims = self.rotary_dim // 2, self.rotary_dim
        index = np.arange(half, dtype=np.float64)
        freq = np.float64(self.theta) ** (-index * 2.0 / dims)
        if self.linear is not None:
            return freq / self.linear
        if self.by_wavelength is not None:
            w = self.by_wavelength
            wavelength = 2.0 * math.pi / freq
            share = np.clip((w["original"] / wavelength - w["low"]) / (w["high"] - w["low"]), 0.0, 1.0)
            between = (1.0 - share) * freq / w["factor"] + share * freq
            return np.where(wavelength < w["original"] / w["high"], freq,
                            np.where(wavelength > w["original"] / w["low"], freq / w["factor"], between))
        s = self.scaling
        if s is None:
            return freq

        def turns(t):
            return dims * math.log(s["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(self.theta))

        lo, hi = max(math.floor(turns(s["fast"])), 0), min(math.ceil(turns(s["slow"])), dims - 1)
        ramp = np.clip((index - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return freq / s["factor"] * ramp + freq * (1.0 - ramp)

    def magnitude(self):
        """What cosines and sines are multiplied by (1 without scaling)."""
        return 1.0 if self.scaling is None else 0.1 * math.log(self.scaling["factor"]) + 1.0

    def angles(self):
        return np.arange(self.max_positions, dtype=np.float64)[:, None] * self.frequencies()[None, :]

    def prepare(self, device, dtype):
        if self._tables is not None and self._tables[0].device == torch.device(device):
            return                      # one part may serve many layers: its tables are built once
        a, m = self.angles(), self.magnitude()
        self._tables = (torch.from_numpy((np.cos(a) * m).astype(np.float32)).to(device).contiguous(),
                        torch.from_numpy((np.sin(a) * m).astype(np.float32)).to(device).contiguous())

    def tables(self):
        return self._tables


class NoPosition(Part):
    """Identity: a one-pair table with angle zero."""
    pairing = "split_half"

    def __init__(self, head_dim, max_positions=1, **_):
        self.head_dim, self.max_positions = head_dim, int(max_positions)
        self._tables = None

    def prepare(self, device, dtype):
        if self._tables is not None and self._tables[0].device == torch.device(device):
            return
        self._tables = (torch.ones(self.max_positions, 1, dtype=torch.float32, device=device),
                        torch.zeros(self.max_positions, 1, dtype=torch.float32, device=device))

    def tables(self):
        return self._tables


register_part("position", "rotary", RotaryEmbedding)
register_part("position", "none", NoPosition)
