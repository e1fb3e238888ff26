"""Rotary position encoding: inv_freq[i] = theta^(-2i/D); the angle of pair (j, j + D/2)
at position p is p * inv_freq[j] (worker/src/inference/qwen2/model.py:93-117). The table
of inverse frequencies is all this part owns: angle, cosine and sine are computed in
float32 inside the kernel that also writes the cache."""

from __future__ import annotations

import math

import torch

from .base import PositionEncoding, register_part


_SHARED = {}


class RotaryPosition(PositionEncoding):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.params["dim"])
        self.theta = float(spec.params["theta"])
        if self.dim < 2 or self.dim % 2:
            raise ValueError("rotary dimension must be even")
        # the reference builds the exponent as arange(0, D, 2).float() / D in float32 (model.py:98)
        exponent = torch.arange(0, self.dim, 2, dtype=torch.float32) / self.dim
        self.inv_freq = 1.0 / (self.theta ** exponent)

    def to_device(self, device) -> None:
        # layers with the same rotation share one table, so that what a step derives from it
        # (cosines and sines of the step's positions) is derived once
        key = (self.dim, self.theta, str(device))
        if key not in _SHARED:
            _SHARED[key] = self.inv_freq.to(device)
        self.inv_freq = _SHARED[key]

    def rotary(self):
        return self.inv_freq


class ScaledRotaryPosition(PositionEncoding):
    """Rotation of the first `dims` dimensions of a head, with the frequencies stretched for contexts beyond the
    trained one ("YaRN"): f_i = base^(-2i/dims); with `scaling` = {factor, original, fast, slow}, the dimension at
    which a frequency makes `turns` turns over `original` positions is dim(turns) = dims ln(original / (2 pi turns))
    / (2 ln base); lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), dims - 1), ramp_i = clamp((i - lo) /
    max(hi - lo, 0.001), 0, 1), and the frequency becomes f_i / factor * ramp_i + f_i * (1 - ramp_i): fast
    dimensions keep theirs, slow ones are divided by the factor. Cosine and sine are both multiplied by
    0.1 ln(factor) + 1 (`rotary_magnitude`). Without `scaling`: plain rotation of `dims` dimensions."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        p = spec.params
        self.dims = int(p["dims"])
        self.base = float(p["base"])
        if self.dims < 2 or self.dims % 2:
            raise ValueError("rotary dimension must be even")
        half = self.dims // 2
        freq = torch.tensor([self.base ** (-2.0 * i / self.dims) for i in range(half)], dtype=torch.float64)
        self.magnitude = 1.0
        scaling = p.get("scaling")
        if scaling:
            factor, original = float(scaling["factor"]), float(scaling["original"])
            fast, slow = float(scaling["fast"]), float(scaling["slow"])

            def dim_of(turns: float) -> float:
                return self.dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(self.base))

            lo = max(math.floor(dim_of(fast)), 0)
            hi = min(math.ceil(dim_of(slow)), self.dims - 1)
            ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)],
                                dtype=torch.float64)
            freq = freq / factor * ramp + freq * (1 - ramp)
            self.magnitude = 0.1 * math.log(factor) + 1.0
        self.inv_freq = freq.to(torch.float32)
        self._key = (self.dims, self.base, repr(sorted(scaling.items())) if scaling else None)

    def to_device(self, device) -> None:
        key = ("scaled",) + self._key + (str(device),)
        if key not in _SHARED:
            _SHARED[key] = self.inv_freq.to(device)
        self.inv_freq = _SHARED[key]

    def rotary(self):
        return self.inv_freq

    def rotary_magnitude(self) -> float:
        return self.magnitude


class BandedRotaryPosition(PositionEncoding):
    """Rotation of the first `dims` dimensions of a head, with the frequencies scaled by bands of wavelength:
    f_i = base^(-2i/dims), wavelength l_i = 2 pi / f_i. With `scaling` = {factor, low, high, original}: a frequency
    whose wavelength is shorter than original / high stays; one whose wavelength is longer than original / low
    becomes f_i / factor; between the two, with s = (original / l_i - low) / (high - low), it becomes
    (1 - s) f_i / factor + s f_i. Computed in float64 and rounded once. Without `scaling`: plain rotation."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        p = spec.params
        self.dims = int(p["dims"])
        self.base = float(p["base"])
        if self.dims < 2 or self.dims % 2:
            raise ValueError("rotary dimension must be even")
        scaling = p.get("scaling")
        freqs = []
        for i in range(self.dims // 2):
            f = self.base ** (-2.0 * i / self.dims)
            if scaling:
                factor, original = float(scaling["factor"]), float(scaling["original"])
                low, high = float(scaling["low"]), float(scaling["high"])
                length = 2 * math.pi / f
                if length > original / low:
                    f = f / factor
                elif not length < original / high:
                    s = (original / length - low) / (high - low)
                    f = (1 - s) * f / factor + s * f
            freqs.append(f)
        self.inv_freq = torch.tensor(freqs, dtype=torch.float64).to(torch.float32)
        self._key = (self.dims, self.base, repr(sorted(scaling.items())) if scaling else None)

    def to_device(self, device) -> None:
        key = ("banded",) + self._key + (str(device),)
        if key not in _SHARED:
            _SHARED[key] = self.inv_freq.to(device)
        self.inv_freq = _SHARED[key]

    def rotary(self):
        return self.inv_freq


class NoPosition(PositionEncoding):
    """For mixers whose order comes from elsewhere (a state, a learned table)."""


register_part("position", "rope", RotaryPosition)
register_part("position", "rope_scaled", ScaledRotaryPosition)
register_part("position", "rope_banded", BandedRotaryPosition)
register_part("position", "none", NoPosition)
