"""Rotary position encoding, half-split pairing.

Tables as the reference builds them (src/utils/constant_table.hpp:28-41):
``freq_j = theta^(-j / (rot/2))`` and ``cos/sin(p * freq_j)`` with ``p * freq_j``
formed in float32.  Pair (j, j + rot/2) of each head vector is rotated
(src/backends/cpu/cpu_operator.cpp:401-407).  ``rotary_dim`` < head_dim leaves
the remaining dims as they are (the reference always rotates the whole head).
"""
from __future__ import annotations

import math

import torch

from .base import PositionEncoding


class RotaryEmbedding(PositionEncoding):
    def __init__(self, head_dim: int, theta: float, rotary_dim: int = None, scaling: dict = None, interleaved: bool = False):
        """``scaling``: None, or YaRN's numbers {factor, original, fast, slow}: frequencies whose wavelength is long
        against ``original`` positions are divided by ``factor``, those with more than ``fast`` turns in ``original``
        positions stay, with a linear ramp over the pair index between the two; cos and sin are multiplied by
        0.1 ln(factor) + 1.  ``interleaved``: pair j is dims (2 j, 2 j + 1) instead of (j, j + rotary_dim / 2); the frequencies
        are the same, and the mixers that form the angles in their kernels (``frequencies()``) read the flag; there are no
        tables for it."""
        self.interleaved = bool(interleaved)
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= head_dim):
            raise ValueError("rotary_dim must be even and at most head_dim")
        self.scaling = dict(scaling) if scaling else None
        #: a scaling with the keys {factor, low, high, original} goes by wavelength: a frequency whose wavelength is
        #: shorter than original / high stays, one longer than original / low is divided by factor, and between the two
        #: the divided and the plain frequency are blended linearly in original / wavelength (no factor on cos and sin)
        self.by_wavelength = bool(self.scaling) and "low" in self.scaling and "high" in self.scaling
        self.cos = self.sin = None
        self._freq = None

    def frequency_values(self):
        """(float64 frequencies of the rotary_dim / 2 pairs, factor on cos and sin)."""
        dims, half = self.rotary_dim, self.rotary_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        f = torch.tensor(self.theta, dtype=torch.float64) ** (-2.0 * i / dims)
        if self.scaling is None:
            return f, 1.0
        factor, original = float(self.scaling["factor"]), float(self.scaling["original"])
        if self.by_wavelength:
            low, high = float(self.scaling["low"]), float(self.scaling["high"])
            wavelength = 2.0 * math.pi / f
            blend = torch.clamp((original / wavelength - low) / (high - low), 0.0, 1.0) if high != low else (wavelength < original / high).double()
            mixed = (1.0 - blend) * f / factor + blend * f
            out = torch.where(wavelength < original / high, f, torch.where(wavelength > original / low, f / factor, mixed))
            return out, 1.0

        def pair_of(turns: float) -> float:
            # the (fractional) pair index whose frequency makes ``turns`` turns in ``original`` positions
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(pair_of(float(self.scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(self.scaling["slow"]))), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0

    def frequencies(self):
        """(float32 frequencies on the device, factor on cos and sin, rotated dims) for kernels that form the angles
        themselves (position * frequency in float32): no table, no limit on positions."""
        return self._freq, self._mag, self.rotary_dim

    def prepare(self, device, max_positions: int) -> None:
        f, self._mag = self.frequency_values()
        self._freq = f.to(torch.float32).to(device)
        if self.scaling is not None or not max_positions or self.interleaved:
            return                   # tables are for the mixers that look angles up; a scaled rotation is formed in the kernel
        half = self.rotary_dim // 2
        # the exponent and the angle are formed in float32, as in the reference; the table is built
        # on the host once and then lies on the device
        j = torch.arange(half, dtype=torch.float32)
        freq = torch.pow(torch.tensor(self.theta, dtype=torch.float32), -j / float(half))
        p = torch.arange(max_positions, dtype=torch.float32)
        ang = p[:, None] * freq[None, :]
        self.cos = torch.cos(ang).contiguous().to(device)
        self.sin = torch.sin(ang).contiguous().to(device)

    def capturable(self, batch):
        return True

    def rotary(self):
        return self.cos, self.sin, self.rotary_dim
