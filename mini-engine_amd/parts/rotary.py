"""Rotary position encoding part (pairs of halves, or of neighbours: the table is the same, the kernels that
rotate are told the pairing).

``inv_freq[j] = 1 / theta ** (2j / rotary_dim)`` in float32, exactly the expression of the
reference (``src/mini_engine/model.py:75``); the angle ``position * inv_freq[j]`` and its cosine and
sine are computed in float32 (``model.py:79-90``) by a kernel, once per position, into a table
``[positions, 2, rotary_dim / 2]`` that the mixer's kernels read.
"""

from __future__ import annotations

import torch

from .base import POSITION_ENCODINGS, PositionEncoding


class Rotary(PositionEncoding):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        rd = int(spec.rotary_dim)
        if rd <= 0 or rd % 2:
            raise ValueError(f"rotary_dim must be a positive even number, got {rd}")
        self.rotary_dim = rd
        self.pairing = getattr(spec, "pairing", "halves")
        if self.pairing not in PAIRINGS:
            raise ValueError(f"a rotation pairs {sorted(PAIRINGS)}, got {self.pairing!r}")
        self.pairing_code = PAIRINGS[self.pairing]
        self.angles = getattr(spec, "angles", "float32")
        if self.angles not in ("float32", "float64"):
            raise ValueError(f"angles are worked out in float32 or float64, got {self.angles!r}")
        self.theta = float(spec.theta)
        inv_freq = 1.0 / (float(spec.theta) ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd))
        self.inv_freq = inv_freq.to(device)

        self._table: torch.Tensor | None = None
        self._retired: list[torch.Tensor] = []

    def tables(self, num_positions: int = 1) -> torch.Tensor:
        """The cos/sin table for positions ``0 .. num_positions - 1`` (grown in powers of two; never
        inside a graph capture, where the engine has sized it beforehand)."""
        if self._table is None or self._table.shape[0] < num_positions:
            from ..ops import kernels as K

            size = 256
            while size < num_positions:
                size *= 2
            if self._table is not None:
                self._retired.append(self._table)  # a captured graph may still read the smaller table
            if self.angles == "float64":  # position times frequency, cosine and sine in double; rounded once
                j = torch.arange(0, self.rotary_dim // 2, dtype=torch.float64, device=self.inv_freq.device)
                freq = torch.exp(-(2.0 * j / self.rotary_dim) * torch.log(torch.tensor(self.theta, dtype=torch.float64)))
                ang = torch.arange(size, dtype=torch.float64, device=freq.device)[:, None] * freq[None, :]
                self._table = torch.stack((torch.cos(ang), torch.sin(ang)), dim=1).to(torch.float32).contiguous()
            else:
                self._table = K.rope_table(self.inv_freq, size)
        return self._table


class YarnRotary(PositionEncoding):
    """Rotation of pairs of halves whose slow pairs are stretched by a factor, the fast ones left alone and those between
    blended (the spec says how); cosines and sines carry the encoding's multiplier. The table is worked out in double
    precision on the host and rounded once."""

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        import math

        rd, base = int(spec.rotary_dim), float(spec.theta)
        if rd <= 0 or rd % 2:
            raise ValueError(f"rotary_dim must be a positive even number, got {rd}")
        if getattr(spec, "pairing", "halves") != "halves":
            raise ValueError("the stretched rotation pairs halves")
        factor, original = float(spec.factor), float(spec.original)
        if not (factor > 0.0 and original > 0.0 and float(spec.fast) > 0.0 and float(spec.slow) > 0.0 and base > 1.0):
            raise ValueError("factor, original, fast and slow must be positive and the base above 1")
        self.rotary_dim, self.pairing, self.pairing_code = rd, "halves", 0
        j = torch.arange(rd // 2, dtype=torch.float64)
        freq = torch.exp(-(2.0 * j / rd) * math.log(base))

        def pair_of(turns: float) -> float:
            return rd * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(pair_of(float(spec.fast))), 0)
        hi = min(math.ceil(pair_of(float(spec.slow))), rd - 1)
        ramp = ((j - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        self.freq = freq / factor * ramp + freq * (1.0 - ramp)
        self.multiplier = 0.1 * math.log(factor) + 1.0
        self._table: torch.Tensor | None = None
        self._retired: list[torch.Tensor] = []

    def tables(self, num_positions: int = 1) -> torch.Tensor:
        if self._table is None or self._table.shape[0] < num_positions:
            size = 256
            while size < num_positions:
                size *= 2
            if self._table is not None:
                self._retired.append(self._table)  # a captured graph may still read the smaller table
            ang = torch.arange(size, dtype=torch.float64)[:, None] * self.freq[None, :]
            table = torch.stack((torch.cos(ang), torch.sin(ang)), dim=1) * self.multiplier
            self._table = table.to(torch.float32).contiguous().to(self.device)
        return self._table


class ScaledRotary(PositionEncoding):
    """Rotation whose slow pairs are slowed by a factor, the fast ones left alone and those between blended by their wavelength
    (the spec says how). Nothing multiplies the cosines and sines. The table is worked out in double precision on the host and
    rounded once."""

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        import math

        rd, base = int(spec.rotary_dim), float(spec.theta)
        if rd <= 0 or rd % 2:
            raise ValueError(f"rotary_dim must be a positive even number, got {rd}")
        self.pairing = getattr(spec, "pairing", "halves")
        if self.pairing not in PAIRINGS:
            raise ValueError(f"a rotation pairs {sorted(PAIRINGS)}, got {self.pairing!r}")
        factor, low, high, original = float(spec.factor), float(spec.low), float(spec.high), float(spec.original)
        if not (factor > 0.0 and original > 0.0 and low > 0.0 and high > low and base > 0.0):
            raise ValueError("factor, original and low must be positive, high above low")
        self.rotary_dim, self.pairing_code = rd, PAIRINGS[self.pairing]
        freq = []
        for j in range(rd // 2):
            f = base ** (-2.0 * j / rd)
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                freq.append(f)
            elif wavelength > original / low:
                freq.append(f / factor)
            else:
                t = (original / wavelength - low) / (high - low)
                freq.append((1.0 - t) * f / factor + t * f)
        self.freq = torch.tensor(freq, dtype=torch.float64)
        self._table: torch.Tensor | None = None
        self._retired: list[torch.Tensor] = []

    def tables(self, num_positions: int = 1) -> torch.Tensor:
        if self._table is None or self._table.shape[0] < num_positions:
            size = 256
            while size < num_positions:
                size *= 2
            if self._table is not None:
                self._retired.append(self._table)  # a captured graph may still read the smaller table
            ang = torch.arange(size, dtype=torch.float64)[:, None] * self.freq[None, :]
            self._table = torch.stack((torch.cos(ang), torch.sin(ang)), dim=1).to(torch.float32).contiguous().to(self.device)
        return self._table


PAIRINGS = {"halves": 0, "neighbours": 1}

POSITION_ENCODINGS.register("rotary", Rotary)
POSITION_ENCODINGS.register("yarn_rotary", YarnRotary)
POSITION_ENCODINGS.register("scaled_rotary", ScaledRotary)
