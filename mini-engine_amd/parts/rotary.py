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


PAIRINGS = {"halves": 0, "neighbours": 1}

POSITION_ENCODINGS.register("rotary", Rotary)
