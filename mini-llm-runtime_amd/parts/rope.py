"""Rotary position encoding over the whole head, split-half pairing (j, j + dim/2):
freq_j = base^(-2j/dim), angle = position * freq_j held in 32-bit, as the reference computes it
(src/minillm/runtime.cpp:231-241, table form src/minillm/cuda/storage.cpp:261-287).  The table
[max_positions, dim] holds cos in its first half and sin in its second.  The part hands the attention
part a `Rotation`: this table, the rotated width (here the whole head) and the pairing (here split-half)."""
from __future__ import annotations

import numpy as np
import torch

from .registry import Rotation, register_part


@register_part("position", "rope_split_half")
class RopeSplitHalf:
    def __init__(self, spec):
        self.dim, self.base = spec.dim, float(spec.base)
        self._tables = {}

    def rotation(self, max_positions, device):
        """The whole head in split-half pairs."""
        return Rotation(self.rotation_table(max_positions, device), self.dim, interleaved=False)

    def rotation_table(self, max_positions, device):
        key = (max_positions, str(device))
        if key not in self._tables:
            half = self.dim // 2
            j = np.arange(half, dtype=np.float64)
            freq = np.power(self.base, -2.0 * j / self.dim).astype(np.float32)
            angle = (np.arange(max_positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32)
            table = np.concatenate([np.cos(angle.astype(np.float64)), np.sin(angle.astype(np.float64))],
                                   axis=1).astype(np.float32)
            self._tables[key] = torch.from_numpy(table).to(device)
        return self._tables[key]


@register_part("position", "rope")
class Rope:
    """Rotary positions over the first `dim` channels of a head, in split-half pairs (j, j + dim/2) or interleaved
    ones (2j, 2j + 1), the frequencies base^(-2j/dim) optionally stretched for long contexts
    (`FrequencyStretch`: a ramp between the pairs that turn fast, which keep their frequency, and those that turn
    slowly, whose frequency is divided by `factor`; cosines and sines are multiplied by 0.1 ln(factor) + 1).
    Frequencies and angles are 32-bit; the table holds cos in its first half and sin in its second."""

    def __init__(self, spec):
        self.dim, self.base = spec.dim, float(spec.base)
        self.interleaved, self.stretch = bool(spec.interleaved), spec.stretch
        if self.dim % 2 != 0 or self.dim < 2:
            raise ValueError(f"a rotation turns an even number of channels, not {self.dim}")
        self._tables = {}

    def frequencies(self):
        """(float32 frequency of every pair, the factor on cosines and sines)."""
        half = self.dim // 2
        j = np.arange(half, dtype=np.float64)
        freq = np.power(self.base, -2.0 * j / self.dim)
        amplitude = 1.0
        st = self.stretch
        if st is not None:
            place = lambda turns: self.dim * np.log(st.original / (2.0 * np.pi * turns)) / (2.0 * np.log(self.base))
            lo = max(np.floor(place(st.fast)), 0.0)
            hi = min(np.ceil(place(st.slow)), self.dim - 1.0)
            ramp = np.clip((j - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            freq = freq / st.factor * ramp + freq * (1.0 - ramp)
            amplitude = 0.1 * np.log(st.factor) + 1.0
        return freq.astype(np.float32), float(amplitude)

    def rotation(self, max_positions, device):
        key = (max_positions, str(device))
        if key not in self._tables:
            freq, amplitude = self.frequencies()
            angle = (np.arange(max_positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32)
            table = np.concatenate([np.cos(angle.astype(np.float64)), np.sin(angle.astype(np.float64))], axis=1) * amplitude
            self._tables[key] = torch.from_numpy(table.astype(np.float32)).to(device)
        return Rotation(self._tables[key], self.dim, interleaved=self.interleaved)
