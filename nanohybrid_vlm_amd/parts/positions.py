"""Position encodings. A position encoding hands the mixer a table of rotation
angles (cosines and sines per position) or nothing; the mixer's kernel turns
queries and keys by it before they are used and stored. A token's position may
have several coordinates (``ModelSpec.position_axes``; a step carries them as
[axes, tokens]): an encoding over several axes also says, pair by pair, which
axis' coordinate looks up the pair's angle (``pair_axes``)."""
from __future__ import annotations

import torch

from .base import POSITION_ENCODINGS, Part


class PositionEncoding(Part):
    """What a mixer asks of its position encoding."""

    def rotation_table(self) -> torch.Tensor | None:
        """[max_position, rotary_dim] float32 (cosines | sines), or None: nothing is turned."""
        return None

    def pair_axes(self) -> torch.Tensor | None:
        """[rotary_dim / 2] int32: the position axis that turns each pair; None: all turn by the first axis."""
        return None

    def to(self, device):
        return self


@POSITION_ENCODINGS.register("rope")
class RotaryEmbedding(PositionEncoding):
    """nanovllm/layers/rotary_embedding.py:83-89: inv_freq_j = base^(-2j/rotary_dim),
    table[p] = [cos(p * inv_freq) | sin(p * inv_freq)] in float32. The rotation
    itself (first half against second half, rotary_embedding.py:6-14) is done by
    the mixer's kernel."""

    def __init__(self, rotary_dim: int, max_position: int, base: float, device=None):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim = rotary_dim
        self.max_position = max_position
        self.base = base
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
        t = torch.arange(max_position, dtype=torch.float32)
        freqs = torch.einsum("i,j->ij", t, inv_freq)
        self.table = torch.cat((freqs.cos(), freqs.sin()), dim=-1).contiguous()   # [max_position, rotary_dim]
        if device is not None:
            self.table = self.table.to(device)

    def rotation_table(self) -> torch.Tensor | None:
        return self.table

    def to(self, device):
        self.table = self.table.to(device)
        return self


@POSITION_ENCODINGS.register("none")
class NoPositions(PositionEncoding):
    """No position signal at all (attention then depends on order only through the mask)."""

    def __init__(self, max_position: int, device=None):
        self.max_position = max_position

    def rotation_table(self):
        return None

    def to(self, device):
        return self


@POSITION_ENCODINGS.register("rotary_frequencies")
class RotaryFrequencies(PositionEncoding):
    """Rotation given by its frequencies alone: pair i of the first ``rotary_dim`` entries of a head turns by
    position * f_i, f_i = base^(-2 i / rotary_dim) / scaling_factor (linear scaling: every frequency divided by one
    number). There is no table: the mixer's kernel takes the angle in float from the position, so no number of
    positions bounds the model. ``frequencies_for(size)`` gives the unscaled frequencies of the same base over
    another size (values that are turned over all their entries)."""

    def __init__(self, rotary_dim: int, base: float, max_position: int, scaling_factor: float | None = None, device=None):
        if rotary_dim % 2 or rotary_dim < 0:
            raise ValueError(f"rotary_dim must be even and not negative, got {rotary_dim}")
        if scaling_factor is not None and not scaling_factor > 0:
            raise ValueError(f"the scaling factor must be positive, got {scaling_factor}")
        self.rotary_dim, self.base, self.max_position, self.scaling_factor = rotary_dim, float(base), max_position, scaling_factor
        self.device = device
        self.freqs = self._frequencies(rotary_dim, scaling_factor)
        self._others: dict[int, torch.Tensor] = {}

    def _frequencies(self, size: int, factor) -> torch.Tensor:
        f = self.base ** (-2.0 * torch.arange(size // 2, dtype=torch.float64) / size)
        if factor is not None:
            f = f / factor
        f = f.to(torch.float32)
        return f.to(self.device) if self.device is not None else f

    def frequencies(self) -> torch.Tensor:
        """[rotary_dim / 2] float32."""
        return self.freqs

    def frequencies_for(self, size: int) -> torch.Tensor:
        if size not in self._others:
            self._others[size] = self._frequencies(size, None)
        return self._others[size]

    def to(self, device):
        self.device = device
        self.freqs = self.freqs.to(device)
        self._others = {n: f.to(device) for n, f in self._others.items()}
        return self


@POSITION_ENCODINGS.register("yarn_frequencies")
class YarnFrequencies(PositionEncoding):
    """Rotation given by frequencies that are scaled part by part (YaRN): with f_i = base^(-2 i / rotary_dim) and
        dim(t) = rotary_dim ln(original / (2 pi t)) / (2 ln base),  lo = max(floor(dim(fast)), 0),
        hi = min(ceil(dim(slow)), rotary_dim - 1),  ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    pair i turns by position * (f_i / factor * ramp_i + f_i (1 - ramp_i)), and cosines and sines are multiplied by
    ``gain()`` = 0.1 ln(factor) + 1. Without ``factor`` the frequencies are the plain ones and the gain is 1. The
    frequencies are kept in float64: the kernels take the angle in double before they take its sine and cosine."""

    def __init__(self, rotary_dim: int, base: float, max_position: int, factor: float | None = None,
                 original: float | None = None, fast: float | None = None, slow: float | None = None, device=None):
        if rotary_dim % 2 or rotary_dim < 0:
            raise ValueError(f"rotary_dim must be even and not negative, got {rotary_dim}")
        self.rotary_dim, self.base, self.max_position = rotary_dim, float(base), max_position
        self.factor = None if factor is None else float(factor)
        i = torch.arange(rotary_dim // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / max(rotary_dim, 1))
        self._gain = 1.0
        if self.factor is not None:
            if not self.factor > 0 or None in (original, fast, slow):
                raise ValueError("scaled frequencies need a positive factor, and original, fast and slow")
            import math

            def dim_of(turns: float) -> float:
                return rotary_dim * math.log(original / (2 * math.pi * turns)) / (2 * math.log(self.base))

            lo = max(math.floor(dim_of(fast)), 0)
            hi = min(math.ceil(dim_of(slow)), rotary_dim - 1)
            ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
            f = f / self.factor * ramp + f * (1 - ramp)
            self._gain = 0.1 * math.log(self.factor) + 1.0
        self.freqs = f if device is None else f.to(device)

    def frequencies(self) -> torch.Tensor:
        """[rotary_dim / 2] float64."""
        return self.freqs

    def gain(self) -> float:
        return self._gain

    def to(self, device):
        self.freqs = self.freqs.to(device)
        return self
