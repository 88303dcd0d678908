"""Rotary position encoding: the table of angles.

The reference builds it on the host (v1/tensortype/common.cpp:6-24):
inv_freq[i] = 1 / base^(2i/D) for i < D/2, the angle of position l is
l * inv_freq[i], and the table holds its cosine and sine as floats.  Dims i
and i + D/2 share an angle and form a rotated pair
(v1/tensortype/hip_kernels/rotary_embed.cpp:20-26); the rotation itself is
fused into the kernel that writes keys and values into their pages.

The reference rounds inv_freq and the angle to float before taking cosine
and sine, which costs about position * 1e-7 radians; here everything up to
the final cosine and sine is computed in double and rounded to float once.
The reference's table has 10000 rows (v1/models/qwen2-7b/inference_fp16.dag:38);
here it has as many as the longest sequence the engine is set up for.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

from .base import POSITIONS, Part, Runtime


def stretched_frequencies(inv: np.ndarray, dims: int, theta: float, factor: float, original: float, fast: float,
                          slow: float) -> Tuple[np.ndarray, float]:
    """Frequencies for contexts `factor` times longer than the `original` one that the model was trained on (the
    scheme known as YaRN): a pair that turns more than `fast` times within the original context keeps its frequency,
    one that turns fewer than `slow` times is slowed down by `factor`, and between the two a ramp that is linear in
    the pair's index mixes both.  The index at which a pair makes t turns is d(t) = dims ln(original / (2 pi t)) /
    (2 ln theta).  Returns the frequencies and the factor 0.1 ln(factor) + 1 that cosines and sines are multiplied by
    (it sharpens the scores that the longer context flattens)."""
    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), dims - 1)
    ramp = np.clip((np.arange(dims // 2, dtype=np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return inv / factor * ramp + inv * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotary_table(n_positions: int, dims: int, theta: float, scaling: Optional[dict] = None) -> Tuple[np.ndarray, np.ndarray]:
    """(cos, sin), float32 [n_positions, dims/2].  scaling: None, or the constants of `stretched_frequencies`
    (factor, original, fast, slow)."""
    i = np.arange(0, dims, 2, dtype=np.float64)
    inv = 1.0 / np.power(np.float64(theta), i / dims)
    mag = 1.0
    if scaling:
        inv, mag = stretched_frequencies(inv, dims, theta, float(scaling["factor"]), float(scaling["original"]),
                                         float(scaling["fast"]), float(scaling["slow"]))
    ang = np.arange(n_positions, dtype=np.float64)[:, None] * inv[None, :]
    return (np.cos(ang) * mag).astype(np.float32), (np.sin(ang) * mag).astype(np.float32)


@POSITIONS.register("rotary")
class RotaryEncoding(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, theta: float, dim: int, scaling: Optional[dict] = None):
        """dim: how many of a head's leading elements are rotated (the rest pass unchanged where the mixer's head is
        larger); scaling: None or {factor, original, fast, slow} (`stretched_frequencies`)."""
        if dim % 2 or dim <= 0:
            raise ValueError(f"rotary dims {dim} must be even and positive")
        self.rt = rt
        self.theta = float(theta)
        self.dim = int(dim)
        self.scaling = dict(scaling) if scaling else None
        if self.scaling:
            for key in ("factor", "original", "fast", "slow"):
                if key not in self.scaling or not float(self.scaling[key]) > 0:
                    raise ValueError(f"rotary scaling needs a positive '{key}'")
        self._tables: Optional[Tuple[torch.Tensor, torch.Tensor]] = None

    def rotary_tables(self, n_positions: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """fp32 cos and sin [>= n_positions, dim/2] on the device, for the fused kernel."""
        if self._tables is None or self._tables[0].shape[0] < n_positions:
            cos, sin = rotary_table(n_positions, self.dim, self.theta, self.scaling)
            self._tables = (torch.from_numpy(cos).to(self.rt.device), torch.from_numpy(sin).to(self.rt.device))
        return self._tables


@POSITIONS.register("none")
class NoPositionEncoding(Part):
    replayable = True

    """Queries and keys as they are."""

    def __init__(self, *, rt: Runtime):
        self.rt = rt
        self.dim = 0

    def rotary_tables(self, n_positions: int):
        return None

    def apply(self, q, k, positions):
        return q, k
