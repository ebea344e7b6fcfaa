"""Rotary position encoding, split-half pairing.

freq[i] = 1 / theta^(2i/rotary) for i < rotary/2, angle = position * freq[i]
(crates/beholdd-model/src/qwen3moe/forward.rs:1844-1868): powers, angles, cosines and sines are
computed in float64 and stored as float32, one row per position, once per model, like the
reference's device path (crates/beholdd-model/src/recorded_attention.rs:438-457).  The pairs
are (x[i], x[i + rotary/2]) (crates/beholdd-kernel/src/vecops.rs:186-197); the attention
kernel applies them.
"""

from __future__ import annotations

import math

import numpy as np
import torch

from .base import POSITION_ENCODINGS


class RotaryEncoding:
    def __init__(self, rotary_dim: int, theta: float, max_position: int):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ValueError(f"rotary width must be positive and even, got {rotary_dim}")
        if not (theta > 0.0):
            raise ValueError(f"RoPE base must be positive and finite, got {theta}")
        self.rotary_dim, self.theta, self.max_position = int(rotary_dim), float(theta), int(max_position)
        self._tables = None

    def tensor_specs(self):
        return []

    def load(self, get):
        pass

    def build_tables(self, device):
        half = self.rotary_dim // 2
        freqs = np.array([1.0 / (self.theta ** ((2 * i) / self.rotary_dim)) for i in range(half)], dtype=np.float64)
        angles = np.arange(self.max_position, dtype=np.float64)[:, None] * freqs[None, :]
        cos = torch.from_numpy(np.cos(angles).astype(np.float32)).to(device).contiguous()
        sin = torch.from_numpy(np.sin(angles).astype(np.float32)).to(device).contiguous()
        self._tables = (cos, sin)

    def tables(self):
        if self._tables is None:
            raise RuntimeError("rotary tables were not built; call build_tables(device) after loading")
        return self._tables


class RotaryFrequencies:
    """The same rotation without a table: freq[i] = base^(-2i/dims) (computed in float64, kept as float32), and the
    kernel that rotates forms the angle position * freq[i] as a float32 product and takes its cosine and sine.
    There is no longest position; `dims` of a vector's dimensions are turned, dimension i with i + dims/2, or, where the
    mixer says so, the neighbours 2i and 2i + 1.

    `stretch` = (factor, original, fast, slow) slows the slow pairs down for contexts longer than `original` positions
    (YaRN: B. Peng, J. Quesnelle, H. Fan, E. Shippole, "YaRN: Efficient Context Window Extension of Large Language
    Models").  With d(t) = dims ln(original / (2 pi t)) / (2 ln base), the pair whose wave turns t times within
    `original` positions, lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1):  freq_i <- freq_i / factor * ramp_i + freq_i (1 - ramp_i),
    and every cosine and sine is multiplied by `magnitude` = 0.1 ln(factor) + 1 (1.0 without a stretch)."""

    def __init__(self, dims: int, base: float, stretch=None):
        if dims <= 0 or dims % 2:
            raise ValueError(f"rotary width must be positive and even, got {dims}")
        if not (base > 0.0):
            raise ValueError(f"rotation base must be positive and finite, got {base}")
        self.dims, self.base = int(dims), float(base)
        self.stretch, self.magnitude = None, 1.0
        if stretch is not None:
            factor, original, fast, slow = (float(value) for value in stretch)
            if not (factor > 0.0 and original > 0.0 and fast > 0.0 and slow > 0.0) or base == 1.0:
                raise ValueError(f"a stretch needs a positive factor, length and turn counts and a base other than 1, got {stretch!r}")
            self.stretch = (factor, original, fast, slow)
            self.magnitude = 0.1 * math.log(factor) + 1.0
        self._frequencies = None

    def values(self) -> np.ndarray:
        """The frequencies in float64, one per pair."""
        plain = np.array([self.base ** (-2.0 * i / self.dims) for i in range(self.dims // 2)], dtype=np.float64)
        if self.stretch is None:
            return plain
        factor, original, fast, slow = self.stretch

        def pair_of(turns: float) -> float:
            return self.dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

        low = max(math.floor(pair_of(fast)), 0)
        high = min(math.ceil(pair_of(slow)), self.dims - 1)
        ramp = np.clip((np.arange(self.dims // 2, dtype=np.float64) - low) / max(high - low, 0.001), 0.0, 1.0)
        return plain / factor * ramp + plain * (1.0 - ramp)

    def frequencies(self, device) -> torch.Tensor:
        if self._frequencies is None or self._frequencies.device != torch.device(device):
            self._frequencies = torch.from_numpy(self.values().astype(np.float32)).to(device).contiguous()
        return self._frequencies


class NoPositionEncoding:
    """For mixers whose order information comes from elsewhere (or nowhere)."""

    def tensor_specs(self):
        return []

    def load(self, get):
        pass

    def build_tables(self, device):
        pass

    def tables(self):
        return (None, None)


@POSITION_ENCODINGS.register("rope")
def _build_rope(config, shared):
    return RotaryEncoding(config.head_dim, config.rope_theta, config.max_position)


@POSITION_ENCODINGS.register("none")
def _build_none(config, shared):
    return NoPositionEncoding()
