"""Rotary position encoding with half-split pairs (i, i + head_dim / 2)
(simply/utils/position_encoding.py:55-110)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import POSITION_ENCODINGS
from .base import PositionEncoding


@POSITION_ENCODINGS.register("rope")
class RoPE(PositionEncoding):
    def __init__(self, head_dim: int, base: float, scale_factor: float = 1.0, min_timescale: float = 1.0):
        if head_dim % 2:
            raise ValueError(f"rope: head_dim {head_dim} must be even")
        self.head_dim = int(head_dim)
        self.base = float(base)
        self.scale_factor = float(scale_factor)
        self.min_timescale = float(min_timescale)
        self._table: torch.Tensor | None = None

    def timescale_host(self) -> torch.Tensor:
        """timescale_i = min * (max / min) ** (2 i / head_dim)   (position_encoding.py:85-88),
        computed in float64 and rounded once to float32."""
        i = torch.arange(self.head_dim // 2, dtype=torch.float64)
        ts = self.min_timescale * (self.base / self.min_timescale) ** (2.0 * i / self.head_dim)
        return ts.to(torch.float32)

    def to_device(self, device) -> None:
        self._table = self.timescale_host().to(device)

    def rotary_table(self):
        if self._table is None:
            raise RuntimeError("rope: to_device() has not been called")
        return self._table, self.scale_factor

    def apply(self, x, positions, num_heads, head_dim, div=1.0):
        if head_dim != self.head_dim:
            raise ValueError(f"rope: built for head_dim {self.head_dim}, applied to {head_dim}")
        table, sf = self.rotary_table()
        ops.rope(x, positions, table, sf, div, num_heads, head_dim)


@POSITION_ENCODINGS.register("partial_rope")
class PartialRoPE(PositionEncoding):
    """Rotation of the first `dims` dimensions of a head only, in half-split pairs (i, i + dims / 2) by the angle
    position * base ** (-2 i / dims); the other dimensions pass unchanged.  The frequencies are computed in float64
    and rounded once to float32; the angle is their 32-bit product with the position."""

    def __init__(self, head_dim: int, dims: int, base: float):
        if dims % 2 or not 0 <= dims <= head_dim:
            raise ValueError(f"partial_rope: {dims} rotated dimensions of {head_dim} (an even number, at most all)")
        if dims and base <= 0:
            raise ValueError("partial_rope: the base must be positive")
        self.head_dim, self.dims, self.base = int(head_dim), int(dims), float(base)
        self._inv_freq: torch.Tensor | None = None

    def inv_freq_host(self) -> torch.Tensor:
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        return (self.base ** (-2.0 * i / max(self.dims, 1))).to(torch.float32)

    def to_device(self, device) -> None:
        self._inv_freq = self.inv_freq_host().to(device)

    def frequencies(self) -> tuple[torch.Tensor | None, int]:
        """(float32 [dims / 2] on the device, dims): what the rotate-and-write kernel of a mixer takes."""
        if self.dims and self._inv_freq is None:
            raise RuntimeError("partial_rope: to_device() has not been called")
        return (self._inv_freq if self.dims else None), self.dims

    def apply(self, x, positions, num_heads, head_dim, div=1.0):
        if head_dim != self.head_dim:
            raise ValueError(f"partial_rope: built for head_dim {self.head_dim}, applied to {head_dim}")
        if div != 1.0:
            raise ValueError("partial_rope: no division")
        inv_freq, dims = self.frequencies()
        # (the kernel's first H heads are rotated in place; no keys, no values, no norm)
        ops.qk_norm_rope_cache_write(x, positions, inv_freq, dims, None, num_heads, 0, head_dim, 1)


@POSITION_ENCODINGS.register("pair_rope")
class PairRoPE(PositionEncoding):
    """Rotation of `dims` consecutive entries in neighbouring pairs (2i, 2i + 1): the pair (u, v) at position p
    becomes mult * (u cos a - v sin a, v cos a + u sin a), a = p * f_i.  Where the rotated entries lie inside a
    vector is the mixer's business.  The frequencies, from f_i = base^(-2i / dims):

      scaling None                                   f_i, mult 1
      {"kind": "linear", "factor"}                   f_i / factor, mult 1
      {"kind": "ramp", "factor", "original", "fast", "slow"}
          f_i / factor * r_i + f_i * (1 - r_i) with a ramp r_i over the pair index that runs from 0 to 1 between the
          dimensions at which `fast` and `slow` turns fit into `original` positions, dim(t) = dims ln(original /
          (2 pi t)) / (2 ln base): lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), dims - 1),
          r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1); mult = 0.1 ln(factor) + 1 on cos and sin.

    Frequencies are computed in float64 and rounded once to float32; the angle is their 32-bit product with the
    position."""

    def __init__(self, dims: int, base: float, scaling: "dict | None" = None):
        if dims % 2 or dims < 0:
            raise ValueError(f"pair_rope: {dims} rotated entries (an even number)")
        if dims and base <= 0:
            raise ValueError("pair_rope: the base must be positive")
        self.dims, self.base = int(dims), float(base)
        self.scaling = dict(scaling) if scaling else None
        kind = self.scaling.get("kind") if self.scaling else None
        if kind not in (None, "linear", "ramp"):
            raise ValueError(f"pair_rope: unknown scaling {kind!r}; known: linear, ramp")
        for key in (("factor",) if kind == "linear" else ("factor", "original", "fast", "slow") if kind else ()):
            if not float(self.scaling.get(key, 0)) > 0:
                raise ValueError(f"pair_rope: {kind} scaling needs a positive {key!r}")
        self._freq: torch.Tensor | None = None

    @property
    def mult(self) -> float:
        """The factor on cos and sin."""
        import math

        if self.scaling and self.scaling["kind"] == "ramp":
            return 0.1 * math.log(float(self.scaling["factor"])) + 1.0
        return 1.0

    def freq_host(self) -> torch.Tensor:
        import math

        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / max(self.dims, 1))
        sc = self.scaling
        if sc and sc["kind"] == "linear":
            f = f / float(sc["factor"])
        elif sc:
            def dim_of(turns):
                return self.dims * math.log(float(sc["original"]) / (2.0 * math.pi * float(turns))) / (2.0 * math.log(self.base))

            lo = max(math.floor(dim_of(sc["fast"])), 0)
            hi = min(math.ceil(dim_of(sc["slow"])), self.dims - 1)
            ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            f = f / float(sc["factor"]) * ramp + f * (1.0 - ramp)
        return f.to(torch.float32)

    def to_device(self, device) -> None:
        self._freq = self.freq_host().to(device)

    def frequencies(self) -> tuple[torch.Tensor | None, int]:
        """(float32 [dims / 2] on the device, dims): what the norm-and-rotate kernel of a mixer takes."""
        if self.dims and self._freq is None:
            raise RuntimeError("pair_rope: to_device() has not been called")
        return (self._freq if self.dims else None), self.dims

    def apply(self, x, positions, num_heads, head_dim, div=1.0):
        if div != 1.0:
            raise ValueError("pair_rope: no division")
        freq, dims = self.frequencies()
        if dims > head_dim:
            raise ValueError(f"pair_rope: {dims} rotated entries in vectors of {head_dim}")
        ops.norm_rope_cache_write(x, positions, freq, dims, num_heads, 0, head_dim, 0, rot_mult=self.mult)
