"""Position encodings for attention mixers.

Rotary, as the reference builds it (ullm/layers/rotary_embedding.py:52-75): inv_freq_i =
1 / base^(2i/d) for i < d/2, angle[p, i] = p * inv_freq_i, cos and sin in 32-bit, one table row per
position.  The table stays 32-bit (the reference casts cos/sin to the activation dtype before the
multiply, rotary_embedding.py:16-17; here the rotation itself is 32-bit).  Pairing "half" rotates
(x[i], x[i + d/2]) as the reference's chunk(2) does (rotary_embedding.py:19-22); the reference then
interleaves the two output halves (rotary_embedding.py:24), a fixed permutation applied to q and k
alike that leaves every q.k unchanged, so outputs are kept in place here.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import PartEnv, PositionEncoding, WeightDecl, register_part


@register_part("position", "none")
class NoPosition(PositionEncoding):
    def kernel_args(self):
        return None, 0, 0


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    """``rotary_dim`` leading dims of each head are rotated; ``pairing`` is "half" or "adjacent".

    ``scaling`` = (factor, original, fast, slow) stretches the frequencies by wavelength: with
    d(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), the pair index at which a pair turns t times over
    ``original`` positions, lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), rotary_dim - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at f_i / factor * ramp_i + f_i * (1 - ramp_i),
    and every cosine and sine is multiplied by 0.1 ln(factor) + 1.

    ``scaling`` = ("by_wavelength", factor, low, high, original) is another stretch: with l = 2 pi / f_i the pair's
    wavelength, pairs with l < original / high keep f_i, pairs with l > original / low turn at f_i / factor, and
    those between, with s = (original / l - low) / (high - low), at (1 - s) f_i / factor + s f_i; cosines and sines
    keep their size."""

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None,
                 pairing: str = "half", max_positions: Optional[int] = None, scaling: Optional[tuple] = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= head_dim):
            raise ValueError(f"rotary_dim={self.rotary_dim} must be even and at most head_dim={head_dim}")
        if pairing not in ("half", "adjacent"):
            raise ValueError(f"unknown rotary pairing {pairing!r}")
        self.style = 1 if pairing == "half" else 2
        self.max_positions = max_positions
        self.scaling = None
        if scaling is not None and scaling[0] == "by_wavelength":
            self.scaling = ("by_wavelength",) + tuple(float(v) for v in scaling[1:])
            if len(self.scaling) != 5 or min(self.scaling[1:]) <= 0 or self.scaling[2] == self.scaling[3]:
                raise ValueError(f"scaling={scaling!r}: ('by_wavelength', factor, low, high, original), all positive, low != high")
        elif scaling is not None:
            self.scaling = tuple(float(v) for v in scaling)
            if len(self.scaling) != 4 or min(self.scaling) <= 0:
                raise ValueError(f"scaling={scaling!r}: (factor, original, fast, slow), all positive")
        self.table: Optional[torch.Tensor] = None

    @staticmethod
    def make_table(rotary_dim: int, theta: float, rows: int, scaling: Optional[tuple] = None) -> torch.Tensor:
        if scaling is None:
            inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
            angles = torch.arange(rows, dtype=torch.float32)[:, None] * inv_freq[None, :]
            return torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous()
        if scaling[0] == "by_wavelength":
            _, factor, low, high, original = scaling
            i = torch.arange(rotary_dim // 2, dtype=torch.float64)
            freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / rotary_dim)
            wavelength = 2 * math.pi / freq
            blend = ((original / wavelength - low) / (high - low)).clamp(0.0, 1.0)
            mixed = (1.0 - blend) * freq / factor + blend * freq
            freq = torch.where(wavelength < original / high, freq, torch.where(wavelength > original / low, freq / factor, mixed))
            angles = torch.arange(rows, dtype=torch.float64)[:, None] * freq[None, :]
            return torch.cat((angles.cos(), angles.sin()), dim=-1).to(torch.float32).contiguous()
        # stretched frequencies: built in 64-bit, so that the 32-bit table is the rounding of the exact angles' values
        factor, original, fast, slow = scaling
        i = torch.arange(rotary_dim // 2, dtype=torch.float64)
        inv_freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / rotary_dim)

        def pair_turning(times: float) -> float:
            return rotary_dim * math.log(original / (2 * math.pi * times)) / (2 * math.log(theta))
        lo = max(math.floor(pair_turning(fast)), 0)
        hi = min(math.ceil(pair_turning(slow)), rotary_dim - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        inv_freq = inv_freq / factor * ramp + inv_freq * (1.0 - ramp)
        magnitude = 0.1 * math.log(factor) + 1.0
        angles = torch.arange(rows, dtype=torch.float64)[:, None] * inv_freq[None, :]
        return (torch.cat((angles.cos(), angles.sin()), dim=-1) * magnitude).to(torch.float32).contiguous()

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        rows = env.context_len if self.max_positions is None else min(env.context_len, self.max_positions)
        # every layer with the same rotation shares one table: built once, read by all their kernels
        self.table = env.shared(("rotary", self.rotary_dim, self.theta, rows, self.scaling),
                                lambda: self.make_table(self.rotary_dim, self.theta, rows, self.scaling).to(env.device))

    def kernel_args(self):
        return self.table, self.rotary_dim, self.style


def log_distance_bucket(distance: int, rows: int, far: int) -> int:
    """The table row of a key ``distance`` >= 0 positions behind the query: the distance itself below
    rows // 2, then rows - rows // 2 further rows spread evenly over the logarithm of the distance up to ``far``,
    every greater distance in the last row."""
    half = rows // 2
    if distance < half:
        return distance
    step = math.log(distance / half) / math.log(far / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(step)))


@register_part("position", "log_distance_bias")
class LogDistanceBias(PositionEncoding):
    """Positions that enter the scores and not the vectors: a learned table [rows, heads] whose row
    :func:`log_distance_bucket` of the distance between query and key is added to the scaled score.  For the
    kernels the table is unrolled by distance once, float32 [heads, distances], up to the first distance
    that falls into the last row; they clamp greater distances to that entry."""

    DEFAULT_ROWS = 32        # what random weights are drawn with; a checkpoint's table has the rows it has

    def __init__(self, heads: int, far: int, weight_name: str, rows: Optional[int] = None):
        self.rows = int(rows) if rows is not None else None       # None: read off the bound tensor
        self.heads, self.far, self.weight_name = int(heads), int(far), weight_name
        self.by_distance: Optional[torch.Tensor] = None

    def weights(self):
        if self.rows is None:
            return [WeightDecl(self.weight_name, (self.DEFAULT_ROWS, self.heads), keep_fp32=True, free_dims=(0,))]
        return [WeightDecl(self.weight_name, (self.rows, self.heads), keep_fp32=True)]

    def buckets(self) -> list:
        """Bucket by distance, ending with the first distance in the last row."""
        out, d = [], 0
        while True:
            out.append(log_distance_bucket(d, self.rows, self.far))
            if out[-1] == self.rows - 1:
                return out
            d += 1

    def bind(self, tensors: Dict[str, torch.Tensor], env: PartEnv) -> None:
        table = tensors[self.weight_name].to(torch.float32)
        self.rows = table.shape[0]
        if self.rows < 2 or self.far <= self.rows // 2:
            raise ValueError(f"{self.weight_name}: a distance table of {self.rows} rows reaching to {self.far}: it needs "
                             f"two rows and a reach beyond rows // 2")
        index = torch.tensor(self.buckets(), dtype=torch.long, device=table.device)
        self.by_distance = table[index].T.contiguous()           # [heads, distances]
        self.by_distance_log2 = (self.by_distance * math.log2(math.e)).contiguous()

    def score_bias(self):
        return self.by_distance

    def score_bias_log2(self):
        """The same table times log2(e), for kernels whose scores are exponents of two."""
        return self.by_distance_log2
