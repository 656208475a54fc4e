"""Position encodings applied to queries and keys inside a mixer.
std/holon_std/ops/units.py:38-63 (`Rope`), formula std/holon_std/ops/reference.py:21-30, table layout
std/holon_std/ops/kernels.py:7-12."""
from __future__ import annotations

import math

import torch

from ..registry import register_part
from .base import Build, Part


def rope_table(max_positions: int, rotary_dim: int, theta: float) -> torch.Tensor:
    """[max_positions, rotary_dim] float32: cos(p * theta^(-2i/rotary_dim)) for i < rotary_dim/2, then the sines.
    Computed on the host in float32, in the reference's order of operations."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    angles = torch.arange(max_positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous()


@register_part("position", "rope")
class Rope(Part):
    """Rotary embedding, half-split ("neox") pairing: dims (i, i + rotary_dim/2) rotate by position * theta_i; dims
    beyond `rotary_dim` pass through."""

    graph_safe = True

    def __init__(self, build: Build, *, theta: float, head_dim: int, rotary_dim: int | None = None) -> None:
        super().__init__(build)
        self.theta, self.head_dim = float(theta), head_dim
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {head_dim}")
        self.table = rope_table(build.max_model_len, self.rotary_dim, self.theta).to(build.device)

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        """Rotate q [T, Hq, D] and k [T, Hkv, D] in place."""
        self.kernels.rope(q, positions, self.table)
        if k is not None:
            self.kernels.rope(k, positions, self.table)

    def fusion(self) -> dict | None:
        return {"position": "rope", "table": self.table}


def banded_frequencies(rotary_dim: int, base: float, scaling: dict | None) -> torch.Tensor:
    """f_i = base^(-2i/rotary_dim) for the rotary_dim/2 pairs, float32 (computed in float64, rounded once). With
    `scaling` = {factor, low, high, original}, by wavelength l = 2 pi / f: waves shorter than original/high keep f,
    waves longer than original/low turn `factor` times slower, and between the two the slow and the plain frequency
    are blended linearly in original/l (the long-context rescaling of Llama 3.1)."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = torch.as_tensor(float(base), dtype=torch.float64) ** (-2.0 * i / rotary_dim)
    if scaling:
        factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        wave = 2 * math.pi / f
        blend = ((original / wave - low) / (high - low)) if high != low else torch.ones_like(f)
        mid = (1 - blend) * f / factor + blend * f
        f = torch.where(wave < original / high, f, torch.where(wave > original / low, f / factor, mid))
    return f.to(torch.float32)


@register_part("position", "rope_banded")
class BandedRope(Rope):
    """Rotary embedding on the first `rotary_dim` dimensions of a head, half-split pairing, with frequencies that may
    be rescaled in bands of wavelength (`scaling`, given as a dict or as its sorted items). Angles are the float32
    product of position and frequency."""

    graph_safe = True

    def __init__(self, build: Build, *, theta: float, head_dim: int, rotary_dim: int | None = None,
                 scaling=None) -> None:
        Part.__init__(self, build)
        self.theta, self.head_dim = float(theta), head_dim
        self.rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {head_dim}")
        self.scaling = dict(scaling) if scaling else None
        freqs = banded_frequencies(self.rotary_dim, self.theta, self.scaling)
        angles = torch.arange(build.max_model_len, dtype=torch.float32)[:, None] * freqs[None, :]
        self.table = torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous().to(build.device)


def yarn_frequencies(rotary_dim: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(f_i for the rotary_dim/2 pairs as float32, computed in float64 and rounded once; the factor both cos and sin
    are multiplied by). Plain: f_i = base^(-2i/rotary_dim), factor 1. With `scaling` = {factor, original, fast, slow}
    (YaRN): the pair that turns t times over `original` positions has index d(t) = rotary_dim ln(original / (2 pi t))
    / (2 ln base); pairs up to lo = max(floor(d(fast)), 0) keep f_i, pairs from hi = min(ceil(d(slow)),
    rotary_dim - 1) on turn `factor` times slower, and between them the two are blended linearly in the index
    (ramp = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)); cos and sin are multiplied by 0.1 ln(factor) + 1."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = torch.as_tensor(float(base), dtype=torch.float64) ** (-2.0 * i / rotary_dim)
    if not scaling:
        return f.to(torch.float32), 1.0
    factor, original, fast, slow = (float(scaling[k]) for k in ("factor", "original", "fast", "slow"))

    def index_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), rotary_dim - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return (f / factor * ramp + f * (1 - ramp)).to(torch.float32), 0.1 * math.log(factor) + 1.0


@register_part("position", "rope_yarn")
class YarnRope(Rope):
    """Rotary embedding on the first `rotary_dim` dimensions of a head with YaRN's rescaling of the frequencies
    (`scaling`, a dict or its sorted items; None: plain frequencies). `interleaved` says that the design pairs
    dimensions (2i, 2i + 1); the table is laid out for the kernels' half-split pairing all the same, and a mixer that
    sees `interleaved` reorders its q and k projections' rows to match (every score stays what it was). Angles are the
    float32 product of position and frequency."""

    graph_safe = True

    def __init__(self, build: Build, *, theta: float, head_dim: int, rotary_dim: int | None = None, scaling=None,
                 interleaved: bool = False) -> None:
        Part.__init__(self, build)
        self.theta, self.head_dim = float(theta), head_dim
        self.rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {head_dim}")
        self.scaling = dict(scaling) if scaling else None
        self.interleaved = bool(interleaved)
        freqs, gain = yarn_frequencies(self.rotary_dim, self.theta, self.scaling)
        angles = torch.arange(build.max_model_len, dtype=torch.float32)[:, None] * freqs[None, :]
        gain = torch.tensor(gain, dtype=torch.float32)
        self.table = torch.cat((angles.cos() * gain, angles.sin() * gain), dim=-1).contiguous().to(build.device)


@register_part("position", "none")
class NoPosition(Part):
    """No position encoding (order enters through the causal mask alone)."""

    graph_safe = True

    def __init__(self, build: Build, *, head_dim: int) -> None:
        super().__init__(build)

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        return None

    def fusion(self) -> dict | None:
        return {"position": "none", "table": None}
