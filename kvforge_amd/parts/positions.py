"""Rotary position encoding: fp32 cos/sin tables that attention applies to queries and keys.

Angles follow src/tokenvault/model.py:41-50: ``inv_freq[j] = 1 / theta^(2j/d)`` in fp32,
``angle = float(position) * inv_freq`` in fp32, then cos and sin.  The tables are computed once
on the host with exactly these operations, so the kernels never evaluate a trigonometric
function of a large angle themselves.  Frequency scaling of type ``llama3`` (absent from the
reference) rescales ``inv_freq`` before the tables are made.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from kvforge_amd.config.model import RopeScaling
from kvforge_amd.parts.base import Positions, WeightSpec
from kvforge_amd.registry import register_positions


@dataclass(frozen=True)
class YarnStretch:
    """Frequency scaling of the YaRN kind.  With ``turns(i)`` the index at which a pair would turn
    ``t`` times over ``original`` positions, ``dims * ln(original / (2 pi t)) / (2 ln theta)``:
    pairs below ``lo = max(floor(turns(fast)), 0)`` keep their frequency, pairs from
    ``hi = min(ceil(turns(slow)), dims - 1)`` on have it divided by ``factor``, the ones between
    are blended linearly; cos and sin are multiplied by ``0.1 ln(factor) + 1``."""

    factor: float
    original: int
    fast: float
    slow: float
    rope_type: str = "yarn"


def yarn_inv_freq(rot_dim: int, theta: float, s: YarnStretch) -> torch.Tensor:
    i = torch.arange(rot_dim // 2, dtype=torch.float64)
    f = float(theta) ** (-2.0 * i / rot_dim)

    def turns(t: float) -> float:
        return rot_dim * math.log(s.original / (2.0 * math.pi * t)) / (2.0 * math.log(theta))

    lo = max(math.floor(turns(s.fast)), 0)
    hi = min(math.ceil(turns(s.slow)), rot_dim - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return (f / s.factor * ramp + f * (1.0 - ramp)).float()


def rotary_magnitude(scaling) -> float:
    """What cos and sin are multiplied by under ``scaling`` (1 for none and for llama3)."""
    if scaling is not None and getattr(scaling, "rope_type", None) == "yarn":
        return 0.1 * math.log(scaling.factor) + 1.0
    return 1.0


def scaled_inv_freq(rot_dim: int, theta: float, scaling: "RopeScaling | YarnStretch | None") -> torch.Tensor:
    inv_freq = 1.0 / (theta ** (torch.arange(0, rot_dim, 2, dtype=torch.float32) / rot_dim))
    if scaling is None:
        return inv_freq
    if scaling.rope_type == "yarn":
        return yarn_inv_freq(rot_dim, theta, scaling)
    if scaling.rope_type != "llama3":
        raise ValueError(f"unsupported rope scaling {scaling.rope_type!r}")
    f = inv_freq.double()
    orig = float(scaling.original_max_position_embeddings)
    wavelen = 2.0 * math.pi / f
    low_wavelen = orig / scaling.low_freq_factor
    high_wavelen = orig / scaling.high_freq_factor
    smooth = (orig / wavelen - scaling.low_freq_factor) / (
        scaling.high_freq_factor - scaling.low_freq_factor)
    blended = (1.0 - smooth) * f / scaling.factor + smooth * f
    out = torch.where(wavelen < high_wavelen, f,
                      torch.where(wavelen > low_wavelen, f / scaling.factor, blended))
    return out.float()


@register_positions("rotary")
class RotaryPositions(Positions):
    """Rotary pairs over the first ``rot_dim`` elements of each head.  ``interleaved=False``: the
    checkpoint pairs element ``i`` with ``i + rot_dim/2`` (half-split); ``True``: it pairs element
    ``2i`` with ``2i + 1``, which is the order the kernels rotate in, so that a mixer has nothing
    to permute.  ``scaling``: ``RopeScaling`` (llama3), ``YarnStretch`` or ``None``."""

    replayable = True

    def __init__(self, rot_dim: int, theta: float, scaling: "RopeScaling | YarnStretch | None" = None,
                 interleaved: bool = False) -> None:
        if rot_dim <= 0 or rot_dim % 2:
            raise ValueError(f"rotary width must be positive and even, got {rot_dim}")
        self.rot_dim, self.theta, self.scaling = int(rot_dim), float(theta), scaling
        self.interleaved = bool(interleaved)
        self.inv_freq = scaled_inv_freq(self.rot_dim, self.theta, scaling)
        self.magnitude = rotary_magnitude(scaling)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def prepare(self, max_positions: int, device: torch.device | str) -> None:
        pos = torch.arange(int(max_positions), dtype=torch.int64)
        freqs = pos.float()[:, None] * self.inv_freq.float()
        cos, sin = freqs.cos(), freqs.sin()
        if self.magnitude != 1.0:
            cos, sin = cos * self.magnitude, sin * self.magnitude
        self.cos = cos.contiguous().to(device)
        self.sin = sin.contiguous().to(device)

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}


@register_positions("learned")
class LearnedPositions(Positions):
    """An absolute encoding: a learned vector per position, ``table[p]``, added to the embedding
    of the token at position ``p`` as it is (no scale).  ``name``: the table's checkpoint name,
    ``[max_positions, width]``."""

    replayable = True

    def __init__(self, name: str, max_positions: int, width: int) -> None:
        self.name, self.max_positions, self.width = name, int(max_positions), int(width)
        self.table: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.max_positions, self.width))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name]

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}

    def held_tensors(self) -> list[torch.Tensor]:
        return [] if self.table is None else [self.table]

    def on_embedding(self, residual: torch.Tensor, step) -> None:
        from kvforge_amd.kernels import ops

        ops.add_positions(residual, self.table, step.positions)
