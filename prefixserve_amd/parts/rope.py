"""Rotary position encoding (rotate-half layout) with optional llama3 frequency scaling."""

from __future__ import annotations

import math
from typing import Any, Mapping

import torch

from .base import RotaryTable, Runtime, register_position


def rope_inv_freq(head_dim: int, theta: float, scaling: Mapping[str, Any] | None) -> torch.Tensor:
    """``rope_inv_freq64`` rounded once to float32, which agrees with the reference's float32
    evaluation to one ulp and does not depend on a library's ``pow``."""
    return rope_inv_freq64(head_dim, theta, scaling).to(torch.float32)


def rope_inv_freq64(head_dim: int, theta: float, scaling: Mapping[str, Any] | None) -> torch.Tensor:
    """inv_freq[i] = 1 / theta^(2i/D), i < D/2, then the llama3 three bands by wavelength:
    long waves divided by ``factor``, short ones unchanged, the middle blended
    (prefixserve/model/llama.py:24-46 of the reference). Evaluated and returned in float64."""
    i = torch.arange(0, head_dim, 2, dtype=torch.float64)
    inv = 1.0 / (torch.tensor(float(theta), dtype=torch.float64) ** (i / head_dim))
    if scaling is not None:
        factor = float(scaling["factor"])
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        old = float(scaling["original_max_position_embeddings"])
        low_wavelen, high_wavelen = old / low, old / high
        wavelen = 2.0 * math.pi / inv
        scaled = torch.where(wavelen > low_wavelen, inv / factor, inv)
        smooth = (old / wavelen - low) / (high - low)
        smoothed = (1.0 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
        inv = torch.where(medium, smoothed, scaled)
    return inv


class RotaryEmbedding(RotaryTable):
    """Pairs (i, i + D/2) of every head are rotated by angle = position * inv_freq[i]
    (prefixserve/model/llama.py:72-77). The angle is a float32 product as in the
    reference's table (llama.py:56-58); its cosine and sine are kept in float32 whatever
    the activation dtype. The table is ``[max_position, D/2, 2]`` = (cos, sin) and is
    read by the kernel that also writes keys and values into their pages.

    ``rotary_dim``: only the model's first that many dimensions of a head rotate (partners
    rotary_dim / 2 apart, frequencies theta^(-2i / rotary_dim)); the table's other pair slots are the
    identity and the mixer lays a head out accordingly. The angles of this form are products in
    float64, rounded once as cosine and sine."""

    def __init__(self, head_dim: int, theta: float, scaling: Mapping[str, Any] | None = None,
                 rotary_dim: int | None = None) -> None:
        if head_dim % 2:
            raise ValueError(f"rotary head_dim must be even, got {head_dim}")
        if rotary_dim is not None and (rotary_dim % 2 or not 0 <= rotary_dim <= head_dim):
            raise ValueError(f"rotary_dim {rotary_dim} must be even and at most head_dim {head_dim}")
        self.rotary_dim = None if rotary_dim is None else int(rotary_dim)
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.scaling = dict(scaling) if scaling is not None else None
        self.table: torch.Tensor | None = None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)

    def prepare(self, max_position: int) -> None:
        if self.rotary_dim is not None:
            table = torch.zeros((max_position, self.head_dim // 2, 2), dtype=torch.float64)
            table[:, :, 0] = 1.0
            if self.rotary_dim:
                inv = rope_inv_freq64(self.rotary_dim, self.theta, self.scaling)
                angle = torch.outer(torch.arange(max_position, dtype=torch.float64), inv)
                table[:, : self.rotary_dim // 2, 0] = angle.cos()
                table[:, : self.rotary_dim // 2, 1] = angle.sin()
            self.table = table.to(torch.float32).contiguous().to(self.rt.device)
            self.max_position = int(max_position)
            return
        inv = rope_inv_freq(self.head_dim, self.theta, self.scaling)
        pos = torch.arange(max_position, dtype=torch.float32)
        angle = torch.outer(pos, inv)  # float32 product, exactly rounded
        a64 = angle.to(torch.float64)
        table = torch.stack((a64.cos(), a64.sin()), dim=-1).to(torch.float32)
        self.table = table.contiguous().to(self.rt.device)
        self.max_position = int(max_position)


def yarn_inv_freq(rotary_dim: int, base: float, scaling: Mapping[str, Any] | None) -> tuple[torch.Tensor, float]:
    """(float64 frequencies f_i = base^(-2i/r), i < r/2, after YaRN scaling; the factor on cos and sin).

    ``scaling`` = (factor s, original length L, fast, slow): a wave that makes t turns over L
    sits at dimension dim(t) = r ln(L / (2 pi t)) / (2 ln base). Below lo = floor(dim(fast)) a
    frequency is kept, above hi = ceil(dim(slow)) it is divided by s, in between the share of
    the divided one rises linearly (lo and hi are kept inside [0, r - 1]; a span of zero counts
    as 0.001). Cosine and sine are multiplied by 0.1 ln(s) + 1."""
    i = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / rotary_dim)
    if scaling is None:
        return f, 1.0
    s, orig = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns: float) -> float:
        return rotary_dim * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), rotary_dim - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / s * ramp + f * (1.0 - ramp), 0.1 * math.log(s) + 1.0


class YarnRotary(RotaryTable):
    """A rotation of the first ``rotary_dim`` dimensions of a head only, with YaRN-scaled
    frequencies and its factor on cosine and sine. The table has ``head_dim / 2`` pair slots
    like every ``RotaryTable``: the first ``rotary_dim / 2`` carry the angles, the others are
    the identity (1, 0), so the kernels that rotate whole heads leave the rest of a head as it
    is. The mixer lays a head out accordingly (``rotary_dim`` tells it to): the partners
    (i, i + rotary_dim/2) of the model's layout sit in slots (i, i + head_dim/2).
    Angles are position x frequency in float64, rounded once to float32 as cos and sin."""

    def __init__(self, head_dim: int, rotary_dim: int, base: float, scaling: Mapping[str, Any] | None = None) -> None:
        if head_dim % 2 or rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and at most head_dim {head_dim} (even)")
        self.head_dim, self.rotary_dim = int(head_dim), int(rotary_dim)
        self.base = float(base)
        self.scaling = dict(scaling) if scaling is not None else None
        self.table: torch.Tensor | None = None

    def prepare(self, max_position: int) -> None:
        table = torch.zeros((max_position, self.head_dim // 2, 2), dtype=torch.float64)
        table[:, :, 0] = 1.0
        if self.rotary_dim:
            freq, gain = yarn_inv_freq(self.rotary_dim, self.base, self.scaling)
            angle = torch.outer(torch.arange(max_position, dtype=torch.float64), freq)
            table[:, : self.rotary_dim // 2, 0] = angle.cos() * gain
            table[:, : self.rotary_dim // 2, 1] = angle.sin() * gain
        self.table = table.to(torch.float32).contiguous().to(self.rt.device)
        self.max_position = int(max_position)


register_position("rope", RotaryEmbedding)
register_position("yarn", YarnRotary)
