"""Rotary position embedding.

Reference: minivllm/models/layers/rotary.py. The table is ``cat(cos, sin)`` of
``position * inv_freq`` with ``inv_freq_i = 1 / theta^(2i / rotary_dim)``, all float32
(rotary.py:35-46); the rotation pairs element i with i + rotary_dim/2 (rotary.py:11-14) and
is computed in float32. ``inv_freq`` is evaluated here by the same float32 expression, the
angles and their cosines and sines by a kernel; the rotation itself is fused into the
attention's q/k kernel, which takes the table from ``rotary()``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .base import PartSpec, PositionEncoding, Runtime, register_position_encoding


@dataclass(frozen=True)
class RotarySpec(PartSpec):
    kind = "rotary"
    rotary_dim: int = 0
    theta: float = 10000.0
    interleaved: bool = False      # pairs (2i, 2i+1) instead of (i, i + rotary_dim/2)
    # stretched low frequencies for contexts longer than the model was made for: (factor, original length, fast, slow),
    # see ``stretched_frequencies``; None: the plain geometric frequencies
    stretch: Optional[Tuple[float, float, float, float]] = None


def inverse_frequencies(rotary_dim: int, theta: float) -> torch.Tensor:
    """float32 [rotary_dim / 2], evaluated as the reference does (rotary.py:35)."""
    return 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))


# a stretched table's cosines and sines are multiplied by MAGNITUDE_SLOPE * ln(factor) + 1
MAGNITUDE_SLOPE = 0.1
# the least width of the ramp between the untouched and the fully stretched pairs
RAMP_FLOOR = 0.001


def stretched_frequencies(rotary_dim: int, theta: float, stretch: Tuple[float, float, float, float]) -> Tuple[torch.Tensor, float]:
    """(float32 [rotary_dim / 2] frequencies, magnitude of the table) for ``stretch`` = (factor, original, fast, slow).

    The pair that turns t times over ``original`` positions has the index d(t) = rotary_dim * ln(original / (2 pi t)) /
    (2 ln theta). Pairs below lo = floor(d(fast)) turn fast enough to be left alone, pairs above hi = ceil(d(slow)) are
    slowed by ``factor``, and between them (lo and hi held inside 0 .. rotary_dim - 1) the two are blended along the
    ramp clamp((i - lo) / max(hi - lo, RAMP_FLOOR), 0, 1). Evaluated in double precision, rounded once."""
    factor, original, fast, slow = (float(v) for v in stretch)
    if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and theta > 1):
        raise ValueError(f"stretched rotary frequencies need positive constants and theta > 1, got {stretch}, theta {theta}")

    def index_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), rotary_dim - 1)
    freqs = []
    for i in range(rotary_dim // 2):
        f = theta ** (-2.0 * i / rotary_dim)
        ramp = min(max((i - lo) / max(hi - lo, RAMP_FLOOR), 0.0), 1.0)
        freqs.append(f / factor * ramp + f * (1.0 - ramp))
    return torch.tensor(freqs, dtype=torch.float32), MAGNITUDE_SLOPE * math.log(factor) + 1.0


@register_position_encoding(RotarySpec.kind)
class RotaryEmbedding(PositionEncoding):
    spec_class = RotarySpec

    def __init__(self, spec: RotarySpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be positive and even, got {spec.rotary_dim}")
        self.spec = spec
        self.rt = rt
        if spec.stretch is None:
            inv_freq, magnitude = inverse_frequencies(spec.rotary_dim, spec.theta), 1.0
        else:
            inv_freq, magnitude = stretched_frequencies(spec.rotary_dim, spec.theta, spec.stretch)
        self.table = rt.ops.rope_table(inv_freq.to(rt.device), rt.max_positions)
        if magnitude != 1.0:
            rt.ops.scale_f32(self.table, magnitude)

    def rotary(self) -> Optional[Tuple[torch.Tensor, bool]]:
        return self.table, self.spec.interleaved

    def step_gather(self, ctx):
        """In a step of single decoded tokens every layer needs the table's rows at the same few
        positions: they are gathered once, in front of the layers, so that no layer has to wait for a
        position before it can ask for its angles."""
        plan = ctx.attention_plan
        if plan is None or not plan.decode_only or self.spec.interleaved or not self.rt.ops.use_fast_kernels:
            return None
        rows = self.rt.workspace.get(f"rotary.rows.{self.spec.rotary_dim}.{self.spec.theta}.{self.spec.stretch}",
                                     (ctx.n_tokens, self.spec.rotary_dim), torch.float32)
        ctx.position_rows[self] = rows
        return ctx.positions, self.table, rows
