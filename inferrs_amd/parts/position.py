"""Position encodings.  "rope": angle[p, i] = p * theta**(-2i/rot_dim), computed in 32-bit
(`inferrs-models/src/models/attention_utils.rs:186-216`); "none": nothing."""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..config.spec import PositionSpec, SpecError
from .base import Position, register_position


def inverse_frequencies(theta: float, rot_dim: int) -> np.ndarray:
    """1 / theta**(2i/rot_dim) for i in 0..rot_dim/2 as the reference computes it
    (`attention_utils.rs:198-203`): the exponent, the power and the quotient are 32-bit
    operations.  The power is taken in 64-bit and rounded once, which is what a correctly
    rounded `powf` returns."""
    i = np.arange(rot_dim // 2, dtype=np.float32)
    exponent = (np.float32(2.0) * i) / np.float32(rot_dim)
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
    return (np.float32(1.0) / power).astype(np.float32)


def linear_scaling(inv_freq: np.ndarray, factor: float) -> np.ndarray:
    """Positions read as position / factor: every frequency divided by it, in 32-bit."""
    if not (factor > 0.0):
        raise SpecError(f"rotary scaling 'linear' needs a positive factor, got {factor}")
    return (inv_freq / np.float32(factor)).astype(np.float32)


def yarn_scaling(inv_freq: np.ndarray, factor: float, original: float, fast: float, slow: float, *, theta: float,
                 rot_dim: int):
    """Pairs that turn fast keep their frequency, slow ones are divided by `factor`, a linear ramp between the pair
    that makes `fast` turns over `original` positions and the one that makes `slow`: with
    pair(t) = rot_dim ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(pair(fast)), 0),
    hi = min(ceil(pair(slow)), rot_dim - 1), ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
    f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i).  cos and sin are multiplied by 0.1 ln(factor) + 1.
    Returns (frequencies, that factor).  (Peng et al., "YaRN: Efficient Context Window Extension of Large
    Language Models".)"""
    if not (factor > 0.0 and original > 0.0 and fast > 0.0 and slow > 0.0 and theta > 1.0):
        raise SpecError(f"rotary scaling 'yarn' needs positive numbers, got factor={factor} original={original} "
                        f"fast={fast} slow={slow} base={theta}")

    def pair(turns: float) -> float:
        return rot_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(pair(fast)), 0)
    hi = min(math.ceil(pair(slow)), rot_dim - 1)
    i = np.arange(inv_freq.shape[0], dtype=np.float64)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = inv_freq.astype(np.float64)
    return (f / factor * ramp + f * (1.0 - ramp)).astype(np.float32), 0.1 * math.log(factor) + 1.0


def llama3_scaling(inv_freq: np.ndarray, factor: float, low: float, high: float, original: float) -> np.ndarray:
    """By wavelength l = 2 pi / f: f stays where l < original / high, becomes f / factor where l > original / low, and
    between the two, with s = (original / l - low) / (high - low), (1 - s) f / factor + s f.  (The frequency scaling of
    Llama 3.1; Grattafiori et al., "The Llama 3 Herd of Models".)"""
    if not (factor > 0.0 and original > 0.0 and high > low >= 0.0):
        raise SpecError(f"rotary scaling 'llama3' needs factor > 0, original > 0 and high > low, got factor={factor} "
                        f"low={low} high={high} original={original}")
    f = inv_freq.astype(np.float64)
    wave = 2.0 * math.pi / f
    s = (original / wave - low) / (high - low)
    blended = (1.0 - s) * f / factor + s * f
    out = np.where(wave < original / high, f, np.where(wave > original / low, f / factor, blended))
    return out.astype(np.float32)


# name of a scaling law -> (inverse frequencies, the law's numbers) -> inverse frequencies, or (inverse frequencies,
# factor on cos and sin); a law that needs the base and the rotated size says so in SCALING_NEEDS_GEOMETRY
SCALING_LAWS = {"linear": linear_scaling, "yarn": yarn_scaling, "llama3": llama3_scaling}
SCALING_NEEDS_GEOMETRY = {"yarn"}


@register_position("rope")
class Rotary(Position):
    graph_safe = True

    def __init__(self, spec: PositionSpec, tensors, dtype, device):
        if spec.rot_dim <= 0 or spec.rot_dim % 2 or spec.rot_dim > spec.head_dim:
            raise SpecError(f"rot_dim {spec.rot_dim} must be even and within head_dim {spec.head_dim}")
        if spec.pairing not in ("half", "interleaved"):
            raise SpecError(f"unknown rotary pairing {spec.pairing!r}")
        self.spec = spec
        self.rot_dim = spec.rot_dim
        self.interleaved = spec.pairing == "interleaved"
        inv_freq = inverse_frequencies(spec.theta, spec.rot_dim)
        self.magnitude = 1.0             # cos and sin are multiplied by this (the kernels that rotate take it)
        if spec.scaling is not None:
            law, numbers = spec.scaling[0], [float(v) for v in spec.scaling[1:]]
            if law not in SCALING_LAWS:
                raise SpecError(f"rotary scaling {law!r} has no entry (known: {sorted(SCALING_LAWS)})")
            extra = dict(theta=float(spec.theta), rot_dim=spec.rot_dim) if law in SCALING_NEEDS_GEOMETRY else {}
            try:
                scaled = SCALING_LAWS[law](inv_freq, *numbers, **extra)
            except TypeError:
                raise SpecError(f"rotary scaling {law!r} does not take the {len(numbers)} numbers {numbers}") from None
            if isinstance(scaled, tuple):
                inv_freq, self.magnitude = scaled[0], float(scaled[1])
            else:
                inv_freq = scaled
        self.inv_freq = torch.from_numpy(inv_freq).to(device)

    def table(self, positions: torch.Tensor) -> Optional[Tuple[torch.Tensor, torch.Tensor]]:
        return ops.rope_table(positions, self.inv_freq)


@register_position("none")
class NoPosition(Position):
    graph_safe = True

    rot_dim = 0
    interleaved = False
    magnitude = 1.0

    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec

    def table(self, positions):
        return None
