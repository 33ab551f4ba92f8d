"""Position encodings."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .. import ops
from .base import POSITIONS, Part, PartSpec


@dataclass(frozen=True)
class Rotation:
    """What a rotary position part hands to a mixer: the rotation's whole shape, so that the mixer and its
    kernels assume none.  ``cos`` and ``sin`` are float32 ``[positions, rotary_dim / 2]`` (None: no rotation);
    the first ``rotary_dim`` elements of a head are rotated, the rest is left alone; ``pairing`` says which two
    elements turn together: "half_split" (i, i + rotary_dim / 2) or "adjacent" (2 i, 2 i + 1)
    (crates/leone/src/cpu.rs:1765-1774)."""
    cos: Optional[torch.Tensor]
    sin: Optional[torch.Tensor]
    pairing: str = "half_split"
    elements: Optional[int] = None     # rotary_dim, for a part that knows it before its tables are made

    @property
    def rotary_dim(self) -> int:
        """How many elements of a head are rotated (0: none)."""
        if self.elements is not None:
            return self.elements
        return 0 if self.cos is None else 2 * self.cos.shape[1]


def rotation_of(position) -> Rotation:
    """The rotation of a position part: what its ``rotation()`` says, or, for a part that only has
    ``tables()``, those tables in half-split pairs; no part, no rotation."""
    if position is None:
        return Rotation(None, None)
    if hasattr(position, "rotation"):
        return position.rotation()
    return Rotation(*position.tables())


@POSITIONS.register("rope_half_split")
class RotaryHalfSplit(Part):
    """Rotates the pairs (i, i + R/2) of a head's first R elements by pos * theta^(-2i/R).

    Reference: crates/leone/src/cpu.rs:1721-1779 (inverse frequencies and the
    rotation), pairing HalfSplit for this architecture (crates/leone/src/model.rs:299-304).
    Parameters: ``rotary_dim`` (R; the whole head for this architecture, fewer elements leave the rest of
    the head unrotated), ``theta``.  The cos/sin table is evaluated in double on the device and kept as float.
    """

    graph_safe = True
    pairing = "half_split"

    def __init__(self, spec: PartSpec, **_):
        self.rotary_dim = int(spec["rotary_dim"])
        self.theta = float(spec["theta"])
        if self.rotary_dim <= 0 or self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even and positive, found {self.rotary_dim}")
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def prepare(self, max_positions: int, device) -> None:
        self.cos, self.sin = ops.rope_table(self.theta, self.rotary_dim, max_positions, device)

    def tables(self) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        return self.cos, self.sin

    def rotation(self) -> Rotation:
        return Rotation(self.cos, self.sin, self.pairing, self.rotary_dim)


@POSITIONS.register("rope_adjacent")
class RotaryAdjacent(RotaryHalfSplit):
    """The same angles on the pairs (2i, 2i + 1) (the reference's Adjacent pairing, crates/leone/src/cpu.rs:1765-1774)."""

    pairing = "adjacent"


def scaled_frequencies(rotary_dim: int, theta: float, factor: float, original: float, fast: float, slow: float):
    """The pairs' frequencies under a length extension, and the factor on cos and sin.  Pair i turns by theta^(-2i/R) a
    position.  ``pair(t) = R ln(original / (2 pi t)) / (2 ln theta)`` is the pair that turns t times over ``original``
    positions; with lo = max(floor(pair(fast)), 0) and hi = min(ceil(pair(slow)), R - 1) the pairs up to lo keep their
    frequency, the pairs from hi on are slowed by ``factor``, and between the two the share of the slowed frequency
    rises linearly, ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1).  cos and sin grow by 0.1 ln(factor) + 1."""
    def pair(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(pair(fast)), 0)
    hi = min(math.ceil(pair(slow)), rotary_dim - 1)
    out = []
    for i in range(rotary_dim // 2):
        f = theta ** (-2.0 * i / rotary_dim)
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


@POSITIONS.register("rope_scaled_adjacent")
class RotaryScaledAdjacent(Part):
    """Rotation of the pairs (2i, 2i + 1) with frequencies stretched for sequences longer than the ``original`` length
    (``scaled_frequencies``); the growth of cos and sin is in the tables.  Parameters: ``rotary_dim``, ``theta``,
    ``factor``, ``original``, ``fast``, ``slow``.  Angles are made in double and the tables kept as float."""

    graph_safe = True
    pairing = "adjacent"

    def __init__(self, spec: PartSpec, **_):
        self.rotary_dim, self.theta = int(spec["rotary_dim"]), float(spec["theta"])
        if self.rotary_dim <= 0 or self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even and positive, found {self.rotary_dim}")
        self.factor, self.original = float(spec["factor"]), float(spec["original"])
        self.fast, self.slow = float(spec["fast"]), float(spec["slow"])
        if not (self.factor > 0.0 and self.original > 0.0 and self.fast > 0.0 and self.slow > 0.0 and self.theta > 1.0):
            raise ValueError("the scaled rotation needs positive factor, original length, fast and slow turns and theta > 1")
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def prepare(self, max_positions: int, device) -> None:
        frequencies, growth = scaled_frequencies(self.rotary_dim, self.theta, self.factor, self.original, self.fast, self.slow)
        angle = torch.arange(max_positions, dtype=torch.float64, device=device)[:, None] * \
            torch.tensor(frequencies, dtype=torch.float64, device=device)[None, :]
        self.cos = (torch.cos(angle) * growth).float().contiguous()
        self.sin = (torch.sin(angle) * growth).float().contiguous()

    def tables(self) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        return self.cos, self.sin

    def rotation(self) -> Rotation:
        return Rotation(self.cos, self.sin, self.pairing, self.rotary_dim)


@POSITIONS.register("none")
class NoPosition(Part):
    """No position encoding: queries and keys are used as projected."""

    graph_safe = True

    def __init__(self, spec: PartSpec, **_):
        pass

    def prepare(self, max_positions: int, device) -> None:
        pass

    def tables(self):
        return None, None

    def rotation(self) -> Rotation:
        return Rotation(None, None)
