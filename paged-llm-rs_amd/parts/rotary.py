"""Rotary position tables (reference: model/rope.rs:32-63).

The angle position * theta^(-2i/dim) is computed in 64-bit on the host and the
tables are kept in 32-bit whatever the model's type is; the half table is stored
once, [max_positions, dim/2], since both halves of a head use the same angles.
"""

from __future__ import annotations

import torch

from ..errors import UnsupportedError
from .registry import POSITIONS, lookup, register_position


class RotaryTables:
    # which elements of a head an angle turns: i and i + dim/2 (False), or 2 i and 2 i + 1 (True)
    neighbours = False

    def __init__(self, spec, device):
        if spec.dim % 2 or spec.dim <= 0:
            raise UnsupportedError(f"a rotation over {spec.dim} values, which do not pair")
        self.dim = spec.dim
        half = spec.dim // 2
        inv = torch.tensor([1.0 / (spec.theta ** (2.0 * i / spec.dim)) for i in range(half)], dtype=torch.float64)
        angle = torch.arange(spec.max_positions, dtype=torch.float64)[:, None] * inv[None, :]
        self.cos = angle.cos().to(torch.float32).to(device).contiguous()
        self.sin = angle.sin().to(torch.float32).to(device).contiguous()
        self.max_positions = spec.max_positions


class RotaryNeighbourTables(RotaryTables):
    """The same angles, turning neighbouring elements: the layout of checkpoints that were not permuted for
    the half-split form."""
    neighbours = True


register_position("rotary_half", RotaryTables)
register_position("rotary_neighbours", RotaryNeighbourTables)


def rotary_tables(spec, device, shared: dict):
    """The tables of a position spec, built by the class its ``kind`` names; layers
    with the same spec share one pair."""
    key = ("position", spec, str(device))
    if key not in shared:
        shared[key] = lookup(POSITIONS, spec.kind, "position encoding")(spec, device)
    return shared[key]


def rotary_frequencies(dims: int, base: float, scaling=None, device=None) -> torch.Tensor:
    """The frequencies base^(-2i/dims), i < dims / 2, worked out in 64-bit and rounded to 32-bit: for kernels that turn by
    position * frequency without tables.  ``scaling`` = (factor, low, high, original) rescales them by their wavelength
    l = 2 pi / f: kept where l < original / high, divided by ``factor`` where l > original / low, and between the two
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    import math

    if dims % 2 or dims <= 0:
        raise UnsupportedError(f"a rotation over {dims} values, which do not pair")
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = (float(v) for v in scaling)
            length = 2.0 * math.pi / f
            if low > 0 and length > original / low:
                f = f / factor
            elif length >= original / high:
                s = (original / length - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    t = torch.tensor(out, dtype=torch.float64).to(torch.float32)
    return t.to(device) if device is not None else t
