"""Rotary position encoding, "rotate-half" layout: the pair (x[i], x[i + R/2]) turns
by position * theta^(-2i/R) (reference atomserve/model.py:142-185).

The part owns the frequencies and, once per step, the table of (cos, sin) of every
token's angles, which every layer with the same spec then shares.  The angles are
formed and range-reduced in fp64 on the device, so that positions in the tens of
thousands lose nothing; the rotation that uses them is fp32.
"""

import math

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import Position, register


class RotaryHalf(Position):
    capturable = True
    pairs = "half"

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.rotary_dim % 2 or spec.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {spec.rotary_dim} must be positive and even")
        i = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float64)
        self.inv_freq = (1.0 / (float(spec.theta) ** (i / spec.rotary_dim))).to(env.device)

    def prepare(self, step) -> torch.Tensor:
        """cos/sin of this step's tokens, fp32 [T, R/2, 2]; computed once per step and spec."""
        key = ("rope_half", self.spec.rotary_dim, self.spec.theta)
        table = step.shared.get(key)
        if table is None:
            table = torch.empty((step.num_tokens, self.spec.rotary_dim // 2, 2), dtype=torch.float32,
                                device=self.env.device)  # fmt: skip
            ops.rope_table(step.positions, self.inv_freq, table)
            step.shared[key] = table
        return table


register("position", "rope_half", RotaryHalf)


class ScaledRotaryHalf(Position):
    """The same layout with frequencies stretched for long contexts (`ScaledRotarySpec`): low pair indices (fast
    turns) keep their frequency, high ones are divided by `factor`, a linear ramp between; cosines and sines are
    multiplied by 0.1 ln(factor) + 1.  Frequencies are made in fp64 here, angles in fp64 on the device."""

    capturable = True
    pairs = "half"

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.rotary_dim % 2 or s.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {s.rotary_dim} must be positive and even")
        if not (s.theta > 1 and s.factor > 0 and s.original > 0 and s.fast > 0 and s.slow > 0):
            raise ValueError("a scaled rotation needs theta > 1 and positive factor, original, fast and slow")
        i = torch.arange(0, s.rotary_dim // 2, dtype=torch.float64)
        freq = float(s.theta) ** (-2.0 * i / s.rotary_dim)

        def dim_of(turns: float) -> float:
            return s.rotary_dim * math.log(s.original / (2 * math.pi * turns)) / (2 * math.log(s.theta))

        lo = max(math.floor(dim_of(s.fast)), 0)
        hi = min(math.ceil(dim_of(s.slow)), s.rotary_dim - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        self.inv_freq = (freq / s.factor * ramp + freq * (1.0 - ramp)).to(env.device)
        self.magnitude = 0.1 * math.log(s.factor) + 1.0

    def prepare(self, step) -> torch.Tensor:
        key = ("rope_half_scaled", self.spec)
        table = step.shared.get(key)
        if table is None:
            table = torch.empty((step.num_tokens, self.spec.rotary_dim // 2, 2), dtype=torch.float32,
                                device=self.env.device)  # fmt: skip
            ops.rope_table(step.positions, self.inv_freq, table, self.magnitude)
            step.shared[key] = table
        return table


register("position", "rope_half_scaled", ScaledRotaryHalf)


class NeighbourRotary(Position):
    """A rotation whose pairs are neighbours, (2i, 2i + 1), pair i turning by position * f_i (stretched as
    `ScaledRotaryHalf` says where the spec names a factor).  The table is that of the "half" layout, [T, R/2, 2]
    with pair i's cosine and sine at index i; a mixer that takes this part brings its queries and keys into an
    order in which pair i is (i, i + R/2) (a permutation of the rows of their projections, which scores do not see)."""

    capturable = True
    pairs = "neighbours"

    def __init__(self, spec, env):
        super().__init__(spec, env)
        s = spec
        if s.rotary_dim % 2 or s.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {s.rotary_dim} must be positive and even")
        if not s.theta > 1:
            raise ValueError("a rotation needs theta > 1")
        i = torch.arange(0, s.rotary_dim // 2, dtype=torch.float64)
        freq = float(s.theta) ** (-2.0 * i / s.rotary_dim)
        self.magnitude = 1.0
        if s.factor > 0:
            if not (s.original > 0 and s.fast > 0 and s.slow > 0):
                raise ValueError("a scaled rotation needs positive original, fast and slow")

            def dim_of(turns: float) -> float:
                return s.rotary_dim * math.log(s.original / (2 * math.pi * turns)) / (2 * math.log(s.theta))

            lo = max(math.floor(dim_of(s.fast)), 0)
            hi = min(math.ceil(dim_of(s.slow)), s.rotary_dim - 1)
            ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
            freq = freq / s.factor * ramp + freq * (1.0 - ramp)
            self.magnitude = 0.1 * math.log(s.factor) + 1.0
        self.inv_freq = freq.to(env.device)

    def prepare(self, step) -> torch.Tensor:
        key = ("rope_neighbours", self.spec)
        table = step.shared.get(key)
        if table is None:
            table = torch.empty((step.num_tokens, self.spec.rotary_dim // 2, 2), dtype=torch.float32,
                                device=self.env.device)  # fmt: skip
            ops.rope_table(step.positions, self.inv_freq, table, self.magnitude)
            step.shared[key] = table
        return table


register("position", "rope_neighbours", NeighbourRotary)
