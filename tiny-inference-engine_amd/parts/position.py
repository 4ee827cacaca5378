"""Rotary position encoding, rotate-half pairing.

``inv_freq[i] = 1 / theta^(2i / head_dim)`` for i < head_dim / 2, computed in
float32 exactly as ``src/backend/rope.h:9-13`` does; the angle of pair
(i, i + head_dim/2) at position p is ``float(p) * inv_freq[i]``
(``src/backend/cpu/cpu_backend.cpp:180-188``). The whole head is rotated; queries
and keys are, values are not. Parameters: ``head_dim``, ``theta``.

For designs that have them: ``rotary_dim`` r (even, at most ``head_dim``): only the first r dimensions of a head
rotate, dimension i paired with i + r/2 and ``inv_freq[i] = theta^(-2i / r)``, the others pass unchanged;
``scaling_factor`` f (linear position scaling): every frequency is divided by f.
"""

from __future__ import annotations

import numpy as np
import torch

from .. import kernels
from ..errors import InvalidArgument
from .base import Position, register_part


@register_part("position", "rope_neox")
class RopeNeox(Position):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True

    def __init__(self, params):
        super().__init__(params)
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.rotary_dim = int(params.get("rotary_dim") or self.head_dim)
        self.scaling_factor = float(params.get("scaling_factor") or 1.0)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise InvalidArgument(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        if not self.scaling_factor > 0:
            raise InvalidArgument(f"the position scaling factor must be positive, got {self.scaling_factor}")
        if not self.theta > 0:
            raise InvalidArgument(f"rope theta must be positive, got {self.theta}")
        self.inv_freq: torch.Tensor = None

    def host_inv_freq(self) -> np.ndarray:
        i = np.arange(self.rotary_dim // 2, dtype=np.float32)
        exponent = (np.float32(2.0) * i) / np.float32(self.rotary_dim)
        freq = (np.float32(1.0) / np.power(np.float32(self.theta), exponent, dtype=np.float32)).astype(np.float32)
        if self.scaling_factor != 1.0:
            # in double precision, rounded once: a float32 division of an already rounded frequency would round twice
            i64 = np.arange(self.rotary_dim // 2, dtype=np.float64)
            freq = (np.power(float(self.theta), -2.0 * i64 / self.rotary_dim) / self.scaling_factor).astype(np.float32)
        return freq

    def load(self, fetch, mode, device) -> None:
        self.inv_freq = torch.from_numpy(self.host_inv_freq()).to(device)

    def rotary_table(self):
        return self.inv_freq, self.rotary_dim, "rotate_half"

    def angles(self, ctx) -> torch.Tensor:
        """cos | sin of this step's positions, ``[T, head_dim]`` float32: computed once a step, shared by all layers."""
        key = ("rope_angles", self.rotary_dim, self.theta, self.scaling_factor)
        table = ctx.notes.get(key)
        if table is None:
            table = ctx.scratch(f"rope.angles:{self.rotary_dim}:{self.theta}:{self.scaling_factor}",
                                (ctx.num_tokens, self.rotary_dim), torch.float32)
            kernels.rope_angles(ctx.batch.positions, self.inv_freq, table)
            ctx.notes[key] = table
        return table


@register_part("position", "none")
class NoPosition(Position):
    """No position encoding: queries and keys are left as they are."""

    capturable = True
    replayable = True

    def rotary_table(self):
        return None, 0, "none"
