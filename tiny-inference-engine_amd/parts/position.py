"""Rotary position encoding, rotate-half pairing.

``inv_freq[i] = 1 / theta^(2i / head_dim)`` for i < head_dim / 2, computed in
float32 exactly as ``src/backend/rope.h:9-13`` does; the angle of pair
(i, i + head_dim/2) at position p is ``float(p) * inv_freq[i]``
(``src/backend/cpu/cpu_backend.cpp:180-188``). The whole head is rotated; queries
and keys are, values are not. Parameters: ``head_dim``, ``theta``.

For designs that have them: ``rotary_dim`` r (even, at most ``head_dim``): only the first r dimensions of a head
rotate, dimension i paired with i + r/2 and ``inv_freq[i] = theta^(-2i / r)``, the others pass unchanged;
``scaling_factor`` f (linear position scaling): every frequency is divided by f.

``rope_yarn`` is a rotation whose frequencies are stretched for contexts longer than the one they were made for
(YaRN): with ``f_i = theta^(-2i / r)`` over the r rotated dimensions and ``scaling`` = (factor, original, fast, slow),

    dim(t) = r ln(original / (2 pi t)) / (2 ln theta),  lo = max(floor(dim(fast)), 0),  hi = min(ceil(dim(slow)), r - 1),
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),   frequency_i = f_i / factor * ramp_i + f_i (1 - ramp_i),

and both the cosine and the sine are multiplied by ``0.1 ln(factor) + 1``. Without ``scaling`` it is the plain
rotation. ``pairing`` says which dimensions form a pair: ``rotate_half`` (i, i + r/2) or ``interleaved`` (2i, 2i + 1).
Parameters: ``head_dim``, ``theta``, ``rotary_dim``, ``pairing``, ``scaling``.

``rope_banded`` scales the frequencies by bands of wavelength: with ``f_i = theta^(-2i / r)``, wavelength
``L_i = 2 pi / f_i`` and ``scaling`` = (factor, low, high, original), a pair keeps ``f_i`` where
``L_i < original / high``, turns with ``f_i / factor`` where ``L_i > original / low``, and in between, with
``s = (original / L_i - low) / (high - low)``, with ``(1 - s) f_i / factor + s f_i``. Amplitudes stay 1. Without
``scaling`` it is the plain rotation. Parameters as for ``rope_yarn``.
"""

from __future__ import annotations

import math

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


@register_part("position", "rope_yarn")
class RopeYarn(Position):
    capturable = True
    replayable = True

    def __init__(self, params):
        super().__init__(params)
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.rotary_dim = int(params.get("rotary_dim") or self.head_dim)
        self.pairing = params.get("pairing", "rotate_half")
        self.scaling = dict(params["scaling"]) if params.get("scaling") else None
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise InvalidArgument(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        if self.pairing not in ("rotate_half", "interleaved"):
            raise InvalidArgument(f"pairs rotate as 'rotate_half' or 'interleaved', not '{self.pairing}'")
        if not self.theta > 0 or self.theta == 1.0:
            raise InvalidArgument(f"rope theta must be positive and not 1, got {self.theta}")
        self.amplitude = 1.0
        if self.scaling is not None:
            for key in ("factor", "original", "fast", "slow"):
                if not float(self.scaling[key]) > 0:
                    raise InvalidArgument(f"rope scaling {key} must be positive, got {self.scaling[key]}")
            self.amplitude = 0.1 * math.log(float(self.scaling["factor"])) + 1.0
        self.inv_freq: torch.Tensor = None

    def host_inv_freq(self) -> np.ndarray:
        """The frequencies in double precision, rounded to float32 once."""
        r = self.rotary_dim
        i = np.arange(r // 2, dtype=np.float64)
        freq = np.power(self.theta, -2.0 * i / r)
        if self.scaling is not None:
            factor, original = float(self.scaling["factor"]), float(self.scaling["original"])

            def dim_of(turns: float) -> float:
                return r * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

            lo = max(math.floor(dim_of(float(self.scaling["fast"]))), 0)
            hi = min(math.ceil(dim_of(float(self.scaling["slow"]))), r - 1)
            ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            freq = freq / factor * ramp + freq * (1.0 - ramp)
        return freq.astype(np.float32)

    def load(self, fetch, mode, device) -> None:
        self.inv_freq = torch.from_numpy(self.host_inv_freq()).to(device)

    def rotary_table(self):
        return self.inv_freq, self.rotary_dim, self.pairing

    def angles(self, ctx) -> torch.Tensor:
        """amplitude * (cos | sin) of this step's positions, ``[T, rotary_dim]`` float32: once a step for all layers
        with the same frequencies."""
        key = ("rope_yarn", self.rotary_dim, self.theta, repr(sorted((self.scaling or {}).items())))
        table = ctx.notes.get(key)
        if table is None:
            table = ctx.scratch("rope.angles:" + repr(key), (ctx.num_tokens, self.rotary_dim), torch.float32)
            kernels.rope_angles(ctx.batch.positions, self.inv_freq, table, self.amplitude)
            ctx.notes[key] = table
        return table


@register_part("position", "rope_banded")
class RopeBanded(RopeYarn):
    """A rotation whose long wavelengths are stretched by a factor, short ones kept, with a linear blend between."""

    def __init__(self, params):
        scaling = dict(params["scaling"]) if params.get("scaling") else None
        super().__init__({**params, "scaling": None})
        self.scaling = scaling
        if scaling is not None:
            for key in ("factor", "low", "high", "original"):
                if not float(scaling[key]) > 0:
                    raise InvalidArgument(f"rope scaling {key} must be positive, got {scaling[key]}")
            if float(scaling["high"]) == float(scaling["low"]):
                raise InvalidArgument("rope scaling needs 'high' and 'low' to differ")

    def host_inv_freq(self) -> np.ndarray:
        r = self.rotary_dim
        i = np.arange(r // 2, dtype=np.float64)
        freq = np.power(self.theta, -2.0 * i / r)
        if self.scaling is not None:
            factor, original = float(self.scaling["factor"]), float(self.scaling["original"])
            low, high = float(self.scaling["low"]), float(self.scaling["high"])
            wavelength = 2.0 * math.pi / freq
            blend = (original / wavelength - low) / (high - low)
            between = (1.0 - blend) * freq / factor + blend * freq
            freq = np.where(wavelength < original / high, freq,
                            np.where(wavelength > original / low, freq / factor, between))
        return freq.astype(np.float32)

    def angles(self, ctx) -> torch.Tensor:
        key = ("rope_banded", self.rotary_dim, self.theta, repr(sorted((self.scaling or {}).items())))
        table = ctx.notes.get(key)
        if table is None:
            table = ctx.scratch("rope.angles:" + repr(key), (ctx.num_tokens, self.rotary_dim), torch.float32)
            kernels.rope_angles(ctx.batch.positions, self.inv_freq, table, 1.0)
            ctx.notes[key] = table
        return table
