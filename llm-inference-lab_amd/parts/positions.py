"""Position encodings."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import PositionEncoding
from .registry import register_part


class RotaryEmbedding(PositionEncoding):
    """Split-half rotation: with ``lo = x[:d/2]``, ``hi = x[d/2:]`` and
    ``angle_i = position * theta^(-2i/d)``, the result is ``[lo*cos - hi*sin,
    hi*cos + lo*sin]``; angles, sines and cosines in float32.

    Formula: rust/engine/src/runner/model/qwen2/kernels.rs:587-631; frequency
    table: rust/engine/src/runner/model/qwen2/engine.rs:304-306.

    ``rotary_dim`` (default: all of ``dim``): only the first ``rotary_dim`` channels of a head
    turn, channel ``i`` with channel ``i + rotary_dim/2`` by ``position * theta^(-2i/rotary_dim)``,
    the others pass unchanged.  The kernels turn channel ``j`` of a head with channel ``j +
    dim/2``, so the part names the order in which a mixer has to lay out the channels of its
    query and key heads (``channel_order()``: scores do not depend on a common order of both)
    and gives the channels that do not turn the frequency 0: an angle of exactly 0, whose cosine
    is 1 and whose sine is 0.  ``padded_dim``: the mixer's kernels work on heads of that many
    channels (the head's own, then zeros); the table and the order are made for those."""

    def __init__(self, dim: int, theta: float, tensors: Optional[Dict[str, str]] = None,
                 rotary_dim: Optional[int] = None, padded_dim: Optional[int] = None):
        super().__init__(tensors)
        self.dim = int(dim)
        self.rotary_dim = self.dim if rotary_dim is None else int(rotary_dim)
        self.padded_dim = self.dim if padded_dim is None else int(padded_dim)
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.dim:
            raise ValueError(f"a head of {dim} channels of which {self.rotary_dim} turn in pairs")
        if self.padded_dim % 2 or self.padded_dim < self.dim + self.dim % 2:
            raise ValueError(f"heads of {dim} channels do not fit an even {self.padded_dim}")
        self.theta = float(theta)
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / max(self.rotary_dim, 1)
        freq = torch.zeros(self.padded_dim // 2, dtype=torch.float64)
        freq[:self.rotary_dim // 2] = 1.0 / (torch.tensor(self.theta, dtype=torch.float64) ** exponent)
        self.inv_freq = freq.to(torch.float32).to(ops.device)

    def channel_order(self):
        """``order[j]``: which channel of a head, as the model file has it, goes to place ``j`` (-1: a
        zero) so that the pairs ``(j, j + padded_dim/2)`` are the pairs that turn together; None if
        that is the file's own order."""
        if self.rotary_dim == self.dim == self.padded_dim:
            return None
        half, places = self.rotary_dim // 2, self.padded_dim // 2
        still = list(range(self.rotary_dim, self.dim))
        first = (len(still) + 1) // 2
        low = list(range(half)) + still[:first]
        high = list(range(half, 2 * half)) + still[first:]
        return low + [-1] * (places - len(low)) + high + [-1] * (places - len(high))

    keeps_launches = True      # (the frequency table goes to the kernels; ``apply`` depends on the rows only)

    def rotary_table(self):
        return self.inv_freq

    def apply(self, q, k, positions):
        self.ops.rope_inplace(q, positions, self.inv_freq)
        self.ops.rope_inplace(k, positions, self.inv_freq)


class PairRotary(PositionEncoding):
    """Rotation of neighbouring channels: of the first ``rotary_dim`` channels of a head, channel
    ``2i`` turns together with channel ``2i + 1`` by the angle ``position * f_i``, ``(u, v) -> (u cos
    - v sin, v cos + u sin)`` with ``f_i = theta^(-2i/rotary_dim)``; the other channels pass.  Angles,
    sines and cosines are float32.

    ``scaling`` (``factor, original, fast, slow``) stretches the slow frequencies for sequences longer
    than the ``original`` length: with ``n(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta)`` (the
    pair whose wave turns ``t`` times over the original length), ``lo = max(floor(n(fast)), 0)``, ``hi
    = min(ceil(n(slow)), rotary_dim - 1)`` and ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``
    the frequency becomes ``f_i / factor * ramp_i + f_i (1 - ramp_i)``, and sines and cosines are
    multiplied by ``magnitude_slope * ln(factor) + 1``.

    Mixers that take this part ask for ``pair_table()``: the frequencies, how many channels turn,
    and the magnitude."""

    keeps_launches = True

    def __init__(self, dim: int, theta: float, tensors: Optional[Dict[str, str]] = None,
                 rotary_dim: Optional[int] = None, scaling: Optional[Dict[str, float]] = None,
                 magnitude_slope: float = 0.1):
        super().__init__(tensors)
        self.dim = int(dim)
        self.rotary_dim = self.dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.dim:
            raise ValueError(f"a head of {dim} channels of which {self.rotary_dim} turn in pairs")
        self.theta = float(theta)
        self.scaling = dict(scaling) if scaling else None
        if self.scaling is not None:
            missing = [k for k in ("factor", "original", "fast", "slow") if k not in self.scaling]
            if missing:
                raise ValueError(f"frequency scaling needs {missing}")
        self.magnitude_slope = float(magnitude_slope)
        self.freq: Optional[torch.Tensor] = None
        self.magnitude = 1.0

    def frequencies(self):
        """``(f [rotary_dim / 2] as Python floats, magnitude)``, worked out in double precision."""
        import math
        n = self.rotary_dim
        f = [self.theta ** (-2.0 * i / n) for i in range(n // 2)]
        sc = self.scaling
        if sc is None:
            return f, 1.0
        factor, original = float(sc["factor"]), float(sc["original"])

        def pair_of(turns):
            return n * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(pair_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(sc["slow"]))), n - 1)
        span = max(hi - lo, 0.001)
        out = []
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / span, 0.0), 1.0)
            out.append(fi / factor * ramp + fi * (1.0 - ramp))
        return out, self.magnitude_slope * math.log(factor) + 1.0

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        f, self.magnitude = self.frequencies()
        self.freq = torch.tensor(f, dtype=torch.float64).to(torch.float32).to(ops.device)

    def pair_table(self):
        return self.freq, self.rotary_dim, self.magnitude


class NoPosition(PositionEncoding):
    """No position encoding: queries and keys are used as projected."""

    keeps_launches = True

    def __init__(self, tensors: Optional[Dict[str, str]] = None, **_):
        super().__init__(tensors)

    def apply(self, q, k, positions):
        return None


register_part("position", "rope", RotaryEmbedding)
register_part("position", "rope_pairs", PairRotary)
register_part("position", "none", NoPosition)
