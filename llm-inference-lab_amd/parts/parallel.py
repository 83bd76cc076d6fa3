"""A mixer made of two: both on one input, their results summed."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from .base import Mixer, NormedInput, PendingSums
from .registry import register_part, build_part


class ParallelMixers(Mixer):
    """``left_scale * left(h) + right_scale * right(h)``: two mixers of any registered kind read
    the same input; their float32 results are summed with two fixed weights.  At most one of the
    two keeps a per-token cache (the run's pages are that one's); per-request state of both is kept
    under the names they give it, which must differ."""

    writes_output = True
    takes_normed_input = True      # (each of the two takes it as it can; the norm itself runs at most once)

    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0,
                 tensors: Optional[Dict[str, str]] = None):
        super().__init__(tensors)
        self.left, self.right = build_part("mixer", left), build_part("mixer", right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        if self.left.cache_spec() is not None and self.right.cache_spec() is not None:
            raise ValueError("the two mixers share one run of the schedule: only one of them may keep a cache")
        clash = set(self.left.state_spec()) & set(self.right.state_spec())
        if clash:
            raise ValueError(f"both mixers keep per-request state called {sorted(clash)}")

    def members(self):
        return [self.left, self.right]

    def tensor_specs(self):
        specs = dict(self.left.tensor_specs())
        specs.update(self.right.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for m in self.members():
            m.bind(tensors, ops, dtype)

    def cache_spec(self):
        return self.left.cache_spec() or self.right.cache_spec()

    def state_spec(self):
        spec = dict(self.left.state_spec())
        spec.update(self.right.state_spec())
        return spec

    @property
    def graph_safe(self):
        return all(m.graph_safe for m in self.members())

    @property
    def keeps_launches(self):
        return all(m.keeps_launches for m in self.members())

    def kernel_libraries(self):
        return [("stream_ops", None)] + [lib for m in self.members() for lib in m.kernel_libraries()]

    def _result(self, mixer, name, h, shape, ctx, entry):
        if isinstance(h, NormedInput) and not mixer.takes_normed_input:
            h = h.tensor()
        y = ctx.scratch(name, shape, torch.float32)
        if mixer.writes_output:
            mixer.forward_into(h, y, ctx, entry)
        else:                               # (a mixer made to add into the stream: into zeros)
            self.ops.activation(y, y, "zero")
            mixer.forward(h, y, ctx, entry)
            pending = getattr(ctx, "pending", None)
            if pending is not None:
                self.ops.add_pending(y, pending)
                ctx.pending = None
        return y

    def forward_into(self, h, out, ctx, entry):
        shape = tuple(out.shape)
        y1 = self._result(self.left, "parallel.left", h, shape, ctx, entry)
        y2 = self._result(self.right, "parallel.right", h, shape, ctx, entry)
        self.ops.scaled_sum(out, y1, self.left_scale, y2, self.right_scale)

    def forward(self, h, residual, ctx, entry):
        y = ctx.scratch("parallel.sum", (1,) + tuple(residual.shape), torch.float32)
        self.forward_into(h, y[0], ctx, entry)
        self.ops.add_pending(residual, PendingSums(y, 1))

    def weight_bytes(self):
        return sum(m.weight_bytes() for m in self.members())


register_part("mixer", "parallel", ParallelMixers)
