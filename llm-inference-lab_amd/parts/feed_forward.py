"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.loader import TensorSpec, MATRIX
from .base import FeedForward, NormedInput
from .registry import register_part

PAIR = 16   # rows of the gate matrix and of the up matrix alternate in runs of 16


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Stack gate ``[I, K]`` and up ``[I, K]`` as ``[2*ceil16(I), K]``: rows
    ``32b .. 32b+15`` are gate rows ``16b .. 16b+15`` and rows ``32b+16 ..
    32b+31`` the up rows of the same outputs, so one 16-column tile of the
    product holds gate and the next one up for the same 16 outputs (rows past
    ``I`` are zero)."""
    inter, k = gate.shape
    padded = (inter + PAIR - 1) // PAIR * PAIR
    out = torch.zeros((2 * padded, k), dtype=gate.dtype, device=gate.device)
    view = out.view(padded // PAIR, 2, PAIR, k)
    g = torch.zeros((padded, k), dtype=gate.dtype, device=gate.device)
    u = torch.zeros((padded, k), dtype=gate.dtype, device=gate.device)
    g[:inter] = gate
    u[:inter] = up
    view[:, 0] = g.view(padded // PAIR, PAIR, k)
    view[:, 1] = u.view(padded // PAIR, PAIR, k)
    return out


def pad_columns(w: torch.Tensor, columns: int) -> torch.Tensor:
    """``w [n, k]`` with zero columns behind it up to ``columns``."""
    if w.shape[1] == columns:
        return w.contiguous()
    out = torch.zeros((w.shape[0], columns), dtype=w.dtype, device=w.device)
    out[:, :w.shape[1]] = w
    return out


def pad_rows(w: torch.Tensor, rows: int) -> torch.Tensor:
    """``w [n, k]`` with zero rows below it up to ``rows``."""
    if w.shape[0] == rows:
        return w.contiguous()
    out = torch.zeros((rows, w.shape[1]), dtype=w.dtype, device=w.device)
    out[:w.shape[0]] = w
    return out


class SwiGLU(FeedForward):
    """``residual += (silu(h Wg^T) * (h Wu^T)) Wd^T`` with ``silu(z) = z / (1 +
    exp(-z))``; accumulators, the sigmoid and the product in float32.

    Formula: rust/engine/src/runner/model/qwen2/engine.rs:1234-1294,
    rust/engine/src/runner/model/qwen2/kernels.rs:1469-1486.

    ``activation="gelu_tanh"``: the gate goes through ``0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715
    z^3)))`` instead of ``silu``; everything else stays."""

    ACTIVATIONS = ("silu", "gelu_tanh")

    def __init__(self, hidden_size: int, intermediate_size: int, tensors: Dict[str, str],
                 activation: str = "silu"):
        super().__init__(tensors)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"a gated feed-forward takes the activations {self.ACTIVATIONS}, got '{activation}'")
        self.activation = activation
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        # the kernels' inner sizes are multiples of 8: an intermediate size that is not is laid out
        # with zero rows of gate and up (whose activation is 0) and zero columns of down behind it
        self.kernel_size = (self.intermediate_size + 7) // 8 * 8
        self.w_gate_up = self.w_down = None

    def tensor_specs(self):
        t, h, i = self.tensor_names, self.hidden_size, self.intermediate_size
        return {
            t["gate_weight"]: TensorSpec((i, h), MATRIX),
            t["up_weight"]: TensorSpec((i, h), MATRIX),
            t["down_weight"]: TensorSpec((h, i), MATRIX),
        }

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "feed-forward (hidden size)")
        t = self.tensor_names
        self.w_gate_up = ops.prepare_weight(
            interleave_gate_up(tensors[t["gate_weight"]], tensors[t["up_weight"]]))
        self.w_down = ops.prepare_weight(pad_columns(tensors[t["down_weight"]], self.kernel_size))

    takes_normed_input = True
    keeps_launches = True

    def _act(self):
        """(silu is what the kernels do when they are told nothing)"""
        return () if self.activation == "silu" else (self.activation,)

    def _act_kw(self):
        return {} if self.activation == "silu" else dict(activation=self.activation)

    def forward_pending(self, h, out, ctx):
        """The result into ``out`` (float32), or, where the down product is left in pieces, the
        pieces themselves (``PendingSums``; ``out`` is not written): for a caller that does
        something else with the result than add it to the stream."""
        rows = h.shape[0]
        if isinstance(h, NormedInput):
            h = h.tensor()
        act = ctx.scratch("swiglu.act", (rows, self.kernel_size), self.dtype)
        self.ops.linear_swiglu(h, self.w_gate_up, act, *self._act())
        splits = self.ops.split_count(rows, self.dtype, self.hidden_size, self.kernel_size)
        if splits > 1:
            parts = ctx.scratch("swiglu.pieces", (splits, rows, self.hidden_size), torch.float32)
            return self.ops.linear_partials(act, self.w_down, parts, splits)
        self.ops.linear_logits(act, self.w_down, out)
        return None

    def forward(self, h, residual, ctx):
        rows = h.shape[0]
        act = ctx.scratch("swiglu.act", (rows, self.kernel_size), self.dtype)
        fuse = isinstance(h, NormedInput) and self.ops.can_fuse(rows, self.dtype, self.hidden_size,
                                                                 self.w_gate_up.shape[0])
        rms = h.rms() if fuse else None      # (folds pieces still owed to the stream; else the norm does)
        if rms is not None:
            self.ops.fused_norm_swiglu(rms[0], rms[2], rms[3], self.w_gate_up, act, **self._act_kw())
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            self.ops.linear_swiglu(h, self.w_gate_up, act, *self._act())
        splits = self.ops.split_count(rows, self.dtype, self.hidden_size, self.kernel_size)
        if splits > 1 and hasattr(ctx, "pending") and ctx.pending is None:
            # a narrow output: the product is cut along the inner size so that it spreads
            # over the chip, and its pieces are left for the next reader of the stream
            parts = ctx.scratch("swiglu.pieces", (splits, rows, self.hidden_size), torch.float32)
            ctx.pending = self.ops.linear_partials(act, self.w_down, parts, splits)
        else:
            self.ops.linear_residual(act, self.w_down, residual, None)

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in (self.w_gate_up, self.w_down))


class DenseFeedForward(FeedForward):
    """``W_down act(W_up h)`` with no gate and no biases; ``activation="relu2"``: ``act(z) =
    max(z, 0) ** 2``, taken on the float32 sums of the first product and rounded once."""

    writes_output = True
    keeps_launches = True
    ACTIVATIONS = ("relu2",)

    def __init__(self, hidden_size: int, intermediate_size: int, tensors: Dict[str, str],
                 activation: str = "relu2"):
        super().__init__(tensors)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"a dense feed-forward takes the activations {self.ACTIVATIONS}, got '{activation}'")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.kernel_size = (self.intermediate_size + 7) // 8 * 8      # (as in ``SwiGLU``: zeros behind an odd width)
        self.activation = activation
        self.w_up = self.w_down = None

    def tensor_specs(self):
        t, h, i = self.tensor_names, self.hidden_size, self.intermediate_size
        return {t["up_weight"]: TensorSpec((i, h), MATRIX), t["down_weight"]: TensorSpec((h, i), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "feed-forward (hidden size)")
        t = self.tensor_names
        self.w_up = ops.prepare_weight(pad_rows(tensors[t["up_weight"]], self.kernel_size))
        self.w_down = ops.prepare_weight(pad_columns(tensors[t["down_weight"]], self.kernel_size))

    def _activated(self, h, ctx):
        rows = h.shape[0]
        act = ctx.scratch("dense_ffn.act", (rows, self.kernel_size), self.dtype)
        fused = getattr(self.ops, "linear_relu2", None) if self.activation == "relu2" else None
        if fused is not None:
            fused(h, self.w_up, act)            # the activation is the first product's epilogue
            return act
        sums = ctx.scratch("dense_ffn.sums", (rows, self.kernel_size), torch.float32)
        self.ops.linear_logits(h, self.w_up, sums)
        self.ops.activation(sums, act, self.activation)
        return act

    def forward_into(self, h, out, ctx):
        self.ops.linear_logits(self._activated(h, ctx), self.w_down, out)

    def forward(self, h, residual, ctx):
        if isinstance(h, NormedInput):
            h = h.tensor()
        self.ops.linear_residual(self._activated(h, ctx), self.w_down, residual, None)

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in (self.w_up, self.w_down))


register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "dense", DenseFeedForward)
