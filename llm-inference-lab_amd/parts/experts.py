"""A feed-forward made of many small ones, of which every token uses a few."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..weights.loader import TensorSpec, MATRIX, VECTOR, INIT_ZEROS
from .base import FeedForward, NormedInput
from .feed_forward import interleave_gate_up, pad_columns, pad_rows
from .registry import register_part, build_part


class RoutedExperts(FeedForward):
    """``residual += sum_k w_k expert_{e_k}(h) (+ shared(h))``: a mixture of ``num_experts`` gated
    feed-forwards ``W_down (silu(W_gate h) * (W_up h))`` of width ``expert_size`` without biases.

    The router has ``num_experts + identity`` outputs, ``z = W_router h`` in float32 (``h`` as the
    products read it; stored weights of 16 bits times activations of 16 bits are exact in 32, so
    the matrix product with 32-bit sums is a 32-bit computation).  Scores ``s = softmax(z)`` over
    all outputs.  The choice is made on ``c = s + correction``: the outputs form ``groups`` equal
    groups of neighbours, a group counts as its largest ``c``, only outputs of the ``groups_keep``
    best groups can be chosen (the others count as minus infinity), and among those the ``top``
    largest ``c`` win (ties: the smaller index).  A chosen output's weight is ``s * scale`` (the
    score without the correction, not renormalised).  The last ``identity`` outputs have no
    tensors: their result is ``h`` itself.  ``shared``: a feed-forward part that every token goes
    through, added to the sum.

    ``scoring="sigmoid"``: the scores are ``sigmoid(z)``, each output by itself, instead of the
    softmax.  ``expert_form="relu2"``: the experts are ``W_down relu(W_up h)^2`` without a gate
    matrix.  ``shared_gate=True``: the shared part's result is multiplied by ``sigmoid(w_sg . h)``,
    one number per token (``shared_gate [1, hidden]``), before it is added.

    Tensor roles: ``router [outputs, hidden]``, ``correction [outputs]`` (absent: none), and the
    experts' ``expert_gate``, ``expert_up``, ``expert_down``, each a name with ``{}`` in the place of
    the expert's number.

    How the experts run: rows are sorted by expert into tiles that the grouped matrix product
    walks (``moe_plan``, ``moe_gate_up``, ``moe_down``, ``moe_combine`` of the kernel set) where the
    kernel set has them; otherwise every expert runs over all rows with the kernel set's plain
    products and a row takes the result with its weight, or with none."""

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, tensors: Dict[str, str],
                 identity: int = 0, scale: float = 1.0, groups: int = 1, groups_keep: int = 1,
                 correction: bool = True, shared: Optional[PartSpec] = None, scoring: str = "softmax",
                 expert_form: str = "swiglu", shared_gate: bool = False):
        super().__init__(tensors)
        if scoring not in ("softmax", "sigmoid"):
            raise ValueError(f"a router scores by 'softmax' or 'sigmoid', got {scoring!r}")
        if expert_form not in ("swiglu", "relu2"):
            raise ValueError(f"experts are 'swiglu' or 'relu2' feed-forwards, got {expert_form!r}")
        if shared_gate and shared is None:
            raise ValueError("a gate on the shared part needs a shared part")
        self.scoring, self.expert_form, self.has_shared_gate = scoring, expert_form, bool(shared_gate)
        self.w_shared_gate = None
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.kernel_size = (self.expert_size + 7) // 8 * 8       # (as in ``SwiGLU``: zeros behind an odd width)
        self.num_experts, self.identity, self.top = int(num_experts), int(identity), int(top)
        self.outputs = self.num_experts + self.identity
        self.scale, self.groups, self.groups_keep = float(scale), int(groups), int(groups_keep)
        if self.outputs <= 0 or not 0 < self.top <= self.outputs:
            raise ValueError(f"a router of {self.outputs} outputs cannot take the top {self.top}")
        if self.groups <= 0 or self.outputs % self.groups or not 0 < self.groups_keep <= self.groups:
            raise ValueError(f"{self.outputs} router outputs do not form {self.groups} equal groups "
                             f"of which {self.groups_keep} are kept")
        if self.groups_keep * (self.outputs // self.groups) < self.top:
            raise ValueError("the kept groups hold fewer outputs than a token takes")
        self.has_correction = bool(correction)
        self.shared = build_part("feed_forward", shared) if shared is not None else None
        self.w_router = self.correction = self.w_gate_up = self.w_down = None
        self.gate_up_rows = 0

    def _expert_names(self, e: int):
        t = self.tensor_names
        gate = t["expert_gate"].format(e) if self.expert_form == "swiglu" else None
        return gate, t["expert_up"].format(e), t["expert_down"].format(e)

    def tensor_specs(self):
        t, w, f = self.tensor_names, self.hidden_size, self.expert_size
        specs = {t["router"]: TensorSpec((self.outputs, w), MATRIX)}
        if self.has_correction:
            specs[t["correction"]] = TensorSpec((self.outputs,), VECTOR, INIT_ZEROS)
        for e in range(self.num_experts):
            gate, up, down = self._expert_names(e)
            if gate is not None:
                specs[gate] = TensorSpec((f, w), MATRIX)
            specs[up], specs[down] = TensorSpec((f, w), MATRIX), TensorSpec((w, f), MATRIX)
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        if self.has_shared_gate:
            specs[t["shared_gate"]] = TensorSpec((1, w), MATRIX)
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "experts (hidden size)")
        t = self.tensor_names
        self.w_router = ops.prepare_weight(tensors[t["router"]].contiguous())
        self.correction = (tensors[t["correction"]].float().contiguous() if self.has_correction
                           else torch.zeros(self.outputs, dtype=torch.float32, device=tensors[t["router"]].device))
        # Every expert's gate and up rows interleaved as the paired epilogue reads them, the experts
        # one below the other: one matrix, of which an expert is a run of whole strips of rows.
        names = [self._expert_names(e) for e in range(self.num_experts)]
        if names and self.expert_form == "relu2":
            # (an expert's up rows in whole strips of 16, its down columns zeros behind an odd width)
            self.gate_up_rows = (self.expert_size + 15) // 16 * 16
            self.w_gate_up = ops.prepare_stacked(torch.cat([pad_rows(tensors[u], self.gate_up_rows) for _, u, _ in names],
                                                           dim=0).contiguous(), self.num_experts)
            self.w_down = ops.prepare_stacked(torch.cat([pad_columns(tensors[d], self.gate_up_rows) for _, _, d in names],
                                                        dim=0).contiguous(), self.num_experts)
        elif names:
            gate_up = [interleave_gate_up(tensors[g], tensors[u]) for g, u, _ in names]
            self.gate_up_rows = gate_up[0].shape[0]
            self.w_gate_up = ops.prepare_stacked(torch.cat(gate_up, dim=0).contiguous(), self.num_experts)
            del gate_up
            self.w_down = ops.prepare_stacked(torch.cat([pad_columns(tensors[d], self.kernel_size) for _, _, d in names], dim=0).contiguous(),
                                              self.num_experts)
        if self.shared is not None:
            self.shared.bind(tensors, ops, dtype)
        if self.has_shared_gate:
            self.w_shared_gate = ops.prepare_weight(tensors[t["shared_gate"]].contiguous())

    takes_normed_input = True

    def forward(self, h, residual, ctx):
        ops = self.ops
        if isinstance(h, NormedInput):
            h = h.tensor()
        rows, top = h.shape[0], self.top
        logits = ctx.scratch("experts.logits", (rows, self.outputs), torch.float32)
        ops.linear_logits(h, self.w_router, logits)
        chosen = ctx.scratch("experts.chosen", (rows, top), torch.int32)
        weights = ctx.scratch("experts.weights", (rows, top), torch.float32)
        grouped = self.num_experts and getattr(ops, "moe_grouped", None) is not None and ops.moe_grouped(self.dtype)
        plan = None
        how = {} if self.scoring == "softmax" else dict(scoring=self.scoring)
        if grouped and ops.moe_select_plan_takes(rows, self.outputs):       # few rows: choice and sorting in one launch
            plan = ops.moe_select_plan(logits, self.correction, self.groups, self.groups_keep, self.scale, chosen,
                                       weights, self.num_experts, ctx.scratch, **how)
        else:
            ops.moe_select(logits, self.correction, self.groups, self.groups_keep, self.scale, chosen, weights, **how)
        if grouped:
            self._grouped(h, residual, ctx, chosen, weights, plan)
        elif self.num_experts:
            relu2 = self.expert_form == "relu2"
            act = ctx.scratch("experts.act", (rows, self.gate_up_rows if relu2 else self.kernel_size), self.dtype)
            y = ctx.scratch("experts.out", (rows, self.hidden_size), torch.float32)
            for e in range(self.num_experts):
                if relu2:
                    ops.linear_relu2(h, ops.stacked_member(self.w_gate_up, e), act)
                else:
                    ops.linear_swiglu(h, ops.stacked_member(self.w_gate_up, e), act)
                ops.linear_logits(act, ops.stacked_member(self.w_down, e), y)
                ops.moe_add_chosen(residual, y, chosen, weights, e, e + 1)
            if self.identity:
                ops.moe_add_chosen(residual, h, chosen, weights, self.num_experts, self.outputs)
        elif self.identity:
            ops.moe_add_chosen(residual, h, chosen, weights, self.num_experts, self.outputs)
        if self.shared is not None and not self.has_shared_gate:
            self.shared.forward(h, residual, ctx)
        elif self.shared is not None:
            y = ctx.scratch("experts.shared_out", (rows, self.hidden_size), torch.float32)
            if self.shared.writes_output:
                self.shared.forward_into(h, y, ctx)
            else:
                ops.activation(y, y, "zero")
                self.shared.forward(h, y, ctx)
                if getattr(ctx, "pending", None) is not None:       # (pieces the shared part left belong to y)
                    ops.add_pending(y, ctx.pending)
                    ctx.pending = None
            g = ctx.scratch("experts.shared_gate", (rows, 1), torch.float32)
            ops.linear_logits(h, self.w_shared_gate, g)
            ops.gated_add(residual, y, g, None)

    def _grouped(self, h, residual, ctx, chosen, weights, plan=None):
        ops = self.ops
        if plan is None:
            plan = ops.moe_plan(chosen, self.num_experts, ctx.scratch)
        if self.expert_form == "relu2":
            act = ctx.scratch("experts.act", (plan.capacity, self.gate_up_rows), self.dtype)
            ops.moe_up_relu2(h, self.w_gate_up, plan, act)
        else:
            act = ctx.scratch("experts.act", (plan.capacity, self.kernel_size), self.dtype)
            ops.moe_gate_up(h, self.w_gate_up, plan, act)
        y = ctx.scratch("experts.out", (plan.capacity, self.hidden_size), torch.float32)
        ops.moe_down(act, self.w_down, plan, y)
        ops.moe_combine(residual, y, plan, chosen, weights, self.num_experts, h)     # (identity outputs too)

    @property
    def graph_safe(self):
        return self.shared is None or self.shared.graph_safe

    @property
    def keeps_launches(self):
        return self.shared is None or self.shared.keeps_launches

    def kernel_libraries(self):
        return [("routed_experts", None)] + (self.shared.kernel_libraries() if self.shared is not None else [])

    def weight_bytes(self):
        """What a step of many rows reads: every expert.  (A step of few rows reads the experts
        its rows chose.)"""
        total = 0
        for w in (self.w_router, self.w_gate_up, self.w_down, self.w_shared_gate):
            if w is not None:
                total += w.numel() * w.element_size()
        return total + (self.shared.weight_bytes() if self.shared is not None else 0)


register_part("feed_forward", "routed_experts", RoutedExperts)
