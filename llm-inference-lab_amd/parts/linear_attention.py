"""Mixers with a recurrent state instead of a cache of keys and values."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.loader import TensorSpec, MATRIX, VECTOR, INIT_NORM
from .base import Mixer, NormedInput, PendingSums, project_normed
from .registry import register_part


class GatedLinearAttention(Mixer):
    """Linear attention with a decay per key channel and a matrix-valued state per head.

    With ``D = key_dim`` and ``E = value_dim``: ``q = Wq h * q_scale`` (``q_scale`` defaults to
    ``D ** -0.5``), ``k = Wk h`` (``heads x D``), ``v = Wv h`` (``heads x E``); decays ``a =
    sigmoid(W2 (W1 h) + b2) ** (1 / tau)`` (``heads x D``, through a projection of rank
    ``decay_rank``); per head, token by token::

        S_t = diag(a_t) S_(t-1) + k_t v_t^T          (S is D x E, zero at a sequence's start)
        o_t = S_t^T q_t

    then every head's ``o_t`` is divided by its root mean square over ``E`` (``eps`` inside the
    root) and multiplied by one weight of size ``E`` that all heads share, the heads are put
    side by side, multiplied by ``silu(Wg h)`` and projected by ``Wo``.

    The state lives in float32 in one slot per request (``state_spec``) and is carried from
    step to step; the decays, the recurrence and the norm are float32 throughout, and the
    projections reach them unrounded (32-bit sums of the matrix products)."""

    writes_output = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay_rank: int,
                 tau: float, tensors: Dict[str, str], norm_eps: float = 1e-6, q_scale: Optional[float] = None):
        super().__init__(tensors)
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        # (None: the rank is whatever the model file's decay tensors have)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        if self.tau <= 0:
            raise ValueError(f"tau must be positive, got {tau}")
        self.q_scale = float(q_scale) if q_scale is not None else self.key_dim ** -0.5
        self.w_in = self.w_o = self.w_decay = self.b_decay = self.norm_weight = None

    @property
    def qk_size(self):
        return self.num_heads * self.key_dim

    @property
    def v_size(self):
        return self.num_heads * self.value_dim

    def tensor_specs(self):
        t, w = self.tensor_names, self.hidden_size
        return {
            t["q_weight"]: TensorSpec((self.qk_size, w), MATRIX),
            t["k_weight"]: TensorSpec((self.qk_size, w), MATRIX),
            t["v_weight"]: TensorSpec((self.v_size, w), MATRIX),
            t["gate_weight"]: TensorSpec((self.v_size, w), MATRIX),
            t["o_weight"]: TensorSpec((w, self.v_size), MATRIX),
            t["out_norm"]: TensorSpec((self.value_dim,), VECTOR, INIT_NORM),
            t["decay_down"]: TensorSpec((self.decay_rank, w), MATRIX),
            t["decay_up"]: TensorSpec((self.qk_size, self.decay_rank), MATRIX),
            t["decay_bias"]: TensorSpec((self.qk_size,), VECTOR),
        }

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_linear_attention_sizes(self.num_heads, self.key_dim, self.value_dim)
        ops.check_product_sizes(self.hidden_size, dtype, "linear attention projections (hidden size)")
        ops.check_product_sizes(self.v_size, dtype, "linear attention output projection (heads * value size)")
        t = self.tensor_names
        rank = int(tensors[t["decay_down"]].shape[0])
        if int(tensors[t["decay_up"]].shape[1]) != rank:
            raise ValueError(f"{t['decay_down']} has {rank} rows but {t['decay_up']} has "
                             f"{int(tensors[t['decay_up']].shape[1])} columns: the two factors of the decay "
                             f"projection do not fit")
        self.decay_rank = rank
        # one product for q, k, v, the gate and the low-rank input of the decays
        self.offsets = {}
        at = 0
        rows = []
        for role in ("q_weight", "k_weight", "v_weight", "gate_weight", "decay_down"):
            self.offsets[role] = at
            rows.append(tensors[t[role]])
            at += rows[-1].shape[0]
        self.in_size = at
        self.w_in = ops.prepare_weight(torch.cat(rows, dim=0).contiguous())
        self.w_o = ops.prepare_weight(tensors[t["o_weight"]].contiguous())
        # the second factor of the decays is applied in float32, inside the decay kernel
        self.w_decay = tensors[t["decay_up"]].float().contiguous()
        self.b_decay = tensors[t["decay_bias"]].float().contiguous()
        self.norm_weight = tensors[t["out_norm"]].float().contiguous()

    def _min_chunk(self) -> int:
        rules = getattr(self.ops, "rules", None)
        return int(getattr(rules, "scan_min_chunk", 16))

    def state_spec(self):
        return {"s": ((self.num_heads, self.key_dim, self.value_dim), torch.float32)}

    def forward_into(self, h, out, ctx, entry):
        ops, rows, o = self.ops, h.shape[0], self.offsets
        proj = ctx.scratch("linear_attention.proj", (rows, self.in_size), torch.float32)
        ops.linear_logits(h, self.w_in, proj)
        decay = ctx.scratch("linear_attention.decay", (rows, self.qk_size), torch.float32)
        ops.gla_decay(proj[:, o["decay_down"]:], self.decay_rank, self.w_decay, self.b_decay, self.tau, decay)
        parts = ctx.scratch("linear_attention.parts",
                            (rows, self.num_heads, ops.gla_slices(self.key_dim), self.value_dim), torch.float32)
        state = entry.state["s"]
        # room for the chunks of a long portion: at most rows / (smallest chunk) + requests
        most = rows // max(1, self._min_chunk()) + ctx.max_reqs
        chunk_state = ctx.scratch("linear_attention.chunk_state",
                                  (most, self.num_heads, self.key_dim, self.value_dim), torch.float32)
        chunk_decay = ctx.scratch("linear_attention.chunk_decay", (most, self.num_heads, self.key_dim), torch.float32)

        def scan():
            # (how many requests the step has and how long the longest portion is are read when
            # the launch is made, also when it is made again from a kept sequence of calls)
            pick = getattr(ops, "gla_scan_chunk", None)
            chunk = pick(rows, ctx.max_q_len, self.num_heads, self.value_dim) if pick is not None else 0
            ops.gla_scan(proj, o["q_weight"], o["k_weight"], o["v_weight"], decay, self.q_scale, self.num_heads,
                         self.key_dim, self.value_dim, state, ctx.all_q_start, ctx.all_req_rows, ctx.n_reqs, parts,
                         chunk, chunk_state if chunk else None, chunk_decay if chunk else None)
        live = getattr(ops, "live", None)
        if live is not None:
            live(scan)
        else:
            scan()
        mixed = ctx.scratch("linear_attention.out", (rows, self.v_size), self.dtype)
        ops.gla_output(parts, self.num_heads, self.key_dim, self.value_dim, self.norm_weight, self.norm_eps, proj,
                       o["gate_weight"], mixed)
        ops.linear_logits(mixed, self.w_o, out)

    def forward(self, h, residual, ctx, entry):
        if isinstance(h, NormedInput):
            h = h.tensor()
        y = ctx.scratch("linear_attention.sum", (1,) + tuple(residual.shape), torch.float32)
        self.forward_into(h, y[0], ctx, entry)
        self.ops.add_pending(residual, PendingSums(y, 1))

    keeps_launches = True

    def kernel_libraries(self):
        return [("linear_attention", None)]

    def weight_bytes(self):
        return sum(w.numel() * w.element_size()
                   for w in (self.w_in, self.w_o, self.w_decay, self.b_decay, self.norm_weight) if w is not None)


class DeltaRuleAttention(Mixer):
    """A recurrent mixer whose matrix-valued state forgets along the current key before it
    learns the new pair (a generalised delta rule).

    With ``D = key_dim`` and ``E = value_dim`` (default ``D``): ``r = Wr h``, ``k = Wk h`` (``heads x
    D``), ``v = Wv h`` (``heads x E``); decays ``w = exp(-decay_scale * sigmoid(W2 tanh(W1 h) + w0))``
    and removal rates ``a = sigmoid(Wa h + ba)``, both per head and key channel; per head, token by
    token, with the unit key ``u = k / sqrt(|k|^2 + key_eps)``::

        S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T     (S is D x E; decay and removal
        o_t = S_t^T r_t                                                        both act on S_(t-1))

    then every head's ``o_t`` is divided by its root mean square over ``E`` (``norm_eps`` inside the
    root), the heads are put side by side, multiplied by a weight of all heads' size and by
    ``sigmoid(Wg h)`` (``gate="silu"``: by ``silu``), and projected by ``Wo``.

    The state lives in float32 in one slot per request (``state_spec``), zero at a sequence's
    start, and is carried from step to step; decays, rates, the unit key, the recurrence and the
    norm are float32 throughout, and the projections reach them unrounded (the 32-bit sums of the
    matrix products).  ``decay_rank`` None: the rank of the decay projection is whatever the model
    file's tensors have.

    Tensor roles: ``r_weight, k_weight, v_weight, gate_weight, rate_weight, rate_bias, decay_down,
    decay_up, decay_bias, out_norm, o_weight``."""

    writes_output = True
    takes_normed_input = True
    keeps_launches = True
    DEFAULT_DECAY_SCALE = 0.6065306597126334      # exp(-1/2)

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, tensors: Dict[str, str],
                 value_dim: Optional[int] = None, decay_rank: Optional[int] = None,
                 decay_scale: float = DEFAULT_DECAY_SCALE, key_eps: float = 1e-6, norm_eps: float = 1e-6,
                 gate: str = "sigmoid"):
        super().__init__(tensors)
        self.hidden_size, self.num_heads, self.key_dim = int(hidden_size), int(num_heads), int(key_dim)
        self.file_value_dim = self.key_dim if value_dim is None else int(value_dim)      # as the model file has it
        # (the products' inner sizes are multiples of 8: zeros behind a head's value channels)
        self.value_dim = (self.file_value_dim + 7) // 8 * 8
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.decay_scale, self.key_eps, self.norm_eps = float(decay_scale), float(key_eps), float(norm_eps)
        if gate not in ("sigmoid", "silu"):
            raise ValueError(f"the output gate is 'sigmoid' or 'silu', got {gate!r}")
        self.gate = gate
        self.w_in = self.w_o = self.w_decay = self.b_decay = self.b_rate = self.norm_weight = None
        self.offsets = {}
        self.in_size = 0

    @property
    def qk_size(self):
        return self.num_heads * self.key_dim

    @property
    def v_size(self):
        return self.num_heads * self.value_dim

    def tensor_specs(self):
        t, w = self.tensor_names, self.hidden_size
        file_v = self.num_heads * self.file_value_dim
        return {
            t["r_weight"]: TensorSpec((self.qk_size, w), MATRIX),
            t["k_weight"]: TensorSpec((self.qk_size, w), MATRIX),
            t["v_weight"]: TensorSpec((file_v, w), MATRIX),
            t["gate_weight"]: TensorSpec((file_v, w), MATRIX),
            t["rate_weight"]: TensorSpec((self.qk_size, w), MATRIX),
            t["rate_bias"]: TensorSpec((self.qk_size,), VECTOR),
            t["decay_down"]: TensorSpec((self.decay_rank, w), MATRIX),
            t["decay_up"]: TensorSpec((self.qk_size, self.decay_rank), MATRIX),
            t["decay_bias"]: TensorSpec((self.qk_size,), VECTOR),
            t["out_norm"]: TensorSpec((file_v,), VECTOR, INIT_NORM),
            t["o_weight"]: TensorSpec((w, file_v), MATRIX),
        }

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_delta_rule_sizes(self.num_heads, self.key_dim, self.value_dim)
        ops.check_product_sizes(self.hidden_size, dtype, "delta rule projections (hidden size)")
        ops.check_product_sizes(self.v_size, dtype, "delta rule output projection (heads * value size)")
        t = self.tensor_names
        rank = int(tensors[t["decay_down"]].shape[0])
        if int(tensors[t["decay_up"]].shape[1]) != rank:
            raise ValueError(f"{t['decay_down']} has {rank} rows but {t['decay_up']} has "
                             f"{int(tensors[t['decay_up']].shape[1])} columns: the two factors of the decay "
                             f"projection do not fit")
        self.decay_rank = rank
        e, ek = self.file_value_dim, self.value_dim

        def value_heads(x):
            """Rows (or entries) of the heads' ``e`` value channels -> of ``ek``, zeros behind."""
            if e == ek:
                return x
            per_head = x.unflatten(0, (self.num_heads, e))
            zeros = torch.zeros((self.num_heads, ek - e) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
            return torch.cat([per_head, zeros], dim=1).flatten(0, 1)
        # one product for r, k, v, the gate, the rates and the low-rank input of the decays
        self.offsets, at, rows = {}, 0, []
        for role in ("r_weight", "k_weight", "v_weight", "gate_weight", "rate_weight", "decay_down"):
            self.offsets[role] = at
            rows.append(value_heads(tensors[t[role]]) if role in ("v_weight", "gate_weight") else tensors[t[role]])
            at += rows[-1].shape[0]
        self.in_size = at
        self.w_in = ops.prepare_weight(torch.cat(rows, dim=0).contiguous())
        self.w_o = ops.prepare_weight(value_heads(tensors[t["o_weight"]].t()).t().contiguous())
        # the second factor of the decays is applied in float32, inside the gates' kernel
        self.w_decay = tensors[t["decay_up"]].float().contiguous()
        self.b_decay = tensors[t["decay_bias"]].float().contiguous()
        self.b_rate = tensors[t["rate_bias"]].float().contiguous()
        self.norm_weight = value_heads(tensors[t["out_norm"]].float()).contiguous()

    def _min_chunk(self) -> int:
        rules = getattr(self.ops, "rules", None)
        return int(getattr(rules, "scan_min_chunk", 16))

    def state_spec(self):
        return {"s": ((self.num_heads, self.key_dim, self.value_dim), torch.float32)}

    def forward_into(self, h, out, ctx, entry):
        ops, rows, o = self.ops, h.shape[0], self.offsets
        proj = ctx.scratch("delta_rule.proj", (rows, self.in_size), torch.float32)
        project_normed(ops, h, self.w_in, proj, self.dtype, self.hidden_size)
        decay = ctx.scratch("delta_rule.decay", (rows, self.qk_size), torch.float32)
        unit = ctx.scratch("delta_rule.unit", (rows, self.qk_size), torch.float32)
        removal = ctx.scratch("delta_rule.removal", (rows, self.qk_size), torch.float32)
        ops.delta_gates(proj, o["decay_down"], self.decay_rank, o["rate_weight"], o["k_weight"], self.w_decay,
                        self.b_decay, self.b_rate, self.decay_scale, self.key_eps, self.num_heads, self.key_dim, decay,
                        unit, removal)
        outs = ctx.scratch("delta_rule.outputs", (rows, self.num_heads, 1, self.value_dim), torch.float32)
        state = entry.state["s"]
        # room for the chunks of a long portion: at most rows / (smallest chunk) + requests
        most = rows // max(1, self._min_chunk()) + ctx.max_reqs
        chunk_state = ctx.scratch("delta_rule.chunk_state", (most, self.num_heads, self.key_dim, self.value_dim),
                                  torch.float32)
        chunk_trans = ctx.scratch("delta_rule.chunk_trans", (most, self.num_heads, self.key_dim, self.key_dim),
                                  torch.float32)

        def scan():
            # (how many requests the step has and how long the longest portion is are read when the
            # launch is made, also when it is made again from a kept sequence of calls)
            pick = getattr(ops, "delta_scan_chunk", None)
            chunk = (pick(rows, ctx.max_q_len, self.num_heads, self.key_dim, self.value_dim) if pick is not None else 0)
            ops.delta_scan(proj, o["r_weight"], o["k_weight"], o["v_weight"], decay, unit, removal, self.num_heads,
                           self.key_dim, self.value_dim, state, ctx.all_q_start, ctx.all_req_rows, ctx.n_reqs, outs,
                           chunk, chunk_state if chunk else None, chunk_trans if chunk else None)
        live = getattr(ops, "live", None)
        if live is not None:
            live(scan)
        else:
            scan()
        mixed = ctx.scratch("delta_rule.out", (rows, self.v_size), self.dtype)
        if self.file_value_dim != self.value_dim:      # (the heads' unit norm is over the file's channels)
            ops.gla_output(outs, self.num_heads, self.key_dim, self.value_dim, self.norm_weight, self.norm_eps, proj,
                           o["gate_weight"], mixed, self.gate, self.file_value_dim)
        else:
            ops.gla_output(outs, self.num_heads, self.key_dim, self.value_dim, self.norm_weight, self.norm_eps, proj,
                           o["gate_weight"], mixed, self.gate)
        ops.linear_logits(mixed, self.w_o, out)

    def forward(self, h, residual, ctx, entry):
        y = ctx.scratch("delta_rule.sum", (1,) + tuple(residual.shape), torch.float32)
        self.forward_into(h, y[0], ctx, entry)
        self.ops.add_pending(residual, PendingSums(y, 1))

    def kernel_libraries(self):
        return [("linear_attention", None)]

    def weight_bytes(self):
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o, self.w_decay, self.b_decay, self.b_rate,
                                                          self.norm_weight) if w is not None)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "delta_rule_attention", DeltaRuleAttention)
