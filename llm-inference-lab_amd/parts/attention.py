"""Attention mixers."""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..config.spec import PartSpec
from ..weights.loader import TensorSpec, MATRIX, VECTOR, INIT_NORM
from .base import Mixer, KVCacheSpec, CacheSpec, PageTensor, NormedInput, PendingSums, project_normed
from .registry import register_part, build_part


class GQAAttention(Mixer):
    """Grouped-query attention over a paged cache.

    ``q = h Wq^T + bq`` (and k, v alike; float32 accumulate, bias added in
    float32), position encoding on q and k, keys and values of the new
    positions written to the cache before the scores are taken, so a step's
    tokens see themselves and each other causally; head ``h`` reads kv head
    ``h // (num_heads / num_kv_heads)``; scores ``q.k * scale`` over the keys
    ``max(0, p - window + 1) .. p`` of the query at position ``p``, softmax and
    the weighted sum of values in float32; then ``residual += attn Wo^T``.

    Formulas: projections rust/engine/src/runner/model/qwen2/engine.rs:1133-1210,
    cache write engine.rs:1072-1082, scores/softmax
    rust/engine/src/runner/model/qwen2/kernels.rs:702-853, output projection and
    residual engine.rs:1225-1233.  The window is not in the reference (it
    rejects ``use_sliding_window``, engine.rs:262).

    ``values_from_keys``: the layer has no value projection; its values are its keys as
    projected (bias added), before the position encoding turns them.  ``output_gate="sigmoid"``:
    one more projection of the layer's input, a single number per head (``gate_weight [heads,
    hidden]``, no bias); head ``h``'s output is multiplied by ``sigmoid`` of its number before the
    output projection.

    The kernels take heads whose size is a multiple of 16: a head of another size is laid out
    with zeros behind its channels (zero rows of the projections, zero columns of the output
    projection), which changes no score and no output."""

    takes_normed_input = True
    OUTPUT_GATES = (None, "sigmoid")

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PartSpec], tensors: Dict[str, str], qkv_bias: bool = True,
                 out_bias: bool = False, window: Optional[int] = None,
                 scale: Optional[float] = None, values_from_keys: bool = False,
                 output_gate: Optional[str] = None):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if output_gate not in self.OUTPUT_GATES:
            raise ValueError(f"an output gate is one of {self.OUTPUT_GATES}, got {output_gate!r}")
        self.values_from_keys = bool(values_from_keys)
        self.output_gate = output_gate
        self.w_gate = None
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.file_head_dim = int(head_dim)                       # a head as the model file has it
        self.head_dim = (self.file_head_dim + 15) // 16 * 16     # and as the kernels see it
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.file_head_dim)
        padded = dict(padded_dim=self.head_dim) if self.head_dim != self.file_head_dim else {}
        self.position = build_part("position", position, **padded) if position is not None else None
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None

    # sizes
    @property
    def q_size(self):
        return self.num_heads * self.head_dim

    @property
    def kv_size(self):
        return self.num_kv_heads * self.head_dim

    def tensor_specs(self):
        t, h = self.tensor_names, self.hidden_size
        q_size, kv_size = self.num_heads * self.file_head_dim, self.num_kv_heads * self.file_head_dim
        # (the random-weights mode draws a tensor by its place in this list: the order stays)
        specs = {t["q_weight"]: TensorSpec((q_size, h), MATRIX), t["k_weight"]: TensorSpec((kv_size, h), MATRIX)}
        if not self.values_from_keys:
            specs[t["v_weight"]] = TensorSpec((kv_size, h), MATRIX)
        specs[t["o_weight"]] = TensorSpec((h, q_size), MATRIX)
        if self.output_gate:
            specs[t["gate_weight"]] = TensorSpec((self.num_heads, h), MATRIX)
        if self.qkv_bias:
            specs[t["q_bias"]] = TensorSpec((q_size,), VECTOR)
            specs[t["k_bias"]] = TensorSpec((kv_size,), VECTOR)
            if not self.values_from_keys:
                specs[t["v_bias"]] = TensorSpec((kv_size,), VECTOR)
        if self.out_bias:
            specs[t["o_bias"]] = TensorSpec((h,), VECTOR)
        if self.position is not None:
            specs.update(self.position.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "attention projections (hidden size)")
        ops.check_product_sizes(self.q_size, dtype, "attention output projection (heads * head size)")
        t = self.tensor_names
        # The order in which the position encoding wants the channels of the query and key heads
        # (scores do not depend on it; values and the output projection keep the file's order).
        order = self.position.channel_order() if self.position is not None else None
        d, dk = self.file_head_dim, self.head_dim
        plain = list(range(d)) + [-1] * (dk - d)          # the file's order, zeros behind

        def heads_in_order(x, heads, order=order):
            """Rows (or entries) of ``heads`` heads of ``d`` channels -> heads of ``dk`` places."""
            order = plain if order is None else order
            if order == list(range(d)):
                return x
            per_head = x.unflatten(0, (heads, d))
            per_head = torch.cat([per_head, torch.zeros_like(per_head[:, :1])], dim=1)     # place -1: a zero
            index = torch.tensor([d if c < 0 else c for c in order], device=x.device)
            return per_head.index_select(1, index).flatten(0, 1)
        # Values that are the keys before they turn: the key rows once more, in the file's order,
        # in the value rows' place, so that the product and its epilogues stay as they are.
        value = "k" if self.values_from_keys else "v"
        # One projection instead of three: the rows of Wq, Wk, Wv stacked.
        self.w_qkv = ops.prepare_weight(torch.cat([heads_in_order(tensors[t["q_weight"]], self.num_heads),
                                                   heads_in_order(tensors[t["k_weight"]], self.num_kv_heads),
                                                   heads_in_order(tensors[t[value + "_weight"]], self.num_kv_heads,
                                                                  None)], dim=0).contiguous())
        if self.qkv_bias:
            parts = [heads_in_order(tensors[t["q_bias"]], self.num_heads),
                     heads_in_order(tensors[t["k_bias"]], self.num_kv_heads),
                     heads_in_order(tensors[t[value + "_bias"]], self.num_kv_heads, None)]
            kept = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
            self.b_qkv = torch.cat([p.to(kept) for p in parts]).contiguous()
        if self.output_gate:
            self.w_gate = ops.prepare_weight(tensors[t["gate_weight"]].contiguous())
        # (the heads' outputs arrive in the values' order: the columns of the output projection
        # are its own, with zero columns behind every head)
        self.w_o = ops.prepare_weight(heads_in_order(tensors[t["o_weight"]].t(), self.num_heads, None).t().contiguous())
        self.b_o = tensors[t["o_bias"]].contiguous() if self.out_bias else None
        if self.position is not None:
            self.position.bind(tensors, ops, dtype)

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, h, residual, ctx, entry):
        ops = self.ops
        rows = h.shape[0]
        table = self.position.rotary_table() if self.position is not None else None
        group = ctx.group(entry.group)
        k_cache = entry.k_cache if entry.writes_cache else None
        v_cache = entry.v_cache if entry.writes_cache else None
        fuse = (isinstance(h, NormedInput) and ops.can_fuse(rows, self.dtype, self.hidden_size, self.q_size + 2 * self.kv_size)
                and (self.position is None or table is not None)
                and not ops.pieces_too_large_to_read_per_block(getattr(ctx, "pending", None)))
        rms = h.rms(accept_pending=True) if fuse else None
        pending = None
        gate = ctx.scratch("attention.gate", (rows, self.num_heads), torch.float32) if self.output_gate else None
        if rms is not None:
            # few rows: norm, the three projections, bias, rotation and the cache
            # write are one kernel
            q = ctx.scratch("attention.q", (rows, self.q_size), self.dtype)
            # pieces still owed to the stream are added as its rows are read, and folded
            # in by the output projection below
            pending = getattr(ctx, "pending", None)
            ops.fused_norm_qkv(rms[0], rms[2], rms[3], self.w_qkv, self.b_qkv, self.num_heads,
                               self.num_kv_heads, self.head_dim, table, ctx.positions, ctx.row_req,
                               group.block_table, group.page_size, k_cache, v_cache, q, pending=pending)
            if gate is not None:           # (the gate reads the same normed rows: norm and product in one kernel too)
                ops.fused_norm_logits(rms[0], None, rms[2], rms[3], self.w_gate, gate, pending=pending)
        elif (ops.can_fuse_qkv_rope(rows, self.dtype, self.head_dim, self.q_size + 2 * self.kv_size,
                                    self.hidden_size)
              and (self.position is None or table is not None)):
            # more rows: the norm on its own, then one kernel for the rest
            if isinstance(h, NormedInput):
                h = h.tensor()
            q = ctx.scratch("attention.q", (rows, self.q_size), self.dtype)
            ops.qkv_rope_cache(h, self.w_qkv, self.b_qkv, self.num_heads, self.num_kv_heads,
                               self.head_dim, table, ctx.positions, ctx.row_req, group.block_table,
                               group.page_size, k_cache, v_cache, q)
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            q = ctx.scratch("attention.qkv", (rows, self.q_size + 2 * self.kv_size), self.dtype)
            ops.linear(h, self.w_qkv, q, self.b_qkv)
            if self.position is not None and table is None:
                qv = q[:, :self.q_size].unflatten(1, (self.num_heads, self.head_dim))
                kv = q[:, self.q_size:self.q_size + self.kv_size].unflatten(
                    1, (self.num_kv_heads, self.head_dim))
                self.position.apply(qv, kv, ctx.positions[:rows])
            ops.rope_kv_write(q, self.num_heads, self.num_kv_heads, self.head_dim, table,
                              ctx.positions, ctx.row_req, group.block_table, group.page_size,
                              k_cache, v_cache)
        if gate is not None and rms is None:
            ops.linear_logits(h, self.w_gate, gate)
        out = ctx.scratch("attention.out", (rows, self.q_size), self.dtype)

        prepare = getattr(ops, "prepare_attention", None)
        prepared = []

        def attend():
            # (how many requests, how long their portions and their histories are: read from
            # the step's description when the launch is made, also when it is made again
            # from a kept sequence of calls; what stays the same then is checked once)
            if prepare is None:
                ops.paged_attention(
                    q, self.num_heads, self.num_kv_heads, self.head_dim,
                    entry.k_cache, entry.v_cache, group.block_table, group.page_size,
                    ctx.q_start, ctx.start_pos, ctx.n_reqs, ctx.max_q_len, ctx.max_ctx_len,
                    self.window, self.scale, out, self._short_requests(ctx))
                return
            if not prepared:
                prepared.append(prepare(
                    q, self.num_heads, self.num_kv_heads, self.head_dim, entry.k_cache, entry.v_cache,
                    group.block_table, group.page_size, getattr(ctx, "all_q_start", ctx.q_start),
                    getattr(ctx, "all_start_pos", ctx.start_pos), self.window, self.scale, out, ctx.row_req))
            prepared[0].launch(ctx.n_reqs, ctx.max_q_len, ctx.max_ctx_len, self._short_requests(ctx))
        live = getattr(ops, "live", None)
        if live is not None:
            live(attend)
        else:
            attend()
        if gate is not None:
            ops.gate_heads(out, gate, self.num_heads, self.head_dim, self.output_gate)
        if pending is not None:
            ops.linear_residual(out, self.w_o, residual, self.b_o, pending=pending)
            ctx.pending = None
            return
        splits = 1
        if getattr(ctx, "pending", 0) is None and ops.pieces_by_tiles(rows, self.hidden_size, self.q_size):
            splits = ops.split_count(rows, self.dtype, self.hidden_size, self.q_size)
        if splits > 1:
            # some rows of a large matrix: cut along the inner size, the pieces left for the
            # norm that reads the stream next
            parts = ctx.scratch("attention.pieces", (splits, rows, self.hidden_size), torch.float32)
            ctx.pending = ops.linear_partials(out, self.w_o, parts, splits, self.b_o)
        else:
            ops.linear_residual(out, self.w_o, residual, self.b_o)

    def _short_requests(self, ctx):
        """Which of the step's requests bring only a few tokens (the kernels serve those by
        another launch than the portions of prompts); worked out once per step, kept in
        the step's notes for the other layers."""
        limit = self.ops.attention_short_limit(self.num_heads, self.num_kv_heads, self.dtype, ctx.max_q_len)
        if limit <= 0:
            return None
        key = ("attention.short", limit)
        if key not in ctx.memo:
            count = longest = 0
            for b in range(ctx.n_reqs):
                n = ctx.host_q_start[b + 1] - ctx.host_q_start[b]
                if n <= limit:
                    count += 1
                    longest = max(longest, ctx.host_start_pos[b] + n)
            ctx.memo[key] = (ctx.row_req, limit, count, longest) if 0 < count < ctx.n_reqs else None
        return ctx.memo[key]

    @property
    def keeps_launches(self):
        return self.position is None or self.position.keeps_launches

    def kernel_libraries(self):
        return [("attention", self.head_dim)]

    def weight_bytes(self):
        total = 0
        for w in (self.w_qkv, self.b_qkv, self.w_o, self.b_o, self.w_gate):
            if w is not None:
                total += w.numel() * w.element_size()
        return total


def rows_by_kernel(ops, ctx, dtype, key_dim, value_dim, page_size):
    """``(long_from, launches)`` of this step for the attention kernels with run-time sizes: requests
    of at least ``long_from`` rows go to the matrix-core kernel; worked out once per step, kept in
    the step's notes for the other layers."""
    pick = getattr(ops, "windowed_attention_long_rows", None)
    long_from = pick(dtype, key_dim, value_dim, page_size) if pick is not None else 0
    if not long_from:
        return 0, 1
    key = ("windowed_attention.split", long_from)
    if key not in ctx.memo:
        starts = ctx.host_q_start
        counts = [starts[b + 1] - starts[b] for b in range(ctx.n_reqs)]
        ctx.memo[key] = ((1 if any(n < long_from for n in counts) else 0)
                         | (2 if any(n >= long_from for n in counts) else 0))
    return long_from, ctx.memo[key]


class WindowedSinkAttention(Mixer):
    """Grouped-query attention through a sliding window that keeps a sequence's first
    positions in sight, with a learned extra term in the softmax's denominator.

    ``q = Wq h`` (``heads x key_dim``), ``k = Wk h`` (``kv_heads x key_dim``), ``v = Wv h``
    (``kv_heads x value_dim``), no biases.  ``qk_norm="whole"``: q, and k alike, is divided by
    the root mean square over its WHOLE width (all heads at once, ``eps`` inside the root)
    and multiplied by a weight of that width, in float32, before it is cut into heads.  The
    query at position i attends to the keys ``i - window < j <= i`` and, beside them, to the
    keys ``j < min(keep_first, i + 1)``
    (``window`` None: every ``j <= i``).  Scores ``q.k * scale``; weights ``exp(s_j - m) /
    (sum_j exp(s_j - m) + exp(sink_h - m))`` where ``sink_h`` is one learned number per head
    (``sink=False``: the plain softmax): the extra term only enlarges the denominator, nothing is
    summed for it.  Head ``h``
    reads kv head ``h // (heads / kv_heads)``.  No position encoding enters the scores.

    ``own_kv=False``: the layer has no key and value projections; its run reads the pages
    of the run that the schedule names as its cache (keys as that run stored them, after
    its norm), with its own queries, window and sink.

    ``position``: a position encoding with a ``pair_table()`` (``rope_pairs``) turns queries and keys
    before the scores are taken; the keys are cached turned.  ``qkv_bias``: the three projections have
    biases (roles ``q_bias``, ``k_bias``, ``v_bias``), added to the float32 sums.
    ``weights="sigmoid"``: no softmax; a visible key weighs ``sigmoid(score + b_h)`` with ``b_h`` one
    learned number per head (role ``score_bias``; ``score_bias=False``: none), and the weights are not
    normalised over the keys.  ``output_gate="sigmoid"``: one more projection of the layer's input, a
    single number per head (role ``gate_weight [heads, hidden]``); head ``h``'s output is multiplied
    by ``sigmoid`` of its number before the output projection.  ``value_mix``: ``"first"`` the layer
    leaves the values of the step's tokens, unrounded, for later layers; ``"mix"`` its values become
    ``(1 - lambda) v + lambda v_first`` with ``v_first`` what the ``"first"`` layer left for the same
    token and ``lambda`` one learned number (role ``value_mix``); the mixed values are what is cached.

    Pages: keys ``[kv_heads, P, key_dim]``, values ``[kv_heads, P, value_dim]``.  The products'
    inner sizes are multiples of 8: a value head of another width is laid out with zeros behind
    its channels (zero rows of the value projection, zero columns of the output projection), which
    changes no output."""

    writes_output = True
    takes_normed_input = True      # (few rows: the norm in front of the mixer runs inside its first product)
    WEIGHTS = ("softmax", "sigmoid")
    VALUE_MIX = (None, "first", "mix")

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                 scale: float, tensors: Dict[str, str], window: Optional[int] = None, keep_first: int = 0,
                 sink: bool = True, qk_norm: Optional[str] = "whole", norm_eps: float = 1e-6,
                 own_kv: bool = True, position: Optional[PartSpec] = None, qkv_bias: bool = False,
                 weights: str = "softmax", score_bias: bool = False, output_gate: Optional[str] = None,
                 value_mix: Optional[str] = None):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if qk_norm not in (None, "whole"):
            raise ValueError(f"qk_norm is None or 'whole', got {qk_norm!r}")
        if weights not in self.WEIGHTS or value_mix not in self.VALUE_MIX or output_gate not in (None, "sigmoid"):
            raise ValueError(f"weights is one of {self.WEIGHTS}, value_mix of {self.VALUE_MIX}, output_gate None or "
                             f"'sigmoid'; got {weights!r}, {value_mix!r}, {output_gate!r}")
        self.weights, self.value_mix, self.output_gate = weights, value_mix, output_gate
        self.qkv_bias, self.has_score_bias = bool(qkv_bias), bool(score_bias)
        self.position = build_part("position", position) if position is not None else None
        # the projections that turn, carry biases, mix values or gate heads go through one kernel
        # of their own, which knows no norm over the whole projection and writes keys and values
        self.rotates = bool(self.position is not None or qkv_bias or value_mix or output_gate)
        if self.rotates and (qk_norm or not own_kv):
            raise ValueError("a position encoding, biases, mixed values or an output gate go with keys and values "
                             "of the layer's own and without a norm over the whole projection")
        if self.position is not None and not hasattr(self.position, "pair_table"):
            raise ValueError(f"{type(self.position).__name__} has no pair_table(): this mixer turns neighbouring channels")
        if weights == "sigmoid" and sink:
            raise ValueError("a sink belongs to a softmax's denominator; sigmoid weights have none")
        if score_bias and weights != "sigmoid":
            raise ValueError("score_bias goes with sigmoid weights")
        self.w_gate_rows = 0
        self.b_in = self.score_bias = None
        self.mix_weight = 0.0
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim = int(key_dim)
        self.file_value_dim = int(value_dim)                       # a value head as the model file has it
        self.value_dim = (self.file_value_dim + 7) // 8 * 8        # and as the kernels and the pages see it
        self.scale = float(scale)
        self.window = None if window is None else int(window)
        self.keep_first = int(keep_first or 0)
        self.has_sink, self.qk_norm, self.norm_eps, self.own_kv = bool(sink), qk_norm, float(norm_eps), bool(own_kv)
        self.w_in = self.w_o = self.q_norm = self.k_norm = self.sink = None

    @property
    def q_size(self):
        return self.num_heads * self.key_dim

    @property
    def k_size(self):
        return self.num_kv_heads * self.key_dim

    @property
    def v_size(self):
        return self.num_kv_heads * self.value_dim

    @property
    def in_size(self):
        return (self.q_size + (self.k_size + self.v_size if self.own_kv else 0)
                + (self.num_heads if self.output_gate else 0))

    def tensor_specs(self):
        t, w = self.tensor_names, self.hidden_size
        file_v = self.num_kv_heads * self.file_value_dim
        specs = {t["q_weight"]: TensorSpec((self.q_size, w), MATRIX),
                 t["o_weight"]: TensorSpec((w, self.num_heads * self.file_value_dim), MATRIX)}
        if self.own_kv:
            specs[t["k_weight"]] = TensorSpec((self.k_size, w), MATRIX)
            specs[t["v_weight"]] = TensorSpec((file_v, w), MATRIX)
        if self.qkv_bias:
            specs[t["q_bias"]] = TensorSpec((self.q_size,), VECTOR)
            specs[t["k_bias"]] = TensorSpec((self.k_size,), VECTOR)
            specs[t["v_bias"]] = TensorSpec((file_v,), VECTOR)
        if self.has_score_bias:
            specs[t["score_bias"]] = TensorSpec((self.num_heads,), VECTOR)
        if self.output_gate:
            specs[t["gate_weight"]] = TensorSpec((self.num_heads, w), MATRIX)
        if self.value_mix and "value_mix" in t:       # (every mixing layer of a model file may carry the number)
            specs[t["value_mix"]] = TensorSpec((), VECTOR)
        if self.position is not None:
            specs.update(self.position.tensor_specs())
        if self.qk_norm:
            specs[t["q_norm"]] = TensorSpec((self.q_size,), VECTOR, INIT_NORM)
            if self.own_kv:
                specs[t["k_norm"]] = TensorSpec((self.k_size,), VECTOR, INIT_NORM)
        if self.has_sink:
            specs[t["sink"]] = TensorSpec((self.num_heads,), VECTOR)
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_windowed_attention_sizes(self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "attention projections (hidden size)")
        ops.check_product_sizes(self.num_heads * self.value_dim, dtype, "attention output projection (heads * value size)")
        t = self.tensor_names
        e, ek = self.file_value_dim, self.value_dim

        def value_heads(x, heads):
            """Rows (or entries) of ``heads`` value heads of ``e`` channels -> of ``ek``, zeros behind."""
            if e == ek:
                return x
            per_head = x.unflatten(0, (heads, e))
            zeros = torch.zeros((heads, ek - e) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
            return torch.cat([per_head, zeros], dim=1).flatten(0, 1)
        rows = [tensors[t["q_weight"]]]
        if self.own_kv:
            rows += [tensors[t["k_weight"]], value_heads(tensors[t["v_weight"]], self.num_kv_heads)]
        if self.output_gate:
            rows.append(tensors[t["gate_weight"]])
        self.w_in = ops.prepare_weight(torch.cat(rows, dim=0).contiguous())       # one product for q (, k, v, gates)
        if self.qkv_bias:
            bias = [tensors[t["q_bias"]].float(), tensors[t["k_bias"]].float(),
                    value_heads(tensors[t["v_bias"]].float(), self.num_kv_heads)]
            if self.output_gate:
                bias.append(torch.zeros(self.num_heads, dtype=torch.float32, device=bias[0].device))
            self.b_in = torch.cat(bias).contiguous()
        if self.has_score_bias:
            self.score_bias = tensors[t["score_bias"]].float().contiguous()
        if self.value_mix == "mix":
            self.mix_weight = float(tensors[t["value_mix"]].float().reshape(-1)[0])
        if self.position is not None:
            self.position.bind(tensors, ops, dtype)
        self.w_o = ops.prepare_weight(value_heads(tensors[t["o_weight"]].t(), self.num_heads).t().contiguous())
        if self.qk_norm:
            self.q_norm = tensors[t["q_norm"]].float().contiguous()
            self.k_norm = tensors[t["k_norm"]].float().contiguous() if self.own_kv else None
        if self.has_sink:
            self.sink = tensors[t["sink"]].float().contiguous()

    def cache_spec(self):
        return CacheSpec((("k", PageTensor((self.num_kv_heads, self.key_dim), 1)),
                          ("v", PageTensor((self.num_kv_heads, self.value_dim), 1))),
                         self.window, self.keep_first if self.window is not None else 0)

    def forward_into(self, h, out, ctx, entry):
        ops, rows = self.ops, h.shape[0]
        if self.own_kv != bool(entry.writes_cache):
            raise ValueError("an attention layer without keys and values of its own reads another run's cache, "
                             "and one that has them writes its own")
        group = ctx.group(entry.group)
        proj = ctx.scratch("windowed_attention.proj", (rows, self.in_size), torch.float32)
        project_normed(ops, h, self.w_in, proj, self.dtype, self.hidden_size)
        q = ctx.scratch("windowed_attention.q", (rows, self.q_size), self.dtype)
        gate = None
        if self.rotates:
            freq, rot_dims, magnitude = self.position.pair_table() if self.position is not None else (None, 0, 1.0)
            if self.output_gate:
                gate = ctx.scratch("windowed_attention.gate", (rows, self.num_heads), torch.float32)
            # (every layer that mixes finds the first such layer's values of the step's rows here)
            first = (ctx.scratch("windowed_attention.first_values", (rows, self.v_size), torch.float32)
                     if self.value_mix else None)
            ops.project_rotate_write(proj, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, self.b_in,
                                     freq, rot_dims, magnitude, self.value_mix, self.mix_weight, first, gate, q,
                                     entry.k_cache, entry.v_cache, group.page_size, ctx.positions, ctx.row_req,
                                     group.block_table)
        else:
            ops.project_norm_write(proj, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, self.own_kv,
                                   self.q_norm, self.k_norm, self.norm_eps, q, entry.k_cache, entry.v_cache,
                                   group.page_size, ctx.positions, ctx.row_req, group.block_table)
        mixed = ctx.scratch("windowed_attention.out", (rows, self.num_heads * self.value_dim), self.dtype)
        sigmoid = self.weights == "sigmoid"
        kind = dict(weights="sigmoid") if sigmoid else {}

        def attend():
            # (which requests bring many rows is read from the step's description when the launch
            # is made, also when it is made again from a kept sequence of calls)
            long_from, launches = self._split(ctx, group.page_size)
            ops.sink_window_attention(q, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim,
                                      entry.k_cache, entry.v_cache, group.block_table, group.page_size,
                                      ctx.positions, ctx.row_req, self.window, self.keep_first,
                                      self.score_bias if sigmoid else self.sink,
                                      self.scale, mixed, ctx.all_q_start, long_from, launches,
                                      ctx.max_ctx_len if self.window is None
                                      else min(ctx.max_ctx_len, self.window + self.keep_first), **kind)
        live = getattr(ops, "live", None)
        if live is not None:
            live(attend)
        else:
            attend()
        if gate is not None:
            ops.gate_heads(mixed, gate, self.num_heads, self.value_dim, self.output_gate)
        ops.linear_logits(mixed, self.w_o, out)

    def forward(self, h, residual, ctx, entry):
        y = ctx.scratch("windowed_attention.sum", (1,) + tuple(residual.shape), torch.float32)
        self.forward_into(h, y[0], ctx, entry)
        self.ops.add_pending(residual, PendingSums(y, 1))

    def _split(self, ctx, page_size):
        return rows_by_kernel(self.ops, ctx, self.dtype, self.key_dim, self.value_dim, page_size)

    keeps_launches = True      # (what depends on the step beyond its rows is asked for at the launch)

    def kernel_libraries(self):
        return [("windowed_attention", None)]

    def weight_bytes(self):
        total = 0
        for w in (self.w_in, self.w_o, self.q_norm, self.k_norm, self.sink, self.b_in, self.score_bias):
            if w is not None:
                total += w.numel() * w.element_size()
        return total


register_part("mixer", "gqa_attention", GQAAttention)
register_part("mixer", "windowed_sink_attention", WindowedSinkAttention)
