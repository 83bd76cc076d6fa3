"""Attention whose keys and values are read out of one small vector per token."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.loader import TensorSpec, MATRIX, VECTOR, INIT_NORM
from .attention import rows_by_kernel
from .base import Mixer, CacheSpec, PageTensor, NormedInput, PendingSums
from .registry import register_part

LATENT_PAD = 32       # the cached vector is laid out in multiples of this (zeros behind it)


class LatentAttention(Mixer):
    """Causal attention without positions over a latent cache.

    ``c_q = rmsnorm(W_dq h) * w_q`` (``q_rank`` wide), ``q = W_uq c_q`` (``heads x dim``);
    ``c = rmsnorm(W_dkv h) * w_c`` (``kv_rank`` wide) is all a token keeps.  Head ``a`` has keys
    ``k_a = U_a c`` (``U_a``: its ``dim`` rows of ``W_uk``) and values ``v_a = V_a c`` (its ``vdim``
    rows of ``W_uv``); the query at position i sees every ``j <= i``; scores ``q_a . k_a * scale``;
    ``sink=True``: the softmax's denominator holds ``exp(sink_a)`` as well, a learned number per
    head with no key and no value.  ``output_gate="sigmoid"``: head ``a``'s output is multiplied
    by ``sigmoid(W_g h)_a``.  Then ``W_o`` on the heads side by side.  Norms, scores, softmax and
    gate are float32.

    The keys and values are never made.  Since ``q_a . (U_a c_j) = (U_a^T q_a) . c_j`` and ``sum_j
    p_j V_a c_j = V_a (sum_j p_j c_j)``, every head asks the SAME cached vectors with its own
    query ``U_a^T q_a`` of ``kv_rank`` numbers and gets a weighted sum of them back, which ``V_a``
    then takes to the head's ``vdim`` outputs: attention of ``heads`` query heads over one
    key/value head whose keys are its values.  A step therefore reads ``kv_rank`` numbers per
    cached token whatever the number of heads, also for the tokens of a prompt's earlier
    portions.  The pages hold the vector twice, row by row for the scores and in quads of keys
    for the weighted sum (the two orders the attention kernels read).

    ``fold_query``: ``U_a^T q_a = (U_a^T W_uq,a) c_q``, so the two products that take the query's
    latent to the cached vector's coordinates can be ONE matrix ``[heads * latent, q_rank]``, made
    in float32 when the part is bound and rounded once.  It has ``latent / dim`` times the rows of
    ``W_uq`` and saves a launch and the head-sized queries' trip through memory; None: folded
    when the latent is at most ``FOLD_UP_TO`` times a head's size.

    Tensor roles: ``dq_weight, dq_norm, uq_weight, dkv_weight, dkv_norm, uk_weight, uv_weight,
    sink, gate_weight, o_weight``."""

    writes_output = True
    keeps_launches = True      # (what depends on the step beyond its rows is asked for at the launch)
    OUTPUT_GATES = (None, "sigmoid")
    FOLD_UP_TO = 2

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, q_rank: int, kv_rank: int,
                 scale: float, tensors: Dict[str, str], norm_eps: float = 1e-6, sink: bool = True,
                 output_gate: str = "sigmoid", fold_query: bool = None):
        super().__init__(tensors)
        if output_gate not in self.OUTPUT_GATES:
            raise ValueError(f"an output gate is one of {self.OUTPUT_GATES}, got {output_gate!r}")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.q_rank_laid = (self.q_rank + 7) // 8 * 8                   # inner sizes of products: multiples of 8
        self.value_laid = (self.value_dim + 7) // 8 * 8                 # (zero rows of V_a, zero columns of W_o behind a head)
        self.latent = (self.kv_rank + LATENT_PAD - 1) // LATENT_PAD * LATENT_PAD
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.has_sink, self.output_gate = bool(sink), output_gate
        self.fold_query = self.latent <= self.FOLD_UP_TO * self.head_dim if fold_query is None else bool(fold_query)
        self.w_in = self.w_uq = self.w_absorb = self.w_value = self.w_o = None
        self.q_norm = self.c_norm = self.sink = None

    @property
    def gates(self):
        return self.num_heads if self.output_gate else 0

    def tensor_specs(self):
        t, w, a = self.tensor_names, self.hidden_size, self.num_heads
        specs = {t["dq_weight"]: TensorSpec((self.q_rank, w), MATRIX),
                 t["dq_norm"]: TensorSpec((self.q_rank,), VECTOR, INIT_NORM),
                 t["uq_weight"]: TensorSpec((a * self.head_dim, self.q_rank), MATRIX),
                 t["dkv_weight"]: TensorSpec((self.kv_rank, w), MATRIX),
                 t["dkv_norm"]: TensorSpec((self.kv_rank,), VECTOR, INIT_NORM),
                 t["uk_weight"]: TensorSpec((a * self.head_dim, self.kv_rank), MATRIX),
                 t["uv_weight"]: TensorSpec((a * self.value_dim, self.kv_rank), MATRIX)}
        if self.has_sink:
            specs[t["sink"]] = TensorSpec((a,), VECTOR)
        if self.output_gate:
            specs[t["gate_weight"]] = TensorSpec((a, w), MATRIX)
        specs[t["o_weight"]] = TensorSpec((w, a * self.value_dim), MATRIX)
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_windowed_attention_sizes(self.num_heads, 1, self.latent, self.latent, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "attention projections (hidden size)")
        ops.check_product_sizes(self.num_heads * self.value_laid, dtype, "attention output projection (heads * value size)")
        t, a = self.tensor_names, self.num_heads

        def grown(x, rows=None, columns=None):
            rows, columns = rows or x.shape[0], columns or x.shape[1]
            if (rows, columns) == tuple(x.shape):
                return x
            out = torch.zeros((rows, columns), dtype=x.dtype, device=x.device)
            out[:x.shape[0], :x.shape[1]] = x
            return out
        # one product for the query's latent, the cached latent and the heads' gates; the latents'
        # rows are laid out with zeros behind them (their norms' weights too, so the zeros stay zeros)
        rows = [grown(tensors[t["dq_weight"]], rows=self.q_rank_laid), grown(tensors[t["dkv_weight"]], rows=self.latent)]
        if self.output_gate:
            rows.append(tensors[t["gate_weight"]])
        self.w_in = ops.prepare_weight(torch.cat(rows, dim=0).contiguous())
        uq = grown(tensors[t["uq_weight"]], columns=self.q_rank_laid)
        self.q_norm = grown(tensors[t["dq_norm"]].float().view(1, -1), columns=self.q_rank_laid).view(-1).contiguous()
        self.c_norm = grown(tensors[t["dkv_norm"]].float().view(1, -1), columns=self.latent).view(-1).contiguous()
        # head a's query in the latent's coordinates: U_a^T q_a, a product with U_a^T [latent, dim]
        uk = grown(tensors[t["uk_weight"]], columns=self.latent).view(a, self.head_dim, self.latent)
        if self.fold_query:
            folded = torch.bmm(uk.float().transpose(1, 2), uq.float().view(a, self.head_dim, self.q_rank_laid))
            self.w_uq = ops.prepare_weight(folded.reshape(a * self.latent, self.q_rank_laid).to(uq.dtype).contiguous())
            self.w_absorb = None
        else:
            self.w_uq = ops.prepare_weight(uq.contiguous())
            self.w_absorb = uk.transpose(1, 2).contiguous()                               # [heads, latent, dim]
        uv, wo = tensors[t["uv_weight"]], tensors[t["o_weight"]]
        self.w_value = torch.zeros((a, self.value_laid, self.latent), dtype=uv.dtype, device=uv.device)
        self.w_value[:, :self.value_dim, :self.kv_rank] = uv.view(a, self.value_dim, self.kv_rank)
        o_laid = torch.zeros((self.hidden_size, a, self.value_laid), dtype=wo.dtype, device=wo.device)
        o_laid[:, :, :self.value_dim] = wo.view(self.hidden_size, a, self.value_dim)
        self.w_o = ops.prepare_weight(o_laid.view(self.hidden_size, a * self.value_laid).contiguous())
        if self.has_sink:
            self.sink = tensors[t["sink"]].float().contiguous()

    def cache_spec(self):
        return CacheSpec((("k", PageTensor((1, self.latent), 1)), ("v", PageTensor((1, self.latent), 1))), None)

    def forward_into(self, h, out, ctx, entry):
        ops, rows, a = self.ops, h.shape[0], self.num_heads
        group = ctx.group(entry.group)
        proj = ctx.scratch("latent_attention.proj", (rows, self.q_rank_laid + self.latent + self.gates), torch.float32)
        ops.linear_logits(h, self.w_in, proj)
        cq = ctx.scratch("latent_attention.query_latent", (rows, self.q_rank_laid), self.dtype)
        gate = ctx.scratch("latent_attention.gate", (rows, a), torch.float32) if self.output_gate else None
        ops.latent_norm_write(proj, self.q_rank, self.q_rank_laid, self.kv_rank, self.latent, self.gates, self.q_norm,
                              self.c_norm, self.norm_eps, cq, gate, entry.k_cache, entry.v_cache, group.page_size,
                              ctx.positions, ctx.row_req, group.block_table)
        ql = ctx.scratch("latent_attention.q_in_latent", (rows, a * self.latent), self.dtype)
        if self.fold_query:
            ops.linear(cq, self.w_uq, ql)
        else:
            q = ctx.scratch("latent_attention.q", (rows, a * self.head_dim), self.dtype)
            ops.linear(cq, self.w_uq, q)
            ops.head_products(q, self.w_absorb, ql)
        mixed = ctx.scratch("latent_attention.mixed", (rows, a * self.latent), self.dtype)

        def attend():
            long_from, launches = rows_by_kernel(ops, ctx, self.dtype, self.latent, self.latent, group.page_size)
            ops.sink_window_attention(ql, a, 1, self.latent, self.latent, entry.k_cache, entry.v_cache,
                                      group.block_table, group.page_size, ctx.positions, ctx.row_req, None, 0,
                                      self.sink, self.scale, mixed, ctx.all_q_start, long_from, launches,
                                      ctx.max_ctx_len)
        live = getattr(ops, "live", None)
        if live is not None:
            live(attend)
        else:
            attend()
        heads = ctx.scratch("latent_attention.heads", (rows, a * self.value_laid), self.dtype)
        ops.head_products(mixed, self.w_value, heads, gate)       # (the heads' sigmoid gates ride on the product)
        ops.linear_logits(heads, self.w_o, out)

    def forward(self, h, residual, ctx, entry):
        if isinstance(h, NormedInput):
            h = h.tensor()
        y = ctx.scratch("latent_attention.sum", (1,) + tuple(residual.shape), torch.float32)
        self.forward_into(h, y[0], ctx, entry)
        self.ops.add_pending(residual, PendingSums(y, 1))

    def kernel_libraries(self):
        return [("windowed_attention", None)]

    def weight_bytes(self):
        total = 0
        for w in (self.w_in, self.w_uq, self.w_absorb, self.w_value, self.w_o, self.q_norm, self.c_norm, self.sink):
            if w is not None:
                total += w.numel() * w.element_size()
        return total


register_part("mixer", "latent_attention", LatentAttention)
