"""Arrangements of parts in a layer, the embedding and the output head."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import PartSpec
from ..weights.loader import TensorSpec, MATRIX, VECTOR, INIT_ZEROS
from .base import Block, Part, NormedInput
from .registry import register_part, build_part


class PreNormBlock(Block):
    """``x += mixer(norm1(x)); x += feed_forward(norm2(x))``; the sums are taken
    in float32 on the float32 residual stream.

    Arrangement: rust/engine/src/runner/model/qwen2/engine.rs:1065-1122 (layer
    loop), 1140-1147 and 1234-1241 (norm before each sublayer)."""

    def __init__(self, hidden_size: int, norm1: PartSpec, mixer: PartSpec, norm2: PartSpec = None,
                 feed_forward: PartSpec = None, tensors: Dict[str, str] = None):
        super().__init__(tensors)
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden_size = int(hidden_size)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer)
        # (a layer may be its mixer alone)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    def mixer_part(self):
        return self.mixer

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)

    def forward(self, residual, ctx, entry):
        h = NormedInput(self.norm1, residual, ctx, "block.normed", self.dtype)
        self.mixer.forward(h if self.mixer.takes_normed_input else h.tensor(), residual, ctx, entry)
        if self.feed_forward is None:
            return
        h = NormedInput(self.norm2, residual, ctx, "block.normed", self.dtype)
        self.feed_forward.forward(h if self.feed_forward.takes_normed_input else h.tensor(),
                                  residual, ctx)

    def weight_bytes(self):
        return sum(p.weight_bytes() for p in self.parts())


class SublayerNormBlock(Block):
    """``x += norm1(mixer(x)); x += norm2(feed_forward(x))``: the sublayers read the stream
    itself and each norm acts on its sublayer's OUTPUT, before the sum.  A block without a
    feed-forward has the first half only.  The stream and both sums are float32; the
    sublayers' products read the stream rounded to the compute dtype.

    A part that ``writes_output`` writes its float32 result into a scratch buffer
    (``forward_into``); any other part (made for blocks that add the sublayer's result
    straight into the stream) is handed a zeroed buffer in the stream's place."""

    def __init__(self, hidden_size: int, mixer: PartSpec, norm1: PartSpec, feed_forward: PartSpec = None,
                 norm2: PartSpec = None, tensors: Dict[str, str] = None):
        super().__init__(tensors)
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden_size = int(hidden_size)
        self.mixer = build_part("mixer", mixer)
        self.norm1 = build_part("norm", norm1)
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        for n in (self.norm1, self.norm2):
            if n is not None and not hasattr(n, "add_into"):
                raise ValueError(f"{type(n).__name__} cannot norm a sublayer's output into the stream (no add_into)")

    def parts(self):
        return [p for p in (self.mixer, self.norm1, self.feed_forward, self.norm2) if p is not None]

    def mixer_part(self):
        return self.mixer

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)

    def _fold(self, residual, ctx):
        pending = getattr(ctx, "pending", None)
        if pending is not None:          # (sums another kind of block left in pieces)
            self.ops.add_pending(residual, pending)
            ctx.pending = None

    NOTE = "sublayer_norm.copy"      # in the step's notes: the run whose last sum left the stream's copy behind

    def _input(self, residual, ctx, entry):
        """The stream as the sublayers' products read it: the stream itself in float32, else its
        rounded copy, which the run just before this one has left behind if it was of this kind."""
        if self.dtype == torch.float32:
            return residual
        h = ctx.scratch("block.stream_copy", tuple(residual.shape), self.dtype)
        memo = getattr(ctx, "memo", None)
        if memo is not None and memo.pop(self.NOTE, None) == entry.index - 1:
            return h
        self.ops.activation(residual, h, "cast")
        return h

    def _sublayer(self, part, h, residual, ctx, *entry):
        y = ctx.scratch("block.sublayer_out", tuple(residual.shape), torch.float32)
        if part.writes_output:
            part.forward_into(h, y, ctx, *entry)
        else:
            self.ops.activation(y, y, "zero")
            part.forward(h, y, ctx, *entry)
            self._fold(y, ctx)
        return y

    def forward(self, residual, ctx, entry):
        self._fold(residual, ctx)
        h = self._input(residual, ctx, entry)
        # every sum's new rows go to the next reader of the stream in the same pass
        copy = h if self.dtype != torch.float32 else None
        y = self._sublayer(self.mixer, h, residual, ctx, entry)
        self.norm1.add_into(y, residual, copy)
        if self.feed_forward is not None:
            y = self._sublayer(self.feed_forward, h, residual, ctx)
            self.norm2.add_into(y, residual, copy)
        memo = getattr(ctx, "memo", None)
        if memo is not None and copy is not None:
            memo[self.NOTE] = entry.index

    def weight_bytes(self):
        return sum(p.weight_bytes() for p in self.parts())


class SandwichNormBlock(Block):
    """A norm before AND behind each sublayer::

        x += scale1 * post_norm1(mixer(norm1(x)));  x += scale2 * post_norm2(feed_forward(norm2(x)))

    ``scale1`` / ``scale2`` (roles of the block's own tensors, or absent): a learned vector that
    multiplies the normed result element by element (a layer scale); it is folded into the
    post-norm's weight when the block is bound.  The post-norms are RMS norms (anything with
    ``rms_params()``); they act on the sublayer's float32 result, and norm, product and sum are
    float32.  A block without a feed-forward has the first half only."""

    def __init__(self, hidden_size: int, norm1: PartSpec, mixer: PartSpec, post_norm1: PartSpec,
                 norm2: PartSpec = None, feed_forward: PartSpec = None, post_norm2: PartSpec = None,
                 tensors: Dict[str, str] = None):
        super().__init__(tensors)
        if len({feed_forward is None, norm2 is None, post_norm2 is None}) != 1:
            raise ValueError("a feed-forward and its two norms come together")
        self.hidden_size = int(hidden_size)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer)
        self.post_norm1 = build_part("norm", post_norm1)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        self.post_norm2 = build_part("norm", post_norm2) if post_norm2 is not None else None
        self.post = [None, None]       # (weight with the layer scale folded in, eps) of each half
        self.next_weight, self.next_eps = None, 0.0      # the feed-forward's norm, if it is an RMS norm

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.post_norm1, self.norm2, self.feed_forward, self.post_norm2)
                if p is not None]

    def mixer_part(self):
        return self.mixer

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        for role in ("scale1", "scale2"):
            if role in self.tensor_names and (role == "scale1" or self.feed_forward is not None):
                specs[self.tensor_names[role]] = TensorSpec((self.hidden_size,), VECTOR)
        return specs

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)
        for i, norm in enumerate((self.post_norm1, self.post_norm2)):
            if norm is None:
                continue
            params = norm.rms_params() if hasattr(norm, "rms_params") else None
            if params is None:
                raise ValueError(f"{type(norm).__name__} is no RMS norm: the norm behind a sublayer is one")
            weight = params[0].float()
            role = f"scale{i + 1}"
            if role in self.tensor_names:
                weight = weight * tensors[self.tensor_names[role]].float()
            self.post[i] = (weight.contiguous(), float(params[1]))
        params = self.norm2.rms_params() if self.norm2 is not None and hasattr(self.norm2, "rms_params") else None
        if params is not None:
            self.next_weight, self.next_eps = params[0].float().contiguous(), float(params[1])

    def kernel_libraries(self):
        return [("stream_ops", None)] + super().kernel_libraries()

    def _fold(self, residual, ctx):
        pending = getattr(ctx, "pending", None)
        if pending is not None:
            self.ops.add_pending(residual, pending)
            ctx.pending = None

    def _half(self, i, h, part, residual, ctx, next_norm, *view):
        """One sublayer: ``h`` is its input (a tensor, or a ``NormedInput`` for a part that may fold
        the norm into its first product); ``next_norm``: the norm that reads the stream next, to run
        in the launch of the sum."""
        ops, rows = self.ops, residual.shape[0]
        if isinstance(h, NormedInput) and not part.takes_normed_input:
            h = h.tensor()
        y = ctx.scratch("block.sublayer_out", (rows, self.hidden_size), torch.float32)
        if part.writes_output:
            part.forward_into(h, y, ctx, *view)
        elif hasattr(part, "forward_pending"):
            pieces = part.forward_pending(h, y, ctx, *view)      # (a product left in pieces is summed by the norm)
            if pieces is not None:
                y = pieces
        else:
            ops.activation(y, y, "zero")
            part.forward(h, y, ctx, *view)
            self._fold(y, ctx)
        weight, eps = self.post[i]
        if next_norm is not None:
            ops.rmsnorm_add(y, weight, eps, residual, next_norm)
        else:
            ops.rmsnorm_add(y, weight, eps, residual)

    def forward(self, residual, ctx, entry):
        self._fold(residual, ctx)
        h = NormedInput(self.norm1, residual, ctx, "block.normed", self.dtype)
        if self.feed_forward is None:
            self._half(0, h, self.mixer, residual, ctx, None, entry)
            return
        # the feed-forward's norm runs in the launch that sums the mixer's result into the stream
        h2 = ctx.scratch("block.normed2", (residual.shape[0], self.hidden_size), self.dtype)
        self._half(0, h, self.mixer, residual, ctx, (self.next_weight, self.next_eps, h2) if self.next_weight is not None else None,
                   entry)
        if self.next_weight is None:
            self.norm2.forward(residual, h2)
        self._half(1, h2, self.feed_forward, residual, ctx, None)

    def weight_bytes(self):
        own = sum(w.numel() * w.element_size() for w, _ in (p for p in self.post if p is not None))
        return own + sum(p.weight_bytes() for p in self.parts())


class GatedConvBlock(Block):
    """A pre-norm layer whose sublayers read their input through a short causal convolution and
    whose results pass a gate before they are summed::

        h = norm1(x);  x += mixer(h + conv1(h)) * sigmoid(R1 h + b1)
        h = norm2(x);  x += feed_forward(h + conv2(h)) * sigmoid(R2 h + b2)

    ``conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j)`` channel by channel over the positions of
    one sequence (``w [width, taps]``, nothing before the sequence's start); the last ``taps - 1``
    inputs of each convolution are per-request state, so a sequence may be cut anywhere.  The gate
    reads the normed ``h`` itself, before the convolution (``R [width, width]``, ``b [width]``).
    ``conv_taps=0``: no convolution; ``residual_gate=False``: the plain sum.  The stream, the
    sigmoid and the sums are float32; the convolution runs on the normed activations in the
    compute dtype, which is also what its state keeps, so a cut changes no number.

    Tensor roles: ``conv1``, ``conv2``, ``gate1_weight``, ``gate1_bias``, ``gate2_weight``,
    ``gate2_bias``."""

    fuse_norm_conv = True      # (False: the norm and the convolution as launches of their own)

    def __init__(self, hidden_size: int, norm1: PartSpec, mixer: PartSpec, norm2: PartSpec = None,
                 feed_forward: PartSpec = None, conv_taps: int = 0, residual_gate: bool = True,
                 tensors: Dict[str, str] = None):
        super().__init__(tensors)
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        self.hidden_size, self.conv_taps, self.residual_gate = int(hidden_size), int(conv_taps), bool(residual_gate)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer)
        self.norm2 = build_part("norm", norm2) if norm2 is not None else None
        self.feed_forward = build_part("feed_forward", feed_forward) if feed_forward is not None else None
        self.w_conv = [None, None]
        self.w_gate = [None, None]
        self.b_gate = [None, None]

    def parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.feed_forward) if p is not None]

    def mixer_part(self):
        return self.mixer

    def _sublayers(self):
        return (1, 2) if self.feed_forward is not None else (1,)

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        t, w = self.tensor_names, self.hidden_size
        for i in self._sublayers():
            if self.conv_taps:
                specs[t[f"conv{i}"]] = TensorSpec((w, self.conv_taps), MATRIX)
            if self.residual_gate:
                specs[t[f"gate{i}_weight"]] = TensorSpec((w, w), MATRIX)
                specs[t[f"gate{i}_bias"]] = TensorSpec((w,), VECTOR, INIT_ZEROS)
        return specs

    def state_spec(self):
        """The mixer's state and, for each convolution, its last ``taps - 1`` inputs (compute dtype)."""
        spec = dict(self.mixer.state_spec())
        if self.conv_taps > 1:
            for i in self._sublayers():
                spec[f"conv{i}"] = ((self.conv_taps - 1, self.hidden_size), None)
        return spec

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        for p in self.parts():
            p.bind(tensors, ops, dtype)
        t = self.tensor_names
        ops.check_product_sizes(self.hidden_size, dtype, "residual gate (hidden size)")
        for i in self._sublayers():
            if self.conv_taps:      # (taps side by side for each channel, float32: four numbers a channel)
                self.w_conv[i - 1] = tensors[t[f"conv{i}"]].float().contiguous()
            if self.residual_gate:
                self.w_gate[i - 1] = ops.prepare_weight(tensors[t[f"gate{i}_weight"]].contiguous())
                self.b_gate[i - 1] = tensors[t[f"gate{i}_bias"]].float().contiguous()

    def kernel_libraries(self):
        return [("stream_ops", None)] + super().kernel_libraries()

    def _fold(self, residual, ctx):
        pending = getattr(ctx, "pending", None)
        if pending is not None:
            self.ops.add_pending(residual, pending)
            ctx.pending = None

    def _norm_conv_fits(self, norm) -> bool:
        """Norm and convolution in one launch: an RMS norm, and no more taps than that kernel has."""
        ops = self.ops
        return (self.fuse_norm_conv and hasattr(norm, "rms_params") and hasattr(ops, "norm_conv")
                and self.conv_taps <= getattr(ops, "NORM_CONV_MAX_TAPS", 0))

    def _half(self, i, norm, part, residual, ctx, entry, *view):
        ops, rows = self.ops, residual.shape[0]
        self._fold(residual, ctx)
        h = ctx.scratch("block.normed", (rows, self.hidden_size), self.dtype)
        hin = h
        fused = self.conv_taps and self._norm_conv_fits(norm)
        if not fused:
            norm.forward(residual, h)
        if self.conv_taps:
            hin = ctx.scratch("block.convolved", (rows, self.hidden_size), self.dtype)
            state = entry.state.get(f"conv{i}")
            if fused:
                # (whether every request brings one row is not a matter of the number of rows)
                weight, eps = norm.rms_params()
                launch = lambda: ops.norm_conv(residual, weight, eps, self.w_conv[i - 1], state, ctx.row_req,
                                               ctx.all_q_start, ctx.all_req_rows, h, hin, ctx.n_rows == ctx.n_reqs)
                live = getattr(ops, "live", None)
                if live is not None:
                    live(launch)
                else:
                    launch()
            else:
                ops.causal_conv(h, self.w_conv[i - 1], state, ctx.positions, ctx.row_req, ctx.all_q_start,
                                ctx.all_req_rows, hin)
        y = ctx.scratch("block.sublayer_out", (rows, self.hidden_size), torch.float32)
        if part.writes_output:
            part.forward_into(hin, y, ctx, *view)
        elif hasattr(part, "forward_pending") and hasattr(ops, "GATED_ADD_MAX_PIECES"):
            # (a product left in pieces is summed by the gated sum itself)
            pieces = part.forward_pending(hin, y, ctx, *view)
            if pieces is not None and pieces.splits <= ops.GATED_ADD_MAX_PIECES:
                y = pieces
            elif pieces is not None:
                ops.activation(y, y, "zero")
                ops.add_pending(y, pieces)
        else:
            ops.activation(y, y, "zero")
            part.forward(hin, y, ctx, *view)
            self._fold(y, ctx)
        gate = None
        if self.residual_gate:
            gate = ctx.scratch("block.gate", (rows, self.hidden_size), torch.float32)
            ops.linear_logits(h, self.w_gate[i - 1], gate)
        ops.gated_add(residual, y, gate, self.b_gate[i - 1])

    def forward(self, residual, ctx, entry):
        self._half(1, self.norm1, self.mixer, residual, ctx, entry, entry)
        if self.feed_forward is not None:
            self._half(2, self.norm2, self.feed_forward, residual, ctx, entry)

    def weight_bytes(self):
        own = sum(w.numel() * w.element_size() for w in self.w_conv + self.w_gate + self.b_gate if w is not None)
        return own + sum(p.weight_bytes() for p in self.parts())


class TokenEmbedding(Part):
    """``x[r] = table[id_r]`` into the float32 residual stream
    (rust/engine/src/runner/model/qwen2/kernels.rs:46-57)."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str]):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.table = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "embedding (hidden size)")
        # in the order the product kernels read, so that a tied output head shares it
        self.table = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)

    def forward(self, ids, out, ctx=None):
        """``ctx``: the step's batch description, for embeddings that need more than the
        ids (positions, say); this one does not."""
        self.ops.embed(self.table, ids, out)

    def weight_bytes(self):
        return 0     # a step reads one row per token, not the table


class PairHashEmbedding(Part):
    """``x[r] = norm(table[id_r] * scale + pairs[row_r])`` into the float32 stream: beside the token's
    own vector a row of a second table that the token and the one before it in its sequence pick
    together, ``row = (previous * mul_prev + id * mul_cur) mod buckets``; a sequence's first token
    takes the row behind the buckets (row number ``buckets``).  The token before a step's first
    one is per-request state (one integer), so a sequence may be cut anywhere.  ``norm``: a norm
    part applied to the sum in place (None: none); sum and norm in float32.

    Tensor roles: ``weight [vocab, hidden]``, ``pairs [buckets + 1, hidden]``."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str], scale: float = 1.0,
                 buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0, norm: PartSpec = None):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.scale, self.buckets, self.mul_prev, self.mul_cur = float(scale), int(buckets), int(mul_prev), int(mul_cur)
        self.norm = build_part("norm", norm) if norm is not None else None
        self.table = self.pairs = None
        self.state = {}

    def tensor_specs(self):
        specs = {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}
        if self.buckets:
            specs[self.tensor_names["pairs"]] = TensorSpec((self.buckets + 1, self.hidden_size), MATRIX)
        if self.norm is not None:
            specs.update(self.norm.tensor_specs())
        return specs

    def state_spec(self):
        return {"previous_token": ((1,), torch.int32)} if self.buckets else {}

    def attach_state(self, state):
        self.state = dict(state)

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        self.table = tensors[self.tensor_names["weight"]].contiguous()
        self.pairs = tensors[self.tensor_names["pairs"]].contiguous() if self.buckets else None
        if self.norm is not None:
            self.norm.bind(tensors, ops, dtype)
            if self.norm.rms_params() is None:
                raise ValueError(f"{type(self.norm).__name__} is no RMS norm: the embedding's kernel takes one")

    def forward(self, ids, out, ctx):
        weight, eps = self.norm.rms_params() if self.norm is not None else (None, 0.0)
        self.ops.embed_pairs(self.table, self.pairs, ids, ctx.positions, ctx.row_req, ctx.all_q_start,
                             ctx.all_req_rows, self.state.get("previous_token"), self.scale, self.buckets,
                             self.mul_prev, self.mul_cur, weight, eps, out)

    def kernel_libraries(self):
        return [("stream_ops", None)]

    def weight_bytes(self):
        return 0     # a step reads two rows per token, not the tables


class LinearHead(Part):
    """``logits = h W^T`` in float32; ``W`` is the embedding table when the
    names coincide (tied), as in rust/engine/src/runner/model/qwen2/engine.rs:299-303
    and 1312-1319.  ``softcap``: the logits are then bent into ``(-cap, cap)``,
    ``cap * tanh(logits / cap)``."""

    def __init__(self, vocab_size: int, hidden_size: int, tensors: Dict[str, str], softcap: float = None):
        super().__init__(tensors)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.softcap = None if softcap is None else float(softcap)     # logits <- cap * tanh(logits / cap)
        self.weight = None

    def tensor_specs(self):
        return {self.tensor_names["weight"]: TensorSpec((self.vocab_size, self.hidden_size), MATRIX)}

    def bind(self, tensors, ops, dtype):
        super().bind(tensors, ops, dtype)
        ops.check_product_sizes(self.hidden_size, dtype, "output head (hidden size)")
        self.weight = ops.prepare_weight(tensors[self.tensor_names["weight"]], shared=True)

    takes_normed_input = True

    def forward(self, h, out):
        fuse = (isinstance(h, NormedInput) and self.ops.can_fuse(out.shape[0], self.dtype, self.hidden_size, out.shape[1])
                and not self.ops.pieces_too_large_to_read_per_block(getattr(h.ctx, "pending", None)))
        rms = h.rms(accept_pending=True) if fuse else None
        if rms is not None:
            # the last reader of the stream: pieces still owed to it are added on the fly
            pending = getattr(h.ctx, "pending", None)
            self.ops.fused_norm_logits(rms[0], rms[1], rms[2], rms[3], self.weight, out, pending=pending)
            h.ctx.pending = None
        else:
            if isinstance(h, NormedInput):
                h = h.tensor()
            self.ops.linear_logits(h, self.weight, out)
        if self.softcap is not None:
            self.ops.softcap(out, self.softcap)

    def kernel_libraries(self):
        return [("stream_ops", None)] if self.softcap is not None else []

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()


register_part("block", "prenorm", PreNormBlock)
register_part("block", "gated_conv", GatedConvBlock)
register_part("embedding", "pair_hash_embedding", PairHashEmbedding)
register_part("block", "sublayer_norm", SublayerNormBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
