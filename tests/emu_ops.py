"""Plain PyTorch references of the kernel set, op by op, on the engine's own
buffers and layouts (paged cache, block tables, interleaved gate/up rows).

Two uses: the GPU tests compare each HIP kernel with the function of the same
name here, and the CPU tests plug this object into the engine in place of the
HIP kernels to exercise the cache manager, the step function and the scheduler
without a GPU.  It is test code, not a fallback: the product never loads it.
All arithmetic is float32 whatever the storage dtype.
"""
from __future__ import annotations

import math

import torch

from llm_inference_lab_amd.cache import layout as cache_layout
from llm_inference_lab_amd.parts import PendingSums


class EmuRecord:
    """The calls a part made while it was recorded (the counterpart of the product's
    ``LaunchRecord``): ``(bound method, (args, kwargs), None)`` or ``(None, closure, None)``."""

    def __init__(self, dry=False):
        self.calls = []
        self.dry = dry

    @staticmethod
    def _same(a, b):
        if isinstance(a, torch.Tensor) or isinstance(b, torch.Tensor):
            return (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor) and a.data_ptr() == b.data_ptr()
                    and a.shape == b.shape and a.stride() == b.stride() and a.dtype == b.dtype)
        if isinstance(a, PendingSums) or isinstance(b, PendingSums):
            return (isinstance(a, PendingSums) and isinstance(b, PendingSums) and a.splits == b.splits
                    and EmuRecord._same(a.parts, b.parts))
        return a == b

    def same_as(self, other):
        if len(self.calls) != len(other.calls):
            return False
        for (fa, aa, _), (fb, ab, _) in zip(self.calls, other.calls):
            if (fa is None) != (fb is None):
                return False
            if fa is None:
                continue
            if fa is not fb or len(aa[0]) != len(ab[0]) or sorted(aa[1]) != sorted(ab[1]):
                return False
            if not all(self._same(x, y) for x, y in zip(aa[0], ab[0])):
                return False
            if not all(self._same(aa[1][k], ab[1][k]) for k in aa[1]):
                return False
        return True


class EmuOps:
    # the operations that do work on tensors: written down while a part is recorded, as the
    # product's kernel set writes down its calls into the kernel libraries
    RECORDED = ("embed", "gather_tokens", "rmsnorm", "linear", "linear_relu2", "linear_residual", "linear_partials",
                "add_pending", "linear_logits", "linear_swiglu", "fused_norm_qkv", "qkv_rope_cache",
                "fused_norm_swiglu", "fused_norm_logits", "rope_inplace", "rope_kv_write",
                "paged_attention", "argmax", "sample", "layernorm", "layernorm_add", "activation",
                "project_norm_write", "sink_window_attention", "gla_decay", "gla_scan", "gla_output",
                "gate_heads", "add_row_vector", "moe_select", "moe_add_chosen", "embed_pairs", "causal_conv", "norm_conv",
                "gated_add", "latent_norm_write", "head_products", "softcap", "project_rotate_write", "delta_gates",
                "delta_scan", "rmsnorm_add", "scaled_sum")

    def __init__(self, device="cpu", fuse=True):
        self.device = torch.device(device)
        self.calls = {}
        self.fuse = fuse
        import types
        self.rules = types.SimpleNamespace(min_steps_per_split=8, scan_min_chunk=16, scan_max_chunk=64)
        self._record = None
        self._depth = 0
        for name in self.RECORDED:
            setattr(self, name, self._recordable(getattr(self, name)))

    # ----------------------------------------------- recorded sequences of calls
    def _recordable(self, method):
        def call(*args, **kwargs):
            record = self._record
            if record is not None and self._depth == 0:      # (an operation's own inner calls are its business)
                record.calls.append((call, (args, kwargs), None))
                if record.dry:      # (nothing is computed; what the caller is handed back all the same)
                    return PendingSums(args[2], args[3]) if method.__name__ == "linear_partials" else None
            self._depth += 1
            try:
                return method(*args, **kwargs)
            finally:
                self._depth -= 1
        call.inner = method
        return call

    def begin_recording(self, dry=False):
        assert self._record is None
        self._record = EmuRecord(dry)
        return self._record

    def end_recording(self):
        record, self._record = self._record, None
        return record

    def live(self, launch):
        record = self._record
        if record is None:
            launch()
            return
        record.calls.append((None, launch, None))
        if record.dry:
            return
        self._record = None
        try:
            launch()
        finally:
            self._record = record

    def replay(self, record):
        for fn, args, _ in record.calls:
            if fn is None:
                args()
            else:
                fn.inner(*args[0], **args[1])

    def fingerprint(self):
        plain = (int, float, str, bool, type(None))
        rules = tuple(sorted((k, v if isinstance(v, plain) else id(v)) for k, v in vars(self.rules).items()))
        return (self.fuse, rules, getattr(self, "num_cus", 0))

    def _count(self, name):
        self.calls[name] = self.calls.get(name, 0) + 1

    @property
    def calls_made(self):
        """Calls so far, as the kernel set of the product counts them."""
        return sum(self.calls.values())

    def check_attention_sizes(self, num_heads, num_kv_heads, head_dim, dtype):
        pass

    def check_product_sizes(self, inner, dtype, what):
        pass

    def synchronize(self):
        pass

    # ------------------------------------------------------------ elementwise
    def embed(self, table, ids, out):
        self._count("embed")
        out.copy_(table[ids.long()].float())

    def gather_tokens(self, dst, dst_index, src, src_index, n):
        self._count("gather_tokens")
        for i in range(n):
            dst[int(dst_index[i])] = src[int(src_index[i])]

    def rmsnorm(self, x, weight, eps, out, rows=None, pending=None):
        self._count("rmsnorm")
        if pending is not None:
            assert rows is None and pending.parts.shape[1:] == x.shape
            x += pending.parts[:pending.splits].float().sum(0)
        v = x.float() if rows is None else x.float()[rows.long()]
        inv = torch.rsqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        out.copy_((v * inv * weight.float()).to(out.dtype))

    # ----------------------------------------------------------------- linear
    def linear(self, x, w, out, bias=None):
        self._count("linear")
        y = x.float() @ w.float().t()
        if bias is not None:
            y = y + bias.float()
        out.copy_(y.to(out.dtype))

    def linear_relu2(self, x, w, out):
        self._count("linear_relu2")
        out.copy_((torch.relu(x.float() @ w.float().t()) ** 2).to(out.dtype))

    def linear_residual(self, x, w, resid, bias=None, pending=None):
        self._count("linear_residual")
        y = x.float() @ w.float().t()
        if bias is not None:
            y = y + bias.float()
        if pending is not None:
            resid.add_(self._owed(pending))
        resid.add_(y)

    # ---------------------------------------------------- sums left in pieces
    MAX_SPLITS = 8
    num_cus = 256

    @staticmethod
    def _owed(pending):
        return pending.parts[:pending.splits].sum(0) if pending is not None else 0.0

    def split_count(self, rows, dtype, n, k):
        if not self.fuse or dtype != torch.bfloat16 or not 0 < rows <= 64:
            return 1
        strips, steps = (n + 15) // 16, (k + 31) // 32
        return max(1, min(self.num_cus // max(strips, 1), steps // self.rules.min_steps_per_split, self.MAX_SPLITS))

    def linear_partials(self, x, w, parts, splits, bias=None):
        """Piece s covers the K steps from s * ceil(steps / splits) on; a step is 32 wide
        for up to 64 rows and 64 wide for more (the two kernels' K tiles)."""
        self._count("linear_partials")
        k = x.shape[1]
        width = 32 if x.shape[0] <= 64 else 64
        steps = (k + width - 1) // width
        per = (steps + splits - 1) // splits
        for s in range(splits):
            lo, hi = min(k, s * per * width), min(k, (s + 1) * per * width)
            parts[s] = x[:, lo:hi].float() @ w[:, lo:hi].float().t()
        if bias is not None:
            parts[0] += bias.float()
        return PendingSums(parts, splits)

    def add_pending(self, x, pending):
        self._count("add_pending")
        x.add_(self._owed(pending))

    def linear_logits(self, x, w, out):
        self._count("linear_logits")
        out.copy_(x.float() @ w.float().t())

    def linear_swiglu(self, x, w_gu, out, activation="silu"):
        """w_gu rows alternate in runs of 16: gate rows of 16 outputs, then the
        up rows of the same outputs."""
        self._count("linear_swiglu")
        inter = out.shape[1]
        y = x.float() @ w_gu.float().t()                       # [M, 2*Ipad]
        y = y.view(x.shape[0], -1, 2, 16)
        gate = y[:, :, 0, :].reshape(x.shape[0], -1)[:, :inter]
        up = y[:, :, 1, :].reshape(x.shape[0], -1)[:, :inter]
        if activation == "gelu_tanh":
            act = 0.5 * gate * (1.0 + torch.tanh(0.7978845608028654 * (gate + 0.044715 * gate ** 3)))
        else:
            act = gate / (1.0 + torch.exp(-gate))
        out.copy_((act * up).to(out.dtype))

    # ------------------------------------------- layer norm, plain activations
    @staticmethod
    def _layernorm(v, weight, eps):
        mean = v.mean(-1, keepdim=True)
        var = ((v - mean) ** 2).mean(-1, keepdim=True)
        return (v - mean) / torch.sqrt(var + eps) * weight.float()

    def layernorm(self, x, weight, eps, out, rows=None):
        self._count("layernorm")
        v = x.float() if rows is None else x.float()[rows.long()]
        out.copy_(self._layernorm(v, weight, eps).to(out.dtype))

    def layernorm_add(self, y, weight, eps, resid, copy=None):
        self._count("layernorm_add")
        resid.add_(self._layernorm(y.float(), weight, eps))
        if copy is not None:
            copy.copy_(resid.to(copy.dtype))

    def activation(self, x, out, kind):
        self._count("activation")
        v = x.float()
        v = {"cast": v, "relu2": torch.relu(v) ** 2, "zero": torch.zeros_like(v)}[kind]
        out.copy_(v.to(out.dtype))

    # --------------------------------- mixers with run-time sizes
    def check_windowed_attention_sizes(self, num_heads, num_kv_heads, key_dim, value_dim, dtype):
        pass

    def check_linear_attention_sizes(self, num_heads, key_dim, value_dim):
        pass

    def project_norm_write(self, proj, num_heads, num_kv_heads, key_dim, value_dim, own_kv, q_norm, k_norm, eps,
                           q_out, k_cache, v_cache, page_size, positions, row_req, block_table):
        self._count("project_norm_write")
        rows = q_out.shape[0]
        qs, ks, vs = num_heads * key_dim, num_kv_heads * key_dim, num_kv_heads * value_dim

        def whole(v, w):
            return v if w is None else v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w.float()
        p = proj.float()
        q_out.copy_(whole(p[:, :qs], q_norm).to(q_out.dtype))
        if not own_kv:
            return
        k = whole(p[:, qs:qs + ks], k_norm).to(k_cache.dtype).view(rows, num_kv_heads, key_dim)
        v = p[:, qs + ks:qs + ks + vs].to(v_cache.dtype).view(rows, num_kv_heads, value_dim)
        for r in range(rows):
            pos = int(positions[r])
            page = int(block_table[int(row_req[r]), pos // page_size])
            o = pos % page_size
            k_cache[page, :, o] = k[r]
            cache_layout.value_quads(v_cache[page])[:, o >> 2, :, o & 3] = v[r]

    def sink_window_attention(self, q, num_heads, num_kv_heads, key_dim, value_dim, k_cache, v_cache, block_table,
                              page_size, positions, row_req, window, keep_first, sink, scale, out,
                              q_start=None, long_from=0, launches=3, max_keys=0, weights="softmax"):
        """(``long_from``, ``launches``: how the kernels share the rows; the result is the same.)"""
        self._count("sink_window_attention")
        rows = q.shape[0]
        qf = q.float().view(rows, num_heads, key_dim)
        group = num_heads // num_kv_heads
        for r in range(rows):
            i, b = int(positions[r]), int(row_req[r])
            lo = max(0, i - window + 1) if window else 0
            js = list(range(min(int(keep_first or 0), lo))) + list(range(lo, i + 1))
            pages = torch.tensor([int(block_table[b, j // page_size]) for j in js])
            offs = torch.tensor([j % page_size for j in js])
            k = k_cache[pages, :, offs].float()          # [keys, G, D]
            v = cache_layout.value_quads(v_cache)[pages, :, offs >> 2, :, offs & 3].float()
            for h in range(num_heads):
                s = (k[:, h // group] @ qf[r, h]) * scale
                if weights == "sigmoid":
                    w = torch.sigmoid(s + (sink[h].float() if sink is not None else 0.0))
                    if out.dtype != torch.float32:      # (the matrix cores take the weights rounded)
                        w = w.to(out.dtype).float()
                    out[r, h * value_dim:(h + 1) * value_dim] = (w @ v[:, h // group]).to(out.dtype)
                    continue
                if sink is not None:
                    s = torch.cat([s, sink[h].float().view(1)])
                w = torch.softmax(s, 0)[:len(js)]
                out[r, h * value_dim:(h + 1) * value_dim] = (w @ v[:, h // group]).to(out.dtype)

    def project_rotate_write(self, proj, num_heads, num_kv_heads, key_dim, value_dim, bias, freq, rot_dims, magnitude,
                             mix, mix_weight, v_first, gate_out, q_out, k_cache, v_cache, page_size, positions,
                             row_req, block_table):
        self._count("project_rotate_write")
        rows = q_out.shape[0]
        qs, ks, vs = num_heads * key_dim, num_kv_heads * key_dim, num_kv_heads * value_dim
        p = proj.float()[:, :qs + ks + vs + (0 if gate_out is None else gate_out.shape[1])]
        if bias is not None:
            p = p + bias.float()
        pos = positions[:rows].float()

        def turned(x, heads):
            x = x.reshape(rows, heads, key_dim).clone()
            if rot_dims:
                ang = pos.unsqueeze(-1) * freq.float()                       # float32 angles
                cos, sin = (torch.cos(ang) * magnitude).unsqueeze(1), (torch.sin(ang) * magnitude).unsqueeze(1)
                u, v = x[..., 0:rot_dims:2].clone(), x[..., 1:rot_dims:2].clone()
                x[..., 0:rot_dims:2] = u * cos - v * sin
                x[..., 1:rot_dims:2] = v * cos + u * sin
            return x
        q_out.copy_(turned(p[:, :qs], num_heads).reshape(rows, qs).to(q_out.dtype))
        k = turned(p[:, qs:qs + ks], num_kv_heads).to(k_cache.dtype)
        v = p[:, qs + ks:qs + ks + vs]
        if mix == "first":
            v_first.copy_(v)
        elif mix == "mix":
            v = (1.0 - mix_weight) * v + mix_weight * v_first
        v = v.to(v_cache.dtype).view(rows, num_kv_heads, value_dim)
        if gate_out is not None:
            gate_out.copy_(p[:, qs + ks + vs:])
        for r in range(rows):
            at = int(positions[r])
            page = int(block_table[int(row_req[r]), at // page_size])
            o = at % page_size
            k_cache[page, :, o] = k[r]
            cache_layout.value_quads(v_cache[page])[:, o >> 2, :, o & 3] = v[r]

    def check_delta_rule_sizes(self, num_heads, key_dim, value_dim):
        pass

    def delta_gates(self, proj, off_low, rank, off_rate, off_k, w2, w0, rate_bias, decay_scale, key_eps, num_heads,
                    key_dim, decay, unit, removal):
        self._count("delta_gates")
        channels = num_heads * key_dim
        z = torch.tanh(proj[:, off_low:off_low + rank].float()) @ w2.float().t()
        if w0 is not None:
            z = z + w0.float()
        decay.copy_(torch.exp(-decay_scale * torch.sigmoid(z)))
        za = proj[:, off_rate:off_rate + channels].float()
        if rate_bias is not None:
            za = za + rate_bias.float()
        k = proj[:, off_k:off_k + channels].float().view(-1, num_heads, key_dim)
        u = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + key_eps)).reshape(-1, channels)
        unit.copy_(u)
        removal.copy_(torch.sigmoid(za) * u)

    def delta_scan_chunk(self, rows, longest, num_heads, key_dim, value_dim):
        return 16 if longest >= 32 else 0

    def delta_scan(self, proj, off_r, off_k, off_v, decay, unit, removal, num_heads, key_dim, value_dim, state, q_start,
                   req_rows, n_reqs, out, chunk=0, chunk_state=None, chunk_trans=None):
        """(``chunk``: how the kernel spreads the work; the recurrence is the same.)"""
        self._count("delta_scan")
        if chunk:
            assert chunk_state.shape[0] >= proj.shape[0] // chunk + n_reqs and chunk_trans.shape[0] == chunk_state.shape[0]
        H, D, E = num_heads, key_dim, value_dim
        o = out.view(-1, H, E)
        for b in range(n_reqs):
            st = state[int(req_rows[b])]
            for t in range(int(q_start[b]), int(q_start[b + 1])):
                r = proj[t, off_r:off_r + H * D].view(H, D)
                k = proj[t, off_k:off_k + H * D].view(H, D)
                v = proj[t, off_v:off_v + H * E].view(H, E)
                dot = torch.einsum("hd,hde->he", unit[t].view(H, D), st)
                new = (decay[t].view(H, D, 1) * st - removal[t].view(H, D, 1) * dot.unsqueeze(-2)
                       + k.unsqueeze(-1) * v.unsqueeze(-2))
                st.copy_(new)
                o[t] = torch.einsum("hde,hd->he", st, r)

    def rmsnorm_add(self, y, weight, eps, x, next_norm=None):
        self._count("rmsnorm_add")
        v = self._owed(y) if isinstance(y, PendingSums) else y.float()
        x.add_(v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight.float())
        if next_norm is not None:
            w, e, out = next_norm
            out.copy_((x / torch.sqrt((x * x).mean(-1, keepdim=True) + e) * w.float()).to(out.dtype))

    def scaled_sum(self, out, y1, a, y2, b):
        self._count("scaled_sum")
        out.copy_(a * y1 + b * y2)

    SCAN_SLICE = 16

    def gla_slices(self, key_dim):
        return (key_dim + self.SCAN_SLICE - 1) // self.SCAN_SLICE

    def gla_decay(self, low, rank, w2, bias, tau, decay):
        self._count("gla_decay")
        z = low[:, :rank].float() @ w2.float().t()
        if bias is not None:
            z = z + bias.float()
        decay.copy_(torch.exp(torch.nn.functional.logsigmoid(z) / tau))

    def gla_scan_chunk(self, rows, longest, num_heads, value_dim):
        return 16 if longest >= 32 else 0

    def gla_scan(self, proj, off_q, off_k, off_v, decay, q_scale, num_heads, key_dim, value_dim, state, q_start,
                 req_rows, n_reqs, parts, chunk=0, chunk_state=None, chunk_decay=None):
        """(``chunk``: how the kernel spreads the work; the recurrence is the same.)"""
        self._count("gla_scan")
        if chunk:
            assert chunk_state.shape[0] >= proj.shape[0] // chunk + n_reqs and chunk_decay.shape[0] == chunk_state.shape[0]
        H, D, E, S = num_heads, key_dim, value_dim, self.SCAN_SLICE
        for b in range(n_reqs):
            slot = int(req_rows[b])
            st = state[slot]
            for t in range(int(q_start[b]), int(q_start[b + 1])):
                q = proj[t, off_q:off_q + H * D].view(H, D) * q_scale
                k = proj[t, off_k:off_k + H * D].view(H, D)
                v = proj[t, off_v:off_v + H * E].view(H, E)
                st.mul_(decay[t].view(H, D, 1)).add_(k.unsqueeze(-1) * v.unsqueeze(-2))
                o = st * q.unsqueeze(-1)                        # [H, D, E]
                for s in range(parts.shape[2]):
                    parts[t, :, s] = o[:, s * S:(s + 1) * S].sum(1)

    def gla_output(self, parts, num_heads, key_dim, value_dim, weight, eps, proj, off_gate, out, gate="silu",
                   norm_count=0):
        self._count("gla_output")
        o = parts.sum(2)                                        # [rows, H, E]
        w = weight.float().view(num_heads, value_dim) if weight.numel() == num_heads * value_dim else weight.float()
        y = o / torch.sqrt((o * o).sum(-1, keepdim=True) / (norm_count or value_dim) + eps) * w
        g = proj[:, off_gate:off_gate + num_heads * value_dim].float().view(-1, num_heads, value_dim)
        out.copy_((y * (g if gate == "silu" else 1.0) * torch.sigmoid(g)).reshape(out.shape).to(out.dtype))

    # ------------------------------------------------- fused few-row kernels
    FUSED_MAX_ROWS = 64
    fuse_max_rows = 16

    def pieces_too_large_to_read_per_block(self, pending):
        return False

    def pieces_by_tiles(self, rows, n, k):
        return False

    def can_fuse(self, rows, dtype, inner, outer=None):
        return self.fuse and dtype == torch.bfloat16 and 0 < rows <= self.fuse_max_rows

    def prepare_weight(self, w, shared=False):
        return w

    def release_shared(self):
        pass

    # --------------------------------------------- gates, offsets, routed experts
    def gate_heads(self, out, gate, num_heads, head_dim, kind="sigmoid"):
        """``out[r, h, :] *= sigmoid(gate[r, h])``, the product in float32, one rounding."""
        self._count("gate_heads")
        assert kind == "sigmoid"
        v = out.float().view(out.shape[0], num_heads, head_dim) * torch.sigmoid(gate.float())[:, :, None]
        out.copy_(v.view(out.shape).to(out.dtype))

    def add_row_vector(self, x, table, row):
        self._count("add_row_vector")
        x += table[row].float()

    def prepare_stacked(self, w, members):
        return w.view(members, w.shape[0] // members, w.shape[1])

    def stacked_member(self, stacked, e):
        return stacked[e]

    def moe_grouped(self, dtype):
        return False

    def moe_select(self, logits, correction, groups, groups_keep, scale, chosen, weights, scoring="softmax"):
        """Per row: softmax (or, ``scoring="sigmoid"``, the sigmoid) of the logits, the choice value
        (score + correction), the kept groups by their best choice value, the ``top`` best of their
        members; ties to the smaller index."""
        self._count("moe_select")
        rows, outputs = logits.shape
        top = chosen.shape[1]
        z = logits.float()
        e = torch.exp(z - z.max(-1, keepdim=True).values)
        s = e / e.sum(-1, keepdim=True) if scoring == "softmax" else torch.sigmoid(z)
        c = s + correction.float()
        per = outputs // groups
        best = c.view(rows, groups, per).max(-1).values
        allowed = torch.zeros(rows, groups, dtype=torch.bool)
        left = best.clone()
        for _ in range(groups_keep):
            g = torch.argmax(left, dim=-1)            # (the first of equal ones)
            allowed[torch.arange(rows), g] = True
            left[torch.arange(rows), g] = -float("inf")
        c = torch.where(allowed[:, :, None].expand(rows, groups, per).reshape(rows, outputs), c,
                        torch.full_like(c, -float("inf")))
        for k in range(top):
            e_k = torch.argmax(c, dim=-1)
            chosen[:, k] = e_k.to(torch.int32)
            weights[:, k] = s[torch.arange(rows), e_k] * scale
            c[torch.arange(rows), e_k] = -float("inf")

    # ------------------------------- hashed pairs, short convolution, gates, latent attention
    def embed_pairs(self, table, pairs, ids, positions, row_req, q_start, req_rows, previous, scale, buckets,
                    mul_prev, mul_cur, norm_weight, eps, out):
        """``out[r] = norm(table[id_r] * scale + pairs[row_r])``; the token before a request's first
        row of the step comes from ``previous[slot]``, which then takes the request's last token."""
        self._count("embed_pairs")
        rows = out.shape[0]
        x = table[ids[:rows].long()].float() * scale
        if buckets:
            last = {}
            for r in range(rows):
                b = int(row_req[r])
                slot = int(req_rows[b])
                if int(positions[r]) == 0:
                    at = buckets
                else:
                    before = int(ids[r - 1]) if r > int(q_start[b]) else int(previous[slot, 0])
                    at = (before * mul_prev + int(ids[r]) * mul_cur) % buckets
                x[r] += pairs[at].float()
                last[slot] = int(ids[r])
            for slot, token in last.items():
                previous[slot, 0] = token
        if norm_weight is not None:
            x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * norm_weight.float()
        out.copy_(x)

    def causal_conv(self, h, weight, state, positions, row_req, q_start, req_rows, out):
        """``out_t = h_t + sum_j weight[:, j] h_(t - taps + 1 + j)`` over the positions of each request;
        inputs from before the step come from ``state [slots, taps - 1, width]`` (the latest last),
        which then takes the request's latest inputs."""
        self._count("causal_conv")
        rows, taps = h.shape[0], weight.shape[1]
        w = weight.float()
        hf = h.float()
        res = hf.clone()
        starts = {}
        for r in range(rows):
            b = int(row_req[r])
            first = int(q_start[b])
            starts.setdefault(b, first)
            slot = int(req_rows[b])
            for j in range(taps):
                back = taps - 1 - j                 # how many positions behind row r
                if back == 0:
                    src = hf[r]
                elif r - back >= first:
                    src = hf[r - back]
                elif state is not None:              # (zeros stand there before the sequence's start)
                    src = state[slot, taps - 1 - (back - (r - first))].float()
                else:
                    continue
                res[r] += w[:, j] * src
        out.copy_(res.to(out.dtype))
        if state is None or taps <= 1:
            return
        for b, first in starts.items():
            n = sum(1 for r in range(rows) if int(row_req[r]) == b)
            slot = int(req_rows[b])
            joined = torch.cat([state[slot].float(), hf[first:first + n]], dim=0)
            state[slot] = joined[-(taps - 1):].to(state.dtype)

    NORM_CONV_MAX_TAPS = 8
    GATED_ADD_MAX_PIECES = 8

    def norm_conv(self, x, norm_weight, eps, weight, state, row_req, q_start, req_rows, h, out, one_row_each):
        """The RMS norm of the stream's rows into ``h`` and ``causal_conv`` over them into ``out``."""
        self._count("norm_conv")
        if one_row_each and x.shape[0] != len({int(b) for b in row_req[:x.shape[0]]}):
            raise ValueError("norm_conv: one_row_each, but a request brings several rows")
        xf = x.float()
        h.copy_((xf / torch.sqrt((xf * xf).mean(-1, keepdim=True) + eps) * norm_weight.float()).to(h.dtype))
        self.causal_conv(h, weight, state, None, row_req, q_start, req_rows, out)
        self.calls["causal_conv"] -= 1              # (one launch, counted above)

    def gated_add(self, x, y, gate, bias):
        """``x += y * sigmoid(gate + bias)``: ``gate [rows, width]`` or one number a row ``[rows, 1]``
        (None: ``x += y``), all float32."""
        self._count("gated_add")
        if isinstance(y, PendingSums):
            y = y.parts[:y.splits].float().sum(0)
        if gate is None:
            x += y
            return
        g = gate.float() + (bias.float() if bias is not None else 0.0)
        x += y * torch.sigmoid(g)

    def latent_norm_write(self, proj, q_rank, q_laid, kv_rank, latent, gates, q_norm, c_norm, eps, cq_out, gate_out,
                          k_cache, v_cache, page_size, positions, row_req, block_table):
        """From ``proj [rows, q_laid + latent + gates]`` float32: the query's latent (RMS norm over its
        first ``q_rank`` numbers, weight ``q_norm``) into ``cq_out``; the cached latent (RMS norm over
        ``kv_rank`` numbers, weight ``c_norm``) into the row's place of both page tensors; the heads'
        gates as they are into ``gate_out``."""
        self._count("latent_norm_write")
        rows = cq_out.shape[0]
        p = proj.float()

        def normed(v, n, w):
            return v / torch.sqrt((v[:, :n] ** 2).sum(-1, keepdim=True) / n + eps) * w.float()
        cq_out.copy_(normed(p[:, :q_laid], q_rank, q_norm).to(cq_out.dtype))
        c = normed(p[:, q_laid:q_laid + latent], kv_rank, c_norm).to(k_cache.dtype)
        if gates:
            gate_out.copy_(p[:, q_laid + latent:q_laid + latent + gates])
        for r in range(rows):
            pos = int(positions[r])
            page = int(block_table[int(row_req[r]), pos // page_size])
            o = pos % page_size
            k_cache[page, 0, o] = c[r]
            cache_layout.value_quads(v_cache[page])[0, o >> 2, :, o & 3] = c[r]

    def head_products(self, x, w, out, gate=None):
        """``out[r, a, :] = w[a] x[r, a, :]`` for a stack ``w [heads, n, k]``; sums in float32; with
        ``gate [rows, heads]``, head ``a`` of row ``r`` times ``sigmoid(gate[r, a])``."""
        self._count("head_products")
        heads, n, k = w.shape
        rows = x.shape[0]
        res = torch.einsum("rak,ank->ran", x.float().view(rows, heads, k), w.float())
        if gate is not None:
            res = res * torch.sigmoid(gate.float()).view(rows, heads, 1)
        out.copy_(res.reshape(rows, heads * n).to(out.dtype))

    def softcap(self, x, cap):
        self._count("softcap")
        x.copy_(cap * torch.tanh(x / cap))

    def moe_add_chosen(self, resid, src, chosen, weights, first, last):
        """``resid[r] += sum over k with first <= chosen[r, k] < last of weights[r, k] * src[r]``."""
        self._count("moe_add_chosen")
        hit = (chosen >= first) & (chosen < last)
        w = (weights * hit).sum(-1, keepdim=True)
        resid += w * src.float()

    def _normed(self, x, rows_index, norm_w, eps, n, pending=None):
        v = x.float() + self._owed(pending)
        v = v if rows_index is None else v[rows_index[:n].long()]
        inv = torch.rsqrt((v * v).sum(-1, keepdim=True) / v.shape[-1] + eps)
        # the kernel rounds x * w to bfloat16 and scales by inv_rms afterwards
        return (v * norm_w.float()).to(torch.bfloat16).float() * inv

    def fused_norm_qkv(self, x, norm_w, eps, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq,
                       positions, row_req, block_table, page_size, k_cache, v_cache, q_out, pending=None):
        self._count("fused_norm_qkv")
        rows = x.shape[0]
        y = self._normed(x, None, norm_w, eps, rows, pending) @ w_qkv.float().t()
        if b_qkv is not None:
            y = y + b_qkv.float()
        qkv = y.clone()                      # float32: the kernel rotates before it rounds
        self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                           block_table, page_size, k_cache, v_cache)
        q_out.copy_(qkv[:, :num_heads * head_dim].to(q_out.dtype))

    def can_fuse_qkv_rope(self, rows, dtype, head_dim, n=None, k=None):
        return self.fuse and dtype == torch.bfloat16 and rows > 0 and head_dim % 16 == 0 and (
            rows <= 64 or (n is not None and 64 % head_dim == 0))

    def qkv_rope_cache(self, h, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions,
                       row_req, block_table, page_size, k_cache, v_cache, q_out):
        self._count("qkv_rope_cache")
        y = h.float() @ w_qkv.float().t()
        if b_qkv is not None:
            y = y + b_qkv.float()
        qkv = y.clone()                      # float32: the kernel rotates before it rounds
        self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                           block_table, page_size, k_cache, v_cache)
        q_out.copy_(qkv[:, :num_heads * head_dim].to(q_out.dtype))

    def fused_norm_swiglu(self, x, norm_w, eps, w_gate_up, out, pending=None, activation="silu"):
        self._count("fused_norm_swiglu")
        h = self._normed(x, None, norm_w, eps, x.shape[0], pending)
        self.linear_swiglu(h, w_gate_up, out, activation)

    def fused_norm_logits(self, x, rows_index, norm_w, eps, w, out, pending=None):
        self._count("fused_norm_logits")
        out.copy_(self._normed(x, rows_index, norm_w, eps, out.shape[0], pending) @ w.float().t())

    # ------------------------------------------------------------------- rope
    @staticmethod
    def _rotate(x, positions, inv_freq):
        # x [rows, heads, d] float32
        half = x.shape[-1] // 2
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        lo, hi = x[..., :half], x[..., half:]
        return torch.cat([lo * c - hi * s, hi * c + lo * s], dim=-1)

    def rope_inplace(self, x, positions, inv_freq):
        self._count("rope_inplace")
        x.copy_(self._rotate(x.float(), positions, inv_freq).to(x.dtype))

    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                      block_table, page_size, k_cache, v_cache):
        self._count("rope_kv_write")
        rows = qkv.shape[0]
        qs, ks = num_heads * head_dim, num_kv_heads * head_dim
        q = qkv[:, :qs].float().view(rows, num_heads, head_dim)
        k = qkv[:, qs:qs + ks].float().view(rows, num_kv_heads, head_dim)
        v = qkv[:, qs + ks:].float().view(rows, num_kv_heads, head_dim)
        if inv_freq is not None:
            q = self._rotate(q, positions[:rows], inv_freq)
            k = self._rotate(k, positions[:rows], inv_freq)
            qkv[:, :qs] = q.reshape(rows, qs).to(qkv.dtype)
        if k_cache is None:
            return
        for r in range(rows):
            p = int(positions[r])
            page = int(block_table[int(row_req[r]), p // page_size])
            assert page >= 0, "write to a position without a page"
            off = p % page_size
            # the numbers of a page lie in the kernels' fragment order
            kflat = k_cache.view(k_cache.shape[0], num_kv_heads, -1)
            vflat = v_cache.view(v_cache.shape[0], num_kv_heads, -1)
            kflat[page][:, cache_layout.key_index(page_size, head_dim)[off]] = k[r].to(k_cache.dtype)
            vflat[page][:, cache_layout.value_index(page_size, head_dim)[:, off]] = v[r].to(v_cache.dtype)

    # -------------------------------------------------------------- attention
    def attention_short_limit(self, num_heads, num_kv_heads, dtype, max_q_len):
        return 0

    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table,
                        page_size, q_start, start_pos, n_reqs, max_q_len, max_ctx_len, window, scale,
                        out, short=None):
        self._count("paged_attention")
        group = num_heads // num_kv_heads
        qs = num_heads * head_dim
        for b in range(n_reqs):
            r0, r1 = int(q_start[b]), int(q_start[b + 1])
            sp = int(start_pos[b])
            end = sp + (r1 - r0)
            # the request's positions, read through its block table (a freed or
            # missing page reads as NaN, so a wrong access shows in the result)
            keys = torch.full((end, num_kv_heads, head_dim), float("nan"))
            vals = torch.full((end, num_kv_heads, head_dim), float("nan"))
            kidx = cache_layout.key_index(page_size, head_dim)
            vidx = cache_layout.value_index(page_size, head_dim)
            kflat = k_cache.view(k_cache.shape[0], num_kv_heads, -1)
            vflat = v_cache.view(v_cache.shape[0], num_kv_heads, -1)
            for j in range(end):
                pg = int(block_table[b, j // page_size])
                if pg >= 0:
                    keys[j] = kflat[pg][:, kidx[j % page_size]].float()
                    vals[j] = vflat[pg][:, vidx[:, j % page_size]].float()
            for r in range(r0, r1):
                p = sp + (r - r0)
                lo = 0 if window is None else max(0, p - window + 1)
                q = qkv[r, :qs].float().view(num_heads, head_dim)
                for h in range(num_heads):
                    kvh = h // group
                    s = (keys[lo:p + 1, kvh] @ q[h]) * scale
                    pr = torch.softmax(s, dim=0)
                    out[r, h * head_dim:(h + 1) * head_dim] = (pr @ vals[lo:p + 1, kvh]).to(out.dtype)

    # --------------------------------------------------------------- sampling
    def argmax(self, logits, out):
        self._count("argmax")
        for b in range(logits.shape[0]):
            row = logits[b]
            if torch.isnan(row).all():
                out[b] = -1
                continue
            row = torch.where(torch.isnan(row), torch.full_like(row, float("-inf")), row)
            m = row.max()
            out[b] = int((row == m).nonzero()[0, 0])

    def sample(self, logits, temperatures, uniforms, out):
        """temperature <= 0: argmax.  Else the smallest index whose cumulative
        probability under softmax(logits / t) reaches u * total."""
        self._count("sample")
        for b in range(logits.shape[0]):
            t = float(temperatures[b])
            if t <= 0.0:
                self.argmax(logits[b:b + 1], out[b:b + 1])
                continue
            z = logits[b].double() / t
            e = torch.exp(z - z.max())
            target = float(uniforms[b]) * float(e.sum())
            cum = torch.cumsum(e, dim=0)
            idx = int(torch.searchsorted(cum, torch.tensor(target, dtype=torch.float64)))
            out[b] = min(idx, logits.shape[1] - 1)
