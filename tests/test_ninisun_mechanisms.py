"""Each mechanism of Ninisun alone, against the plain implementation's function for it: the
kernel set's operation on the engine's own layouts (pages, block tables, state slots), once
as the PyTorch reference on the CPU and once as the HIP kernel on the GPU.  Where random
numbers would hide a fault, one query and key are scaled so that one score stands out."""
import math

import pytest
import torch

import helpers as H          # noqa: F401
import plain_ninisun as P
from test_vivevik_mechanisms import BACKENDS, DTYPES, F64, Paged, cache_rounded, close, ops_of, randn
from llm_inference_lab_amd.cache.layout import value_quads
from llm_inference_lab_amd.parts.base import PendingSums
from llm_inference_lab_amd.parts.positions import PairRotary


# ------------------------------------------------------------------ the stream
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("hidden", [8, 72, 1000, 2600])
def test_norm_of_a_result_into_the_stream(backend, hidden):
    ops = ops_of(backend)
    dev = ops.device
    y = randn(9, hidden, seed=1, scale=30.0).to(dev)
    w = (1.0 + randn(hidden, seed=2, scale=0.3)).to(dev)
    x = randn(9, hidden, seed=3).to(dev)
    want = x.cpu().to(F64) + P.rms_norm(y.cpu().to(F64), w.cpu().to(F64), 1e-5)
    ops.rmsnorm_add(y, w, 1e-5, x)
    close(x, want, torch.float32, "stream += norm(y)", f32=3e-6)
    # the result in three pieces
    pieces = randn(4, 9, hidden, seed=4).to(dev)
    x2 = randn(9, hidden, seed=5).to(dev)
    want = x2.cpu().to(F64) + P.rms_norm(pieces[:3].cpu().to(F64).sum(0), w.cpu().to(F64), 1e-3)
    ops.rmsnorm_add(PendingSums(pieces, 3), w, 1e-3, x2)
    close(x2, want, torch.float32, "stream += norm(sum of pieces)", f32=3e-6)
    # the norm that reads the stream next, in the same launch
    for dtype in DTYPES:
        x3 = randn(9, hidden, seed=6).to(dev)
        w_next = (1.0 + randn(hidden, seed=7, scale=0.3)).to(dev)
        h = torch.full((9, hidden), float("nan"), dtype=dtype, device=dev)
        want = x3.cpu().to(F64) + P.rms_norm(y.cpu().to(F64), w.cpu().to(F64), 1e-5)
        ops.rmsnorm_add(y, w, 1e-5, x3, (w_next, 1e-6, h))
        close(x3, want, torch.float32, "stream += norm(y), with the next norm", f32=3e-6)
        close(h, P.rms_norm(want, w_next.cpu().to(F64), 1e-6), dtype, "the next norm of the new rows")


@pytest.mark.parametrize("backend", BACKENDS)
def test_weighted_sum_of_two_results(backend):
    ops = ops_of(backend)
    a, b = randn(7, 50, seed=1).to(ops.device), randn(7, 50, seed=2).to(ops.device)
    out = torch.empty_like(a)
    ops.scaled_sum(out, a, 0.8, b, -1.7)
    close(out, 0.8 * a.cpu().to(F64) - 1.7 * b.cpu().to(F64), torch.float32, "a y1 + b y2", f32=1e-6)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 9, 40, 300])
def test_gelu_gate_as_the_epilogue_of_a_product(backend, dtype, rows):
    """Few rows and many (the product kernels differ), both dtypes: the tanh form of gelu on the
    gate's float32 sums, times the up product."""
    from llm_inference_lab_amd.parts.feed_forward import interleave_gate_up
    ops = ops_of(backend)
    x = randn(rows, 72, seed=5).to(dtype)
    gate, up = randn(200, 72, seed=6, scale=0.4).to(dtype), randn(200, 72, seed=7, scale=0.3).to(dtype)
    out = torch.empty(rows, 200, dtype=dtype, device=ops.device)
    ops.linear_swiglu(x.to(ops.device), ops.prepare_weight(interleave_gate_up(gate, up).to(ops.device)), out, "gelu_tanh")
    want = P.gelu_tanh(x.to(F64) @ gate.to(F64).T) * (x.to(F64) @ up.to(F64).T)
    close(out, want, dtype, "gelu(x Wg^T) * (x Wu^T)", f32=2e-5)
    # and silu still is what it was
    ops.linear_swiglu(x.to(ops.device), ops.prepare_weight(interleave_gate_up(gate, up).to(ops.device)), out)
    g = x.to(F64) @ gate.to(F64).T
    close(out, g * torch.sigmoid(g) * (x.to(F64) @ up.to(F64).T), dtype, "silu gate", f32=2e-5)


# ------------------------------------------------------------------ rotation
@pytest.mark.parametrize("rotation", [
    dict(dims=8, base=10000.0), dict(dims=20, base=2e5, scaling=dict(factor=3.0, original=512, fast=16.0, slow=2.0)),
    dict(dims=16, base=500.0, scaling=dict(factor=8.0, original=64, fast=4.0, slow=0.5)),
    dict(dims=2, base=7.0, scaling=dict(factor=2.0, original=16, fast=2.0, slow=2.0)),
])
def test_frequencies_and_their_stretching(rotation):
    part = PairRotary(dim=32, theta=rotation["base"], rotary_dim=rotation["dims"], scaling=rotation.get("scaling"))
    got, magnitude = part.frequencies()
    want, want_magnitude = P.rotary_frequencies(rotation)
    assert torch.allclose(torch.tensor(got, dtype=F64), want, rtol=1e-12, atol=0)
    assert abs(magnitude - want_magnitude) < 1e-12
    if "scaling" in rotation:        # the fastest pair is untouched, the slowest divided by the factor (where the ramp spans them)
        assert got[0] <= rotation["base"] ** 0 and got[-1] >= want[-1] - 1e-18


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,dims", [(16, 16), (24, 6), (9, 4), (32, 0)])
def test_projection_bias_rotation_value_mixing_and_the_cache_write(backend, dtype, D, dims):
    """Biases are added first; of every query and key head the first ``dims`` channels turn in
    neighbouring pairs by their row's position, the rest pass; values are mixed with the first
    layer's before they are stored; the gates pass through."""
    ops = ops_of(backend)
    dev = ops.device
    H_, G, E, n = 3, 1, 24, 37
    rotation = dict(dims=dims, base=50.0, scaling=dict(factor=3.0, original=16, fast=2.0, slow=0.5)) if dims else None
    cache = Paged(ops, dtype, [n + 300], G, D, E)
    sizes = (H_ * D, G * D, G * E, H_)
    proj = randn(n, sum(sizes) + 5, seed=5, scale=2.0)
    bias = randn(sum(sizes), seed=6)
    positions = [300 + i for i in range(n)]              # far from zero: angles of many turns
    freq, magnitude = (None, 1.0)
    if dims:
        f, magnitude = P.rotary_frequencies(rotation)
        freq = f.to(torch.float32).to(dev)
    first = randn(n, G * E, seed=8).to(dev)
    first_before = first.clone()
    p64 = proj.to(F64)[:, :sum(sizes)] + bias.to(F64)
    want_q = p64[:, :sizes[0]].view(n, H_, D)
    want_k = p64[:, sizes[0]:sizes[0] + sizes[1]].view(n, G, D)
    if dims:
        want_q, want_k = P.rotate_pairs(want_q, positions, rotation), P.rotate_pairs(want_k, positions, rotation)
    v64 = p64[:, sizes[0] + sizes[1]:sizes[0] + sizes[1] + sizes[2]]
    for mix, lam in (("mix", 0.3), ("first", 0.0), (None, 0.0)):
        q = torch.empty(n, H_ * D, dtype=dtype, device=dev)
        gate = torch.full((n, H_), float("nan"), device=dev)
        ops.project_rotate_write(proj.to(dev), H_, G, D, E, bias.to(dev), freq, dims, magnitude, mix, lam, first, gate, q,
                                 cache.k_cache, cache.v_cache, cache.page,
                                 torch.tensor(positions, dtype=torch.int32, device=dev),
                                 torch.zeros(n, dtype=torch.int32, device=dev), cache.table)
        close(q, want_q.reshape(n, -1), dtype, "queries", f32=1e-4)       # (float32 angles of 300 radians)
        close(gate, p64[:, -H_:], torch.float32, "gates", f32=1e-6)
        want_v = (0.7 * v64 + 0.3 * first_before.cpu().to(F64)) if mix == "mix" else v64
        if mix == "first":
            close(first, v64, torch.float32, "the first layer's values, unrounded", f32=1e-6)
        for pos in (300, 303, 304, 319, 320, 336):
            page = int(cache.table[0, pos // 16])
            close(cache.k_cache[page, :, pos % 16], want_k[pos - 300], dtype, f"key at {pos}", f32=1e-4)
            close(value_quads(cache.v_cache[page])[:, (pos % 16) >> 2, :, pos & 3], want_v[pos - 300].view(G, E), dtype,
                  f"value at {pos} ({mix})")


def test_rotation_is_relative():
    """What the scores see of two positions is their distance (the plain functions, as a check of
    the oracle itself): the same pair of vectors at (5, 2) and at (105, 102)."""
    rotation = dict(dims=8, base=100.0)
    q, k = randn(1, 1, 12, seed=1).to(F64), randn(1, 1, 12, seed=2).to(F64)
    a = (P.rotate_pairs(q, [5], rotation) * P.rotate_pairs(k, [2], rotation)).sum()
    b = (P.rotate_pairs(q, [105], rotation) * P.rotate_pairs(k, [102], rotation)).sum()
    assert abs(float(a - b)) < 1e-9


# ------------------------------------------------------------------ attention weights
def _paged_case(ops, dtype, lengths, new, H_, G, D, E, seed, stand_out=()):
    """Keys, values and queries of some requests in pages; ``stand_out``: (request, query position,
    key position) triples whose query is made to point at that key."""
    ks = [randn(n, G, D, seed=seed + i) for i, n in enumerate(lengths)]
    vs = [randn(n, G, E, seed=seed + 10 + i) for i, n in enumerate(lengths)]
    qs = [randn(n, H_, D, seed=seed + 20 + i) for i, n in enumerate(lengths)]
    for b, i, j in stand_out:
        for h in range(H_):
            qs[b][i, h] = ks[b][j, h // (H_ // G)] * 6.0 / ks[b][j, h // (H_ // G)].norm()
    cache = Paged(ops, dtype, lengths, G, D, E, seed=seed)
    for b, n in enumerate(lengths):
        proj = torch.cat([torch.zeros(n, H_ * D), ks[b].reshape(n, -1), vs[b].reshape(n, -1)], 1)
        cache.write(proj, H_, list(range(n)), [b] * n)
    rows_q = torch.cat([cache_rounded(qs[b][n - new[b]:], dtype) for b, n in enumerate(lengths)])
    positions = [p for b, n in enumerate(lengths) for p in range(n - new[b], n)]
    row_req = [b for b in range(len(lengths)) for _ in range(new[b])]
    return cache, ks, vs, qs, rows_q, positions, row_req


def _attend(cache, rows_q, H_, positions, row_req, window, keep_first, head_term, scale, weights):
    ops, dev = cache.ops, cache.ops.device
    out = torch.full((rows_q.shape[0], H_ * cache.E), float("nan"), dtype=cache.dtype, device=dev)
    pick = getattr(ops, "windowed_attention_long_rows", None)
    long_from = pick(cache.dtype, cache.D, cache.E, cache.page) if pick is not None else 0
    counts = [row_req.count(b) for b in range(max(row_req) + 1)]
    starts = [sum(counts[:b]) for b in range(len(counts) + 1)]
    launches = (1 if any(n < long_from for n in counts if n) else 0) | (2 if any(n >= long_from for n in counts) else 0)
    ops.sink_window_attention(rows_q.reshape(rows_q.shape[0], -1).to(cache.dtype).to(dev), H_, cache.G, cache.D, cache.E,
                              cache.k_cache, cache.v_cache, cache.table, cache.page,
                              torch.tensor(positions, dtype=torch.int32, device=dev),
                              torch.tensor(row_req, dtype=torch.int32, device=dev), window, keep_first, head_term, scale,
                              out, torch.tensor(starts, dtype=torch.int32, device=dev), long_from,
                              launches if long_from else 1, max(positions) + 1, weights=weights)
    return out


# sizes with and without matrix-core kernels; groups of 1, 2, 4 and 7 heads per key/value head
SHAPES = [(4, 2, 16, 24), (4, 2, 32, 16), (8, 2, 96, 64), (3, 1, 64, 48), (14, 2, 64, 64), (2, 2, 24, 200), (8, 2, 96, 192),
          (4, 1, 128, 256), (6, 2, 64, 192), (2, 2, 32, 192)]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H_,G,D,E", SHAPES)
def test_sigmoid_weights_over_prompts_and_decoded_rows(backend, dtype, H_, G, D, E):
    """No softmax: every visible key weighs sigmoid(score + bias of the head), nothing is
    normalised.  Portions of prompts behind a history, tiles of rows that hold two requests, single
    decoded rows behind hundreds of keys (cut into shares and merged), the very first position."""
    if backend == "emu" and H_ * (D + E) > 1400:
        pytest.skip("the references on the CPU take the small shapes; the kernels all of them")
    ops = ops_of(backend)
    lengths, new = [330, 45, 70, 1, 150], [50, 45, 1, 1, 1]
    stand = [(0, 329, 3), (0, 300, 299), (1, 44, 0), (2, 69, 17), (4, 149, 64)]      # far keys, page borders
    cache, ks, vs, qs, rows_q, positions, row_req = _paged_case(ops, dtype, lengths, new, H_, G, D, E, 30, stand)
    bias = torch.tensor([0.7 * h - 2.0 for h in range(H_)]).to(ops.device)
    scale = 0.9 / math.sqrt(D)
    out = _attend(cache, rows_q, H_, positions, row_req, None, 0, bias, scale, "sigmoid")
    at = 0
    for b, n in enumerate(lengths):
        want = P.sigmoid_attention(cache_rounded(qs[b][n - new[b]:], dtype).to(F64), cache_rounded(ks[b], dtype).to(F64),
                                   cache_rounded(vs[b], dtype).to(F64), scale, bias.cpu().to(F64))
        close(out[at:at + new[b]], want.reshape(new[b], -1), dtype, f"request {b}", f32=3e-5, bf16=2.5e-2)
        at += new[b]
    # without a bias, and nothing like a softmax: the weights of a row do not sum to one
    out0 = _attend(cache, rows_q, H_, positions, row_req, None, 0, None, scale, "sigmoid")
    want0 = P.sigmoid_attention(cache_rounded(qs[0][280:], dtype).to(F64), cache_rounded(ks[0], dtype).to(F64),
                                cache_rounded(vs[0], dtype).to(F64), scale, torch.zeros(H_, dtype=F64))
    close(out0[:50], want0.reshape(50, -1), dtype, "no bias", f32=3e-5, bf16=2.5e-2)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H_,G,D,E", [(4, 2, 16, 24), (4, 2, 32, 16), (8, 2, 64, 32), (8, 2, 96, 192), (2, 1, 128, 256)])
@pytest.mark.parametrize("window,keep_first", [(24, 3), (16, 0), (5, 9), (48, 7), (300, 2)])
def test_softmax_without_a_sink_at_the_window_s_edges(backend, dtype, H_, G, D, E, window, keep_first):
    """The plain softmax (no sink) through a window with a kept prefix: a key that would take nearly
    all the weight sits just inside or just outside, in a prompt's portion and for a decoded row."""
    if backend == "emu" and H_ * (D + E) > 1400:
        pytest.skip("the references on the CPU take the small shapes; the kernels all of them")
    ops = ops_of(backend)
    for decode in (False, True):
        n = 130
        for j_off, seen in ((window - 1, True), (window, False)):
            i = n - 1
            j = i - j_off
            if j < 0:
                continue
            seen = seen or j < keep_first
            lengths, new = [n, 20], [1 if decode else 40, 20]
            cache, ks, vs, qs, rows_q, positions, row_req = _paged_case(ops, dtype, lengths, new, H_, G, D, E, 50 + j_off,
                                                                        [(0, i, j)])
            out = _attend(cache, rows_q, H_, positions, row_req, window, keep_first, None, 1.0, "softmax")
            want = P.softmax_attention(cache_rounded(qs[0][n - new[0]:], dtype).to(F64), cache_rounded(ks[0], dtype).to(F64),
                                       cache_rounded(vs[0], dtype).to(F64), 1.0, window, keep_first)
            close(out[:new[0]], want.reshape(new[0], -1), dtype, f"window {window}, key {j}", f32=3e-5, bf16=2.5e-2)
            last = out[new[0] - 1, :E].float().cpu()
            near = float((last - cache_rounded(vs[0], dtype)[j, 0]).abs().max())
            assert (near < 0.1) == seen, f"query {i} {'misses' if seen else 'sees'} key {j} (window {window}, kept {keep_first})"
        # the kept prefix: its last key seen, the next one not (once the window has passed both)
        for j, seen in ((keep_first - 1, True), (keep_first, False)):
            i = n - 1
            if j < 0 or i - j < window:
                continue
            cache, ks, vs, qs, rows_q, positions, row_req = _paged_case(ops, dtype, [n], [1 if decode else 33], H_, G, D, E,
                                                                        70 + j, [(0, i, j)])
            out = _attend(cache, rows_q, H_, positions, row_req, window, keep_first, None, 1.0, "softmax")
            near = float((out[-1, :E].float().cpu() - cache_rounded(vs[0], dtype)[j, 0]).abs().max())
            assert (near < 0.1) == seen, f"kept prefix {keep_first}: query {i} and key {j}"


# ------------------------------------------------------------------ the delta rule
@pytest.mark.parametrize("backend", BACKENDS)
def test_decays_removal_rates_and_unit_keys(backend):
    ops = ops_of(backend)
    rows, rank, heads, D = 11, 5, 4, 13
    channels = heads * D
    proj = randn(rows, 3 + rank + 2 * channels, seed=1, scale=3.0)
    proj[3, 3 + rank + channels:3 + rank + channels + D] = 0.0            # a key of length zero: the eps keeps it finite
    proj = proj.to(ops.device)
    w2 = randn(channels, rank, seed=2, scale=2.0).to(ops.device)
    w0 = randn(channels, seed=3, scale=10.0).to(ops.device)                 # both ends of the sigmoid
    ab = randn(channels, seed=4, scale=5.0).to(ops.device)
    decay, unit, removal = (torch.empty(rows, channels, device=ops.device) for _ in range(3))
    ops.delta_gates(proj, 3, rank, 3 + rank, 3 + rank + channels, w2, w0, ab, math.exp(-0.5), 1e-6, heads, D, decay, unit,
                    removal)
    p = proj.cpu().to(F64)
    z = torch.tanh(p[:, 3:3 + rank]) @ w2.cpu().to(F64).T + w0.cpu().to(F64)
    close(decay, torch.exp(-math.exp(-0.5) * torch.sigmoid(z)), torch.float32, "decays", f32=3e-6)
    k = p[:, 3 + rank + channels:].view(rows, heads, D)
    u = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)).reshape(rows, channels)
    close(unit, u, torch.float32, "unit keys", f32=3e-6)
    close(removal, torch.sigmoid(p[:, 3 + rank:3 + rank + channels] + ab.cpu().to(F64)) * u, torch.float32, "removals", f32=3e-6)
    assert float(decay.min()) >= math.exp(-math.exp(-0.5)) - 1e-6 and float(decay.max()) <= 1.0
    assert torch.isfinite(unit).all()


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("chunk", [0, 16, 32])
@pytest.mark.parametrize("heads,D,E", [(2, 16, 16), (3, 24, 24), (1, 40, 40), (2, 64, 64), (1, 128, 128), (2, 8, 72), (1, 200, 16),
                                       (1, 32, 300)])
def test_delta_rule_scan_in_portions_with_states_in_slots(backend, heads, D, E, chunk):
    """Three requests of unequal length in one call, then their next portions (down to one token) in
    a second one from the states the first left in scattered slots, against the plain recurrence over
    the whole sequences; whole runs and chunks that run side by side (chunks that end inside a
    request's rows, requests shorter than a chunk)."""
    ops = ops_of(backend)
    dev = ops.device
    lengths, first = [137, 5, 64], [90, 4, 2]
    ld = 3 * heads * D + heads * E + 7
    off_r, off_k, off_v = 5, 5 + heads * D, 5 + 2 * heads * D
    state = torch.zeros(6, heads, D, E, device=dev)
    state[4] = 9.0                                   # (a slot nobody uses must stay as it is)
    slots = torch.tensor([3, 0, 5], dtype=torch.int32, device=dev)
    data, wants = [], []
    for b, n in enumerate(lengths):
        proj = randn(n, ld, seed=10 + b)
        decay = torch.exp(-0.6 * torch.rand(n, heads * D, generator=torch.Generator().manual_seed(20 + b)))
        rate = torch.rand(n, heads * D, generator=torch.Generator().manual_seed(30 + b))
        r, k = proj[:, off_r:off_r + heads * D].view(n, heads, D), proj[:, off_k:off_k + heads * D].view(n, heads, D)
        v = proj[:, off_v:off_v + heads * E].view(n, heads, E)
        unit = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)).reshape(n, -1)
        data.append((proj, decay, unit, rate * unit))
        wants.append(_plain_delta(r.to(F64), k.to(F64), v.to(F64), decay.view(n, heads, D).to(F64),
                                  rate.view(n, heads, D).to(F64)))
    for part in (0, 1):
        spans = [(0, first[b]) if part == 0 else (first[b], lengths[b]) for b in range(3)]
        proj, decay, unit, removal = (torch.cat([data[b][i][lo:hi] for b, (lo, hi) in enumerate(spans)]).to(dev)
                                      for i in range(4))
        starts = [0]
        for lo, hi in spans:
            starts.append(starts[-1] + hi - lo)
        rows = proj.shape[0]
        out = torch.full((rows, heads, 1, E), float("nan"), device=dev)
        most = rows // chunk + 3 if chunk else 0
        ops.delta_scan(proj, off_r, off_k, off_v, decay, unit, removal, heads, D, E, state,
                       torch.tensor(starts, dtype=torch.int32, device=dev), slots, 3, out, chunk,
                       torch.full((most, heads, D, E), float("nan"), device=dev) if chunk else None,
                       torch.full((most, heads, D, D), float("nan"), device=dev) if chunk else None)
        for b, (lo, hi) in enumerate(spans):
            close(out[starts[b]:starts[b + 1], :, 0], wants[b][0][lo:hi], torch.float32, f"request {b}, part {part}", f32=3e-5)
    for b in range(3):
        close(state[int(slots[b])], wants[b][1], torch.float32, f"state of request {b}", f32=3e-5)
    assert float((state[4] - 9.0).abs().max()) == 0.0


def _plain_delta(r, k, v, w, a):
    """(The plain recurrence takes square states; this is its equation for values of another width.)"""
    if v.shape[-1] == r.shape[-1]:
        return P.delta_rule(r, k, v, w, a)
    T, H_, D = r.shape
    S = torch.zeros(H_, D, v.shape[-1], dtype=F64)
    out = torch.zeros(T, H_, v.shape[-1], dtype=F64)
    for t in range(T):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + 1e-6)
        S = w[t].unsqueeze(-1) * S - (a[t] * u).unsqueeze(-1) * torch.einsum("hd,hde->he", u, S).unsqueeze(-2) \
            + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = torch.einsum("hde,hd->he", S, r[t])
    return out, S


def test_delta_rule_removes_what_the_key_held():
    """The oracle's own sense: with no decay (w = 1) and a full removal rate (a = 1), writing the
    same unit key twice leaves only the second value under it."""
    D = 8
    k = torch.zeros(2, 1, D, dtype=F64)
    k[:, 0, 2] = 1.0
    v = randn(2, 1, D, seed=1).to(F64)
    ones = torch.ones(2, 1, D, dtype=F64)
    out, S = P.delta_rule(k.clone(), k, v, ones, ones)
    assert torch.allclose(out[1, 0], v[1, 0], atol=1e-5)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_unit_norm_weight_of_all_heads_and_sigmoid_gate(backend, dtype):
    """Every head's output divided by its own root mean square, a weight that differs from head to
    head, the sigmoid (not silu) of the gate."""
    ops = ops_of(backend)
    rows, heads, E = 9, 3, 40
    parts = randn(rows, heads, 1, E, seed=1, scale=5.0)
    parts[:, 1] *= 100.0                          # (a norm over all heads at once would differ)
    weight = (1.0 + randn(heads * E, seed=2, scale=0.5))
    proj = randn(rows, 11 + heads * E, seed=3, scale=2.0)
    out = torch.empty(rows, heads * E, dtype=dtype, device=ops.device)
    ops.gla_output(parts.to(ops.device), heads, 16, E, weight.to(ops.device), 1e-5, proj.to(ops.device), 11, out, "sigmoid")
    o = parts[:, :, 0].to(F64)
    want = P.unit_rms(o, 1e-5).reshape(rows, -1) * weight.to(F64) * torch.sigmoid(proj[:, 11:].to(F64))
    close(out, want, dtype, "norm, weight, gate", f32=2e-5)
