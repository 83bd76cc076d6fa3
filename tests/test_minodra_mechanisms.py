"""Minodra's mechanisms one by one against the plain implementation's functions (tests/plain_minodra.py):
the norm with one number as its weight, the embedding with hashed pairs over steps, the short
convolution over cuts (with an input that shows which taps were read), the gated sum, the sigmoid
router's choice and weights, the mixture of squared-ReLU experts with its gated shared expert, the soft
cap, and the latent attention in one-layer models whose tensors make one key stand out: far back among
hundreds, on both sides of page borders, in prompts and decoded, with a sink that takes most of the
weight or almost none.  Every body runs on the CPU with the kernels' PyTorch references and on the GPU
with the kernels."""
import math

import pytest
import torch

import helpers as H          # noqa: F401
import minodra_cases as M
import plain_minodra as P
from emu_ops import EmuOps
from llm_inference_lab_amd.config.spec import PartSpec
from llm_inference_lab_amd.parts import RMSNorm, RoutedExperts

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def ops_of(backend):
    if backend == "emu":
        return EmuOps()
    from llm_inference_lab_amd.kernels.hip_ops import HipOps
    return HipOps("cuda:0")


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def ints(values, device):
    return torch.tensor(values, dtype=torch.int32, device=device)


def close(got, want, dtype, what="", f32=2e-5, bf16=2e-2):
    err = float((got.detach().cpu().double() - want.double()).abs().max())
    size = max(1.0, float(want.abs().max()))
    assert err <= (f32 if dtype == torch.float32 else bf16) * size, f"{what}: off by {err} (values up to {size})"


class Scratch:
    """The least a part needs of a step: named scratch buffers and no sums owed."""

    def __init__(self, device):
        self.device, self.pending, self.memo = device, None, {}

    def scratch(self, name, shape, dtype):
        return torch.zeros(shape, dtype=dtype, device=self.device)


def description(portions, slots, device):
    """row_req, q_start, req_rows of a step whose request b brings ``portions[b]`` rows and lives in
    slot ``slots[b]``."""
    row_req, q_start = [], [0]
    for b, n in enumerate(portions):
        row_req += [b] * n
        q_start.append(q_start[-1] + n)
    return ints(row_req, device), ints(q_start, device), ints(slots, device)


# ------------------------------------------------------------------ norm, embedding, cap
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,eps", [(8, 1e-6), (72, 1e-3), (1000, 1e-5)])
def test_norm_with_one_number_as_its_weight(backend, dtype, hidden, eps):
    ops = ops_of(backend)
    part = RMSNorm(hidden, eps, dict(weight="n"), scalar=True)
    assert part.tensor_specs()["n"].shape == ()
    g = torch.tensor(1.37).to(torch.bfloat16)
    part.bind({"n": g.to(ops.device)}, ops, dtype)
    x = randn(9, hidden, seed=1, scale=3.0)
    x[3] *= 1e-3                                       # (a row small enough for eps to matter)
    out = torch.zeros(9, hidden, dtype=dtype, device=ops.device)
    part.forward(x.to(ops.device), out)
    close(out, P.scalar_norm(x.to(F64), g, eps), dtype, "norm")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("buckets,mul_prev,mul_cur", [(61, 113, 11), (1, 3, 5), (1019, 1, 1), (7, 1000003, 999983)])
def test_hashed_pairs_over_steps(backend, buckets, mul_prev, mul_cur):
    """Two sequences fed in unequal portions through slots 2 and 0; the previous token crosses every
    cut through the slot, and a sequence's first token takes the row behind the buckets."""
    ops = ops_of(backend)
    dev, vocab, hidden, eps = ops.device, 300, 40, 1e-5
    w = {"embed": randn(vocab, hidden, seed=1).to(torch.bfloat16), "bigram": randn(buckets + 1, hidden, seed=2).to(torch.bfloat16),
         "embed.norm": torch.tensor(0.8).to(torch.bfloat16)}
    cfg = dict(embedding=dict(scale=2.5, bigram=dict(buckets=buckets, mul_prev=mul_prev, mul_cur=mul_cur)), norm=dict(eps=eps))
    seqs = [[int(t) for t in torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(5 + n))] for n in (11, 6)]
    want = [P.embed(s, cfg, w) for s in seqs]
    table, pairs = w["embed"].float().to(dev), w["bigram"].float().to(dev)
    norm_w = w["embed.norm"].float().reshape(1).expand(hidden).contiguous().to(dev)
    previous = torch.zeros(4, 1, dtype=torch.int32, device=dev)
    done = [0, 0]
    for portions in ([4, 1], [1, 3], [6, 2]):
        ids, positions = [], []
        for b, n in enumerate(portions):
            ids += seqs[b][done[b]:done[b] + n]
            positions += list(range(done[b], done[b] + n))
        row_req, q_start, req_rows = description(portions, [2, 0], dev)
        out = torch.zeros(sum(portions), hidden, device=dev)
        ops.embed_pairs(table, pairs, ints(ids, dev), ints(positions, dev), row_req, q_start, req_rows, previous, 2.5,
                        buckets, mul_prev, mul_cur, norm_w, eps, out)
        at = 0
        for b, n in enumerate(portions):
            close(out[at:at + n], want[b][done[b]:done[b] + n], torch.float32, f"request {b} from {done[b]}")
            at += n
            done[b] += n


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cap", [25.0, 5.0, 0.7])
def test_soft_cap(backend, cap):
    ops = ops_of(backend)
    x = randn(7, 33, seed=3, scale=20.0)
    got = x.clone().to(ops.device)
    ops.softcap(got, cap)
    close(got, cap * torch.tanh(x.to(F64) / cap), torch.float32, "cap")
    assert float(got.abs().max()) <= cap


# ------------------------------------------------------------------ convolution, gated sum
def conv_over_cuts(ops, dtype, h, weight, cuts, fused, norm_w=None, eps=1e-5):
    """One sequence in slot 1 beside a decoy in slot 0, fed in the portions ``cuts``."""
    dev = ops.device
    n, width = h.shape
    taps = weight.shape[1]
    state = torch.zeros(3, max(taps - 1, 0), width, dtype=dtype, device=dev) if taps > 1 else None
    out, at = [], 0
    for step, c in enumerate(cuts):
        decoy = randn(2, width, seed=90 + step)
        x = torch.cat([decoy, h[at:at + c]]).to(dev)
        row_req, q_start, req_rows = description([2, c], [0, 1], dev)
        res = torch.zeros(2 + c, width, dtype=dtype, device=dev)
        if fused:
            normed = torch.zeros_like(res)
            ops.norm_conv(x.float(), norm_w.to(dev), eps, weight.to(dev), state, row_req, q_start, req_rows, normed, res, False)
        else:
            ops.causal_conv(x.to(dtype), weight.to(dev), state, None, row_req, q_start, req_rows, res)
        out.append(res[2:].cpu())
        at += c
    return torch.cat(out)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7, 11])
@pytest.mark.parametrize("cuts", [[23], [1] * 23, [2, 2, 3, 1, 9, 2, 4], [5, 18]])
def test_convolution_over_cuts(backend, dtype, taps, cuts):
    """``h + conv(h)`` of a sequence cut into portions (shorter than the taps, single tokens, whole)
    against the plain implementation over the whole sequence."""
    ops = ops_of(backend)
    width = 24
    h = randn(23, width, seed=taps).to(torch.bfloat16).float()
    weight = randn(width, taps, seed=50 + taps, scale=0.7)
    want = h.to(F64) + P.causal_conv(h.to(F64), weight)
    close(conv_over_cuts(ops, dtype, h, weight, cuts, fused=False), want, dtype, "convolution")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("taps", [2, 4, 8])
def test_an_input_reaches_exactly_the_taps(backend, taps):
    """One input row stands alone among zeros: the outputs of its own position and the ``taps - 1``
    after it carry it, each through its own tap, and the position ``taps`` after it does not, also
    where a cut lies between them (the norm and the convolution in one launch, and apart)."""
    ops = ops_of(backend)
    width, at, n = 16, 5, 20
    x = torch.zeros(n, width)
    x[at] = randn(width, seed=1).abs() + 1.0
    weight = randn(width, taps, seed=2).abs() + 1.0
    g, eps = torch.full((width,), 1.5), 1e-5
    h = P.scalar_norm(x.to(F64), torch.tensor(1.5), eps)
    want = h + P.causal_conv(h, weight)
    for t in range(n):
        seen = at <= t < at + taps
        assert bool(want[t].min() > 0.5) == seen and (seen or float(want[t].abs().max()) == 0.0)
    for cuts in ([n], [at + 1, n - at - 1], [at, 1, 1, 1, n - at - 3], [at + taps - 1, 1, n - at - taps],
                 [at + taps, n - at - taps], [1] * n):
        got = conv_over_cuts(ops, torch.float32, x, weight, cuts, fused=True, norm_w=g, eps=eps)
        close(got, want, torch.float32, f"norm and convolution, cuts {cuts}")
        got = conv_over_cuts(ops, torch.float32, h.float(), weight, cuts, fused=False)
        close(got, want, torch.float32, f"convolution, cuts {cuts}")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("rows,width", [(1, 8), (6, 72), (40, 328)])
def test_gated_sum_into_the_stream(backend, rows, width):
    ops = ops_of(backend)
    x, y, h = randn(rows, width, seed=1), randn(rows, width, seed=2), randn(rows, width, seed=3)
    w, b = randn(width, width, seed=4, scale=2.0 / width ** 0.5), randn(width, seed=5)
    want = x.to(F64) + y.to(F64) * P.residual_gate(h.to(F64), w, b)
    gate = (h.to(F64) @ w.to(F64).T).float()
    got = x.clone().to(ops.device)
    ops.gated_add(got, y.to(ops.device), gate.to(ops.device), b.to(ops.device))
    close(got, want, torch.float32, "gated sum")


# ------------------------------------------------------------------ router, mixture
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top", [(8, 4), (5, 1), (6, 6), (64, 8), (100, 3)])
def test_the_sigmoid_routers_choice_and_weights(backend, experts, top):
    """The choice is made on score + correction, the weights are the scores without it and are not
    normalised; equal choice values go to the smaller index."""
    ops = ops_of(backend)
    rows, width = 33, 48
    h = randn(rows, width, seed=1).to(torch.bfloat16)
    w = {"router": randn(experts, width, seed=2, scale=2.0 / width ** 0.5).to(torch.bfloat16),
         "correction": randn(experts, seed=3, scale=0.4)}
    logits = (h.to(F64) @ w["router"].to(F64).T).float()
    logits[0] = 0.0                                    # (a row of equal scores: the correction alone decides)
    logits[1, :] = logits[1, 0]
    want_c, want_w = P.route(h.to(F64), w, "", top)
    s = torch.sigmoid(logits.to(F64))
    order = torch.sort(s + w["correction"].to(F64), dim=-1, descending=True, stable=True).indices[:, :top]
    want_c[:2], want_w[:2] = order[:2], torch.gather(s, 1, order)[:2]
    got_c = torch.zeros(rows, top, dtype=torch.int32, device=ops.device)
    got_w = torch.zeros(rows, top, device=ops.device)
    ops.moe_select(logits.to(ops.device), w["correction"].float().to(ops.device), 1, 1, 1.0, got_c, got_w, scoring="sigmoid")
    choice = s + w["correction"].to(F64)
    gaps = (choice[:, :, None] - choice[:, None, :]).abs() + torch.eye(experts, dtype=F64)[None] * 9.0
    sure = gaps.flatten(1).min(-1).values > 1e-6
    sure[:2] = True
    assert int(sure.sum()) > rows // 2
    assert torch.equal(got_c.cpu().long()[sure], want_c[sure])
    close(got_w.cpu()[sure], want_w[sure], torch.float32, "weights", f32=1e-6)
    # the weights are the scores, not what the choice was made on, and are not normalised
    assert float((torch.gather(choice, 1, want_c) - want_w).abs().max()) > 0.1
    if top > 2:
        assert float(got_w.sum(-1).max()) > 1.0


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 5, 70, 300])
@pytest.mark.parametrize("shape", [dict(experts=6, top=3, shared=40, ff=24, width=64),
                                   dict(experts=5, top=1, shared=None, ff=20, width=48),
                                   dict(experts=3, top=3, shared=12, ff=8, width=72),
                                   dict(experts=40, top=6, shared=64, ff=32, width=128)])
def test_the_mixture_of_experts_alone(backend, dtype, rows, shape):
    """The part with its own tensors against the plain implementation's mixture; rows whose choice
    rests on a close call are left out of the comparison (not of the batch)."""
    ops = ops_of(backend)
    width, ff, n, top = shape["width"], shape["ff"], shape["experts"], shape["top"]
    names = dict(router="m.router", correction="m.correction", expert_up="m.e{}.up", expert_down="m.e{}.down")
    shared = None
    if shape["shared"] is not None:
        shared = PartSpec("dense", params=dict(hidden_size=width, intermediate_size=shape["shared"], activation="relu2"),
                          tensors=dict(up_weight="m.shared.up", down_weight="m.shared.down"))
        names["shared_gate"] = "m.shared.sg"
    part = RoutedExperts(width, ff, n, top, names, correction=True, scoring="sigmoid", expert_form="relu2", shared=shared,
                         shared_gate=shared is not None)
    tensors = {}
    for i, (name, spec) in enumerate(part.tensor_specs().items()):
        if name.endswith("correction"):
            t = randn(*spec.shape, seed=100 + i, scale=0.3)
        elif name.endswith(("router", "shared.sg")):
            t = randn(*spec.shape, seed=100 + i, scale=3.0 / width ** 0.5)
        else:
            t = randn(*spec.shape, seed=100 + i, scale=1.0 / spec.shape[-1] ** 0.5)
        tensors[name] = t.to(torch.bfloat16)
    h = randn(rows, width, seed=11).to(torch.bfloat16)
    plain_w = {k[2:]: v.to(F64) for k, v in tensors.items()}
    raw = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=n, top=top))
    if shared is not None:
        raw["shared"] = dict(ff=shape["shared"])
    want = P.mixture(h.to(F64), raw, plain_w, "")
    c = torch.sigmoid(h.to(F64) @ plain_w["router"].T) + plain_w["correction"]
    gaps = (c[:, :, None] - c[:, None, :]).abs() + torch.eye(n, dtype=F64)[None] * 9.0
    sure = gaps.flatten(1).min(-1).values > 1e-5
    assert int(sure.sum()) >= rows // 2
    kept = {k: (v.to(ops.device) if dtype == torch.bfloat16 or v.dim() != 2 else v.float().to(ops.device))
            for k, v in tensors.items()}
    part.bind(kept, ops, dtype)
    resid = randn(rows, width, seed=12)
    got = resid.clone().to(ops.device)
    ctx = Scratch(ops.device)
    part.forward(h.to(dtype).to(ops.device), got, ctx)
    if ctx.pending is not None:
        ops.add_pending(got, ctx.pending)
    close(got.cpu()[sure], (resid.to(F64) + want)[sure], dtype, "stream + mixture", f32=5e-5, bf16=4e-2)


# ------------------------------------------------------------------ latent attention: keys that stand out
def one_layer_with_a_key_that_stands_out(heads=3, dim=16, vdim=8, q_rank=24, kv_rank=40, width=64, vocab=40, sink=0.0):
    """A model of one latent attention layer (no convolution's memory: one tap of weight zero; no
    feed-forward) in which the key of token 1 takes nearly all the weight of the query of token 2
    whenever it is seen: one channel of every head's key and query carries a large product for that
    pair and nearly nothing for the filler tokens.  Returns (raw config, tensors)."""
    raw = dict(architecture="Minodra", vocab=vocab, width=width, norm=dict(eps=1e-6), canon=dict(taps=1),
               embedding=dict(scale=1.0), layers=[M.latent(heads, dim, vdim, q_rank, kv_rank, 1.0, mlp=None)])
    cfg = H.lab.MinodraConfig.from_dict(raw)
    t = M.make_tensors(cfg, 3, sharp=0.3)
    t["l0.canon1"] = torch.zeros_like(t["l0.canon1"])
    t["l0.mix.sink"] = torch.full_like(t["l0.mix.sink"], sink)
    eps = 1e-6
    h = P.scalar_norm(P.embed(list(range(vocab)), raw, t), t["l0.norm1"], eps)           # every token's input of the mixer
    # the key's side: a direction of the cached latent that token 1 has and the fillers have little of
    c = P.vector_norm(h @ t["l0.mix.dkv"].to(F64).T, t["l0.mix.dkv.norm"], eps)
    cq = P.vector_norm(h @ t["l0.mix.dq"].to(F64).T, t["l0.mix.dq.norm"], eps)
    uk, uq = t["l0.mix.uk"].to(F64) * 0.2, t["l0.mix.uq"].to(F64) * 0.2
    for a in range(heads):
        uk[a * dim + dim - 1] = 4.0 * c[1] / (c[1] @ c[1])
        uq[a * dim + dim - 1] = 4.0 * cq[2] / (cq[2] @ cq[2])
    t["l0.mix.uk"], t["l0.mix.uq"] = uk.to(torch.bfloat16), uq.to(torch.bfloat16)
    return raw, t


def run_prompt_or_decode(raw, tensors, ids, backend, decode_from, page_size=16, dtype="f32"):
    cfg = H.lab.MinodraConfig.from_dict(raw)
    kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
    engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=page_size, num_pages=40,
                          max_requests=1, max_batch_tokens=512, max_seq_len=512, **kw)
    req = engine.open("r")
    if decode_from >= len(ids):
        out = engine.step([H.lab.StepEntry(req, ids, [len(ids) - 1])])
    else:
        engine.step([H.lab.StepEntry(req, ids[:decode_from], [])])
        for i in range(decode_from, len(ids)):
            out = engine.step([H.lab.StepEntry(req, [ids[i]], [0])])
    return out.float().cpu()[0].double()


def with_and_without(raw, tensors, length, back):
    ids = [3 + (7 * i) % 30 for i in range(length)]
    ids[-1] = 2
    without = list(ids)
    if back > 0:
        ids[-1 - back] = 1
    return ids, without


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoded", [False, True])
def test_a_key_anywhere_in_the_past_is_seen(backend, decoded):
    """Attention without positions and without a window: the key that stands out is seen next to the
    query, at the sequence's start and on both sides of the borders of the 16-token pages; the plain
    implementation itself says that the key matters (its logits with and without differ)."""
    raw, tensors = one_layer_with_a_key_that_stands_out()
    for at in (20, 31, 32, 47):                        # the query's position, around page borders
        for back in sorted({1, 2, 15, 16, 17, at - 16, at - 15, at}):
            if not 0 < back <= at:
                continue
            ids, without = with_and_without(raw, tensors, at + 1, back)
            want = M.plain_of(raw, tensors, ids)[-1]
            assert float((M.plain_of(raw, tensors, without)[-1] - want).abs().max()) > 0.3, "the key does not stand out"
            got = run_prompt_or_decode(raw, tensors, ids, backend, at if decoded else at + 1)
            assert float((got - want).abs().max()) < 2e-4, (at, back)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("sizes", [dict(heads=4, dim=32, vdim=16, q_rank=48, kv_rank=64),
                                   dict(heads=2, dim=8, vdim=24, q_rank=8, kv_rank=136),
                                   dict(heads=3, dim=16, vdim=16, q_rank=24, kv_rank=300),
                                   dict(heads=5, dim=12, vdim=12, q_rank=20, kv_rank=40)])
def test_a_far_key_among_hundreds(backend, decoded, sizes):
    raw, tensors = one_layer_with_a_key_that_stands_out(**sizes)
    for back in (250, 329):
        ids, without = with_and_without(raw, tensors, 330, back)
        want = M.plain_of(raw, tensors, ids)[-1]
        assert float((M.plain_of(raw, tensors, without)[-1] - want).abs().max()) > 0.3
        got = run_prompt_or_decode(raw, tensors, ids, backend, 300 if decoded else 330, page_size=64)
        assert float((got - want).abs().max()) < 2e-4, back


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("sink", [-20.0, 8.0, 11.0])
def test_the_sink_counts_once_and_is_not_scaled(backend, decoded, sink):
    """A sink far below the scores changes nothing; one of the size of the largest score (the key that
    stands out scores 8 after the scale) takes half of that query's weight or most of it, and the plain
    implementation with half the sink differs, so a lost sink, a sink counted per key or a scaled one
    would show."""
    raw, tensors = one_layer_with_a_key_that_stands_out(sink=sink)
    raw["layers"][0]["mixer"]["scale"] = 0.5           # (a scaled sink would count as exp(sink / 2))
    ids, _ = with_and_without(raw, tensors, 40, 7)
    want = M.plain_of(raw, tensors, ids)[-1]
    other = dict(tensors)
    other["l0.mix.sink"] = torch.full_like(tensors["l0.mix.sink"], sink * 0.5 if sink > 0 else -40.0)
    differs = float((M.plain_of(raw, other, ids)[-1] - want).abs().max())
    assert (differs > 0.05) == (sink > 0), differs
    got = run_prompt_or_decode(raw, tensors, ids, backend, 33 if decoded else 40)
    assert float((got - want).abs().max()) < 2e-4


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_first_tokens_of_a_sequence(backend):
    """Positions 0, 1, 2 as a prompt and token by token: the first has one key, its own, and the sink."""
    raw, tensors = one_layer_with_a_key_that_stands_out(sink=1.0)
    for ids in ([2], [1, 2], [1, 7, 2], [9, 1, 2, 2]):
        want = M.plain_of(raw, tensors, ids)[-1]
        for decode_from in (len(ids), 1):
            got = run_prompt_or_decode(raw, tensors, ids, backend, decode_from)
            assert float((got - want).abs().max()) < 2e-4, (ids, decode_from)


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_gate_of_a_head_reads_the_mixers_input(backend):
    """With the gate's matrix set so that one head's gate is closed for one token and open for the
    others, that head's output is gone at that token's positions only."""
    raw, tensors = one_layer_with_a_key_that_stands_out(sink=-20.0)
    eps, vocab = 1e-6, raw["vocab"]
    h = P.scalar_norm(P.embed(list(range(vocab)), raw, tensors), tensors["l0.norm1"], eps)
    g = tensors["l0.mix.g"].to(F64) * 0.1
    g[1] = -12.0 * h[2] / (h[2] @ h[2])                 # head 1 closes where the input is token 2's
    tensors["l0.mix.g"] = g.to(torch.bfloat16)
    ids, _ = with_and_without(raw, tensors, 24, 5)
    want = M.plain_of(raw, tensors, ids)[-1]
    open_gate = dict(tensors)
    open_gate["l0.mix.g"] = (g * 0).to(torch.bfloat16)
    assert float((M.plain_of(raw, open_gate, ids)[-1] - want).abs().max()) > 0.05
    for decode_from in (24, 20):
        got = run_prompt_or_decode(raw, tensors, ids, backend, decode_from)
        assert float((got - want).abs().max()) < 2e-4
    assert math.isfinite(float(want.abs().max()))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("fold", [0, 100])
@pytest.mark.parametrize("name", ["A", "B"])
def test_the_querys_two_products_as_one_matrix_or_apart(backend, fold, name, monkeypatch):
    """``U_a^T (W_uq c_q)`` in two products, or ``(U_a^T W_uq) c_q`` with one matrix made when the part
    is bound: the same logits, in every layer of a configuration whatever its sizes would choose."""
    from llm_inference_lab_amd.parts.latent_attention import LatentAttention
    monkeypatch.setattr(LatentAttention, "FOLD_UP_TO", fold)
    cfg = M.config_of(name)
    ids = M.random_ids(cfg, 41, 3)
    want = M.plain_logits(name, 1, ids)
    kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
    engine = M.make_engine(name, 1, "f32", **kw)
    assert all(b.mixer.fold_query == (fold > 0) for b in engine.model.blocks)
    req = engine.open("r")
    first = engine.step([H.lab.StepEntry(req, ids[:30], list(range(30)))]).float().cpu().double()
    rest = [engine.step([H.lab.StepEntry(req, [t], [0])]).float().cpu().double()[0] for t in ids[30:]]
    got = torch.cat([first, torch.stack(rest)])
    assert float((got - want).abs().max()) < 2e-4
