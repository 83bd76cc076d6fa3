"""Ninisun through the engine (its cache and state manager, step function, scheduler) against
the plain implementation: once on the CPU with the per-kernel PyTorch references in place
of the HIP kernels, once on the GPU with the kernels themselves."""
import pytest
import torch

import helpers as H
import ninisun_cases as N
import plain_ninisun
from emu_ops import EmuOps

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]
LENGTHS = {"P": [1, 9, 37, 83], "Q": [2, 30, 71], "R": [5, 52, 90], "S": [4, 41, 66]}
# Logits have a standard deviation of about 2.  float32: sums in another order than the float64
# plain implementation.  bfloat16: bounds on the root mean square and the largest difference over
# all logits, twice what the kernels' references in float32 arithmetic with the same roundings
# are off the plain implementation at these sharp configurations.
TOL = {"f32": 2e-4}
TOL_BF16 = (0.12, 1.2)      # (root mean square, max)


def engine_of(name, backend, dtype, **kw):
    if backend == "emu":
        return N.make_engine(name, 1, dtype, ops=EmuOps(), device="cpu", **kw)
    return N.make_engine(name, 1, dtype, **kw)


def sequences_of(name, lengths=None):
    cfg = N.config_of(name)
    return {f"r{i}": N.random_ids(cfg, n, 10 + i) for i, n in enumerate(lengths or LENGTHS[name])}


def all_decode(seqs):
    """Every token in a step of its own: what a prompt's step computed must equal this."""
    steps = []
    for rid, ids in seqs.items():
        steps += [([(rid, 1, True)], [rid] if i == len(ids) - 1 else []) for i in range(len(ids))]
    return steps


CUTS = {"whole": H.steps_whole, "decode": H.steps_prefill_then_decode, "token by token": all_decode,
        "portions": H.steps_portions,
        "small portions": lambda s: H.steps_portions(s, sizes=(2, 3, 2, 5, 2, 2, 17, 2)),
        "mixed": H.steps_mixed}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
@pytest.mark.parametrize("cut", list(CUTS))
def test_every_cut_matches_plain(backend, name, cut):
    """Whole prompts, decoding, portions down to two tokens, mixed batches with few pages and
    slots (freed and used again): the logits at every position are the plain implementation's."""
    seqs = sequences_of(name)
    want = {rid: N.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    engine = engine_of(name, backend, "f32", page_size=16, num_pages=14, max_requests=3 if cut == "mixed" else 2)
    steps = CUTS[cut](seqs) if cut != "mixed" else H.steps_mixed(seqs, max_live=3)
    got = H.run_trace(engine, seqs, steps)
    bad = H.first_wrong(got, want, TOL["f32"])
    assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
    engine.cache.check()
    m = engine.cache.metrics()
    assert m["rows_used"] == 0 and all(g["pages_used"] == 0 for g in m["groups"])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_bfloat16_mixed_batches(backend, name):
    seqs = sequences_of(name)
    want = {rid: N.plain_logits(name, 1, ids) for rid, ids in seqs.items()}
    engine = engine_of(name, backend, "bf16", page_size=16, num_pages=14, max_requests=3)
    got = H.run_trace(engine, seqs, H.steps_mixed(seqs, max_live=3))
    diff = torch.cat([got[rid].double() - want[rid] for rid in got])
    assert not torch.isnan(diff).any()
    rms, worst = float(diff.pow(2).mean().sqrt()), float(diff.abs().max())
    assert rms < TOL_BF16[0] and worst < TOL_BF16[1], (rms, worst)


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_batch_of_unequal_requests_equals_each_alone(backend):
    """The same positions computed alone and beside other requests: the same numbers, beyond the
    order of a few sums."""
    name = "P"
    seqs = sequences_of(name, [3, 61, 28])
    alone = {}
    for rid, ids in seqs.items():
        engine = engine_of(name, backend, "f32", max_requests=1)
        alone.update(H.run_trace(engine, {rid: ids}, H.steps_whole({rid: ids})))
    engine = engine_of(name, backend, "f32", max_requests=3)
    reqs = {rid: engine.open(rid) for rid in seqs}
    out = engine.step([H.lab.StepEntry(reqs[rid], ids, list(range(len(ids)))) for rid, ids in seqs.items()]).float().cpu()
    at = 0
    for rid, ids in seqs.items():
        err = float((out[at:at + len(ids)] - alone[rid]).abs().max())
        assert err < 2e-5, (rid, err)
        at += len(ids)


@pytest.mark.parametrize("backend", BACKENDS)
def test_window_pages_are_given_back_and_the_kept_prefix_stays(backend):
    """A long decode through windows that cross many pages: pages behind the window go back to
    the pool while the pages of the kept first positions stay, and the logits stay right."""
    name = "P"
    cfg = N.config_of(name)
    ids = N.random_ids(cfg, 150, 5)
    engine = engine_of(name, backend, "f32", page_size=16, num_pages=24, max_requests=1)
    req = engine.open("long")
    want = N.plain_logits(name, 1, ids)
    out = engine.step([H.lab.StepEntry(req, ids[:20], [19])]).float().cpu()
    assert float((out[0].double() - want[19]).abs().max()) < TOL["f32"]
    for i in range(20, len(ids)):
        out = engine.step([H.lab.StepEntry(req, [ids[i]], [0])]).float().cpu()
        assert float((out[0].double() - want[i]).abs().max()) < TOL["f32"], f"decoded position {i}"
    held = {gi: [lp for lp, p in enumerate(pages) if p >= 0] for gi, pages in enumerate(req.pages)}
    windowed = 0
    for gi, g in enumerate(engine.cache.groups):
        if g.window is not None and g.window < 100:
            windowed += 1
            if g.spec.keep_first:
                assert held[gi][0] == 0, "the page of the kept first positions was given back"
            assert len(held[gi]) < len(req.pages[gi]), "no page behind the window was given back"
        else:
            assert len(held[gi]) == len(req.pages[gi]), "a layer that sees every position lost a page"
    assert windowed
    engine.close(req)
    engine.cache.check()


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_slot_used_again_starts_from_zero(backend):
    """The recurrent state of a finished request must not leak into the one that gets its slot."""
    name = "Q"
    cfg = N.config_of(name)
    engine = engine_of(name, backend, "f32", max_requests=1)
    first, second = N.random_ids(cfg, 40, 1), N.random_ids(cfg, 25, 2)
    a = engine.open("a")
    engine.step([H.lab.StepEntry(a, first, [])])
    engine.close(a)
    b = engine.open("b")
    assert b.row == a.row
    out = engine.step([H.lab.StepEntry(b, second, list(range(len(second))))]).float().cpu()
    err = float((out.double() - N.plain_logits(name, 1, second)).abs().max())
    assert err < TOL["f32"], err
    engine.close(b)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["P", "Q"])
def test_the_first_tokens_of_a_sequence(backend, name):
    """Positions 0, 1, 2 one by one (an empty state, a window with one key, no history)."""
    cfg = N.config_of(name)
    ids = N.random_ids(cfg, 4, 8)
    want = N.plain_logits(name, 1, ids)
    engine = engine_of(name, backend, "f32")
    req = engine.open("x")
    for i, t in enumerate(ids):
        out = engine.step([H.lab.StepEntry(req, [t], [0])]).float().cpu()
        assert float((out[0].double() - want[i]).abs().max()) < TOL["f32"], i


@pytest.mark.parametrize("backend", BACKENDS)
def test_greedy_generation_through_the_scheduler(backend):
    """``Engine.generate``: the framework's own entry point, scheduler, sampler and cache, with
    fewer pages than all requests together would need."""
    name = "P"
    cfg = N.config_of(name)
    tensors = N.make_tensors(cfg, 1)
    prompts = [N.random_ids(cfg, n, 30 + n) for n in (5, 40, 17, 9)]
    engine = engine_of(name, backend, "f32", page_size=16, num_pages=12, max_requests=2, max_batch_tokens=32)
    results = engine.generate(prompts, max_new_tokens=8)
    for prompt, res in zip(prompts, results):
        ids = list(prompt)
        got = list(res.output_ids if hasattr(res, "output_ids") else res)
        assert len(got) == 8
        for n, token in enumerate(got):
            logits = plain_ninisun.forward(cfg.to_dict(), tensors, ids)[-1]
            best = int(logits.argmax())
            assert token == best or float(logits[best] - logits[token]) < 1e-4, (n, token, best)
            ids.append(token)
    engine.cache.check()
    assert engine.cache.metrics()["rows_used"] == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_decode_steps_replayed_from_a_graph(dtype):
    """Decode steps captured into a HIP graph and replayed, with the program's own eager steps
    (new requests' prompts) between the replays: every token the one an engine without graphs
    computes.  More requests than rows, so slots are reused between replays."""
    name = "P"
    cfg = N.config_of(name)
    prompts = [N.random_ids(cfg, n, 40 + n) for n in (7, 30, 12, 3)]
    runs = {}
    for graph in (False, True):
        engine = N.make_engine(name, 1, dtype, page_size=16, num_pages=40, max_requests=2, max_batch_tokens=32, graph=graph)
        runs[graph] = engine.generate(prompts, max_new_tokens=40)
        if graph:
            assert engine.metrics()["graphs"]["replays"] > 20
    assert runs[True] == runs[False]
