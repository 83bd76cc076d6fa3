"""Ninisun configurations drawn at random (widths, head counts, key and value widths, the order
of the layers, which layers mix their values, windows and kept prefixes shorter and longer than
the sequences and the 16-token pages, how many channels turn and with which frequencies, states of
several sizes, the two weights of a parallel layer, feed-forwards present or not): mixed batches
through the engine against the plain implementation, float32 tight and bfloat16 by the root
mean square."""
import random

import pytest
import torch

import helpers as H
import ninisun_cases as N
import plain_ninisun
from emu_ops import EmuOps

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]


def draw_rotation(rng, dim):
    dims = rng.choice([0, 2, 4, dim // 2 // 2 * 2, dim // 2 * 2])
    if not dims:
        return None
    scaling = None
    if rng.random() < 0.5:
        scaling = (rng.choice([1.0, 2.0, 4.0, 16.0]), rng.choice([8, 64, 1024]), rng.choice([2.0, 8.0, 32.0]),
                   rng.choice([0.25, 1.0, 2.0]))
    return N.rot(dims, rng.choice([10.0, 1e4, 3e5, 2e6]), scaling)


def draw_config(seed):
    rng = random.Random(seed)
    width = rng.choice([32, 48, 64, 96, 128])
    layers = []
    mixed = None                 # (kv heads, value width) of the layers that mix their values
    for i in range(rng.randint(2, 6)):
        ff = rng.choice([None, 8 * rng.randint(2, 20)])
        if rng.random() < 0.35:
            kv = rng.choice([1, 2])
            heads = kv * rng.choice([1, 2, 4])
            dim, vdim = rng.choice([8, 16, 24, 32, 64, 96]), rng.choice([8, 16, 32, 48, 64, 192])
            while heads * vdim % 8:
                vdim += 8
            r_heads, r_dim = rng.choice([1, 2, 3, 6]), rng.choice([8, 16, 24, 32, 64])
            while r_heads * r_dim % 8:
                r_dim += 8
            layers.append(N.parallel((heads, kv, dim, vdim, rng.choice([0.1, 0.3, 1.0]), draw_rotation(rng, dim)),
                                     (r_heads, r_dim), rng.choice([0.2, 0.75, 1.0, 1.7]), rng.choice([0.3, 0.85, 1.0, 2.1]),
                                     ff=ff))
            continue
        mask = dict(size=rng.choice([1, 2, 5, 16, 17, 31, 44, 64, 500]), keep_first=rng.choice([0, 0, 1, 4, 7, 15, 16, 33]))
        v_mix = rng.random() < 0.6
        if v_mix and mixed is not None:
            kv, vdim = mixed
        else:
            kv, vdim = rng.choice([1, 2, 3]), rng.choice([8, 16, 32, 48, 64, 128])
        heads = kv * rng.choice([1, 2, 4, 7])
        while heads * vdim % 8:
            if v_mix and mixed is not None:
                heads += kv
            else:
                vdim += 8
        if v_mix and mixed is None:
            mixed = (kv, vdim)
        dim = rng.choice([8, 16, 32, 40, 64, 96, 128])
        layers.append(N.attention(heads, kv, dim, vdim, rng.choice([0.1, 0.5, 1.0]), draw_rotation(rng, dim), v_mix=v_mix,
                                  ff=ff, **(mask if rng.random() < 0.85 else {})))
    return dict(architecture="Ninisun", vocab=rng.choice([50, 131, 256]), width=width,
                norm=dict(eps=rng.choice([1e-6, 1e-5, 1e-3])), layers=layers)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("seed", range(16))
def test_drawn_configuration(backend, seed):
    raw = draw_config(seed)
    cfg = H.lab.NinisunConfig.from_dict(raw)
    tensors = N.make_tensors(cfg, seed)
    seqs = {f"r{i}": N.random_ids(cfg, n, 100 * seed + i) for i, n in enumerate([3, 45, 70, 20])}
    want = {rid: plain_ninisun.forward(cfg.to_dict(), tensors, ids) for rid, ids in seqs.items()}
    for dtype in ("f32", "bf16"):
        kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=16,
                              max_requests=3, max_batch_tokens=128, max_seq_len=128, **kw)
        got = H.run_trace(engine, seqs, H.steps_mixed(seqs, seed=seed, max_live=3, budget=64))
        diff = torch.cat([got[rid].double() - want[rid] for rid in got])
        assert not torch.isnan(diff).any()
        size = max(1.0, float(torch.cat(list(want.values())).std()))
        if dtype == "f32":
            bad = H.first_wrong(got, want, 2e-4 * size)
            assert bad is None, f"{raw}\nfirst wrong logits at (request, position, error) = {bad}"
        else:
            rms = float(diff.pow(2).mean().sqrt())
            assert rms < 0.06 * size, (raw, rms)
        engine.cache.check()
        assert engine.cache.metrics()["rows_used"] == 0


# Two configurations at the sizes of small real models: head sizes that the matrix-core attention
# kernels take (groups of 4 heads and of 3 share their keys), values twice as wide as keys on the
# left, states of 64 x 64 and 128 x 128 (scans in chunks), windows that cross the 64-token pages.
REAL = {
    "M": dict(architecture="Ninisun", vocab=1000, width=256, norm=dict(eps=1e-6), layers=[
        N.attention(8, 2, 64, 64, 0.125, N.rot(32, 1e4), size=100, keep_first=4, v_mix=True, ff=512),
        N.parallel((8, 2, 64, 128, 0.125, N.rot(16, 2e5, (6.0, 256, 16.0, 2.0))), (4, 64), 0.75, 1.25, ff=512),
        N.attention(8, 2, 64, 64, 0.125, N.rot(32, 1e4), size=100, keep_first=4, v_mix=True, ff=512),
    ]),
    "N": dict(architecture="Ninisun", vocab=777, width=384, norm=dict(eps=1e-5), layers=[
        N.parallel((6, 2, 128, 128, 0.09, N.rot(64, 1e4)), (2, 128), 1.1, 0.6, ff=576),
        N.attention(6, 6, 32, 96, 0.18, N.rot(32, 1e4, (2.0, 128, 8.0, 0.5)), size=70, keep_first=0, v_mix=True),
        N.attention(12, 6, 96, 96, 0.1, N.rot(8, 1e6), v_mix=True, ff=200),
    ]),
}


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(REAL))
def test_sizes_of_small_real_models(name):
    cfg = H.lab.NinisunConfig.from_dict(REAL[name])
    tensors = N.make_tensors(cfg, 3)
    for t in tensors:                       # (wider rows: products of order one again)
        if tensors[t].dim() == 2 and t != "embed" and not t.endswith((".w1", ".w2")):
            tensors[t] = (tensors[t].float() * 0.5).to(torch.bfloat16)
    seqs = {f"r{i}": N.random_ids(cfg, n, 50 + i) for i, n in enumerate([260, 45, 130, 200])}
    want = {rid: plain_ninisun.forward(cfg.to_dict(), tensors, ids) for rid, ids in seqs.items()}
    size = max(1.0, float(torch.cat(list(want.values())).std()))
    for dtype in ("f32", "bf16"):
        for cut in (H.steps_prefill_then_decode, lambda s: H.steps_mixed(s, seed=1, max_live=3, budget=192)):
            engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=64, num_pages=20,
                                  max_requests=3, max_batch_tokens=384, max_seq_len=384)
            got = H.run_trace(engine, seqs, cut(seqs))
            diff = torch.cat([got[rid].double() - want[rid] for rid in got])
            assert not torch.isnan(diff).any()
            if dtype == "f32":
                bad = H.first_wrong(got, want, 5e-4 * size)
                assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
            else:
                rms = float(diff.pow(2).mean().sqrt())
                assert rms < 0.06 * size, rms
            engine.cache.check()


def test_configuration_round_trip_and_errors():
    """``to_dict`` gives back what ``from_dict`` read; what cannot be a model of this design is refused
    with the place named."""
    from llm_inference_lab_amd.config import ConfigError
    for seed in range(8):
        raw = draw_config(seed)
        cfg = H.lab.NinisunConfig.from_dict(raw)
        assert H.lab.NinisunConfig.from_dict(cfg.to_dict()) == cfg
    good = draw_config(1)
    for breaker, needle in [
        (lambda r: r["layers"].append(dict(type="other", mixer={}, mlp=None)), "unknown layer type"),
        (lambda r: r.pop("norm"), "norm"),
        (lambda r: r["layers"][0]["mixer"].update(heads=0) if "heads" in r["layers"][0]["mixer"]
         else r["layers"][0]["mixer"]["left"].update(heads=0), "positive"),
    ]:
        import copy
        bad = copy.deepcopy(good)
        breaker(bad)
        with pytest.raises(ConfigError) as err:
            H.lab.NinisunConfig.from_dict(bad)
        assert needle in str(err.value)
    # two layers that mix their values must agree on what a token's values are
    bad = dict(architecture="Ninisun", vocab=50, width=32, norm=dict(eps=1e-5), layers=[
        N.attention(2, 1, 16, 16, 0.5, N.rot(4, 100.0), v_mix=True), N.attention(2, 2, 16, 16, 0.5, N.rot(4, 100.0), v_mix=True)])
    with pytest.raises(ConfigError):
        H.lab.NinisunConfig.from_dict(bad)
