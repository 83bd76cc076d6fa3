"""Minodra configurations drawn at random (widths, head counts and key / value sizes beside the
multiples of 16, latents narrower and wider than a head, beside the multiples of 32 and up to 520, one to
twelve taps, pair tables of one bucket to thousands or none, with and without a soft cap, dense feed-forwards,
mixtures with every expert chosen or one, with and without a shared expert, layers without a
feed-forward): mixed batches through the engine against the plain implementation, float32 tight and
bfloat16 position by position."""
import random

import pytest
import torch

import helpers as H
import minodra_cases as M
from emu_ops import EmuOps

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]


def draw_mlp(rng):
    kind = rng.choice(["none", "dense", "moe", "moe"])
    if kind == "none":
        return None
    if kind == "dense":
        return M.dense(rng.choice([8 * rng.randint(2, 20), 20, 36, 100]))
    experts = rng.choice([1, 2, 3, 5, 8, 12])
    return M.moe(rng.choice([8 * rng.randint(1, 6), 12, 20]), experts, rng.randint(1, min(experts, 4)),
                 shared=rng.choice([None, 8 * rng.randint(1, 8), 28]))


def draw_config(seed):
    rng = random.Random(1000 + seed)
    layers = []
    for _ in range(rng.randint(1, 4)):
        layers.append(M.latent(rng.choice([1, 2, 3, 5, 8]), rng.choice([8, 16, 24, 32, 40, 64]),
                               rng.choice([8, 16, 24, 48, 64]), rng.choice([8, 12, 24, 64, 100]),
                               rng.choice([8, 20, 32, 33, 64, 96, 128, 136, 200, 300, 520]), rng.choice([0.05, 0.2, 0.5, 1.0]),
                               mlp=draw_mlp(rng)))
    raw = dict(architecture="Minodra", vocab=rng.choice([50, 131, 256]), width=rng.choice([32, 48, 64, 96, 128]),
               norm=dict(eps=rng.choice([1e-6, 1e-5, 1e-3])), canon=dict(taps=rng.choice([1, 2, 3, 4, 4, 5, 8, 9, 12])),
               embedding=dict(scale=rng.choice([0.5, 1.0, 9.0])), layers=layers)
    if rng.random() < 0.75:
        raw["embedding"]["bigram"] = dict(buckets=rng.choice([1, 2, 61, 1019, 4093]), mul_prev=rng.choice([1, 113, 65537]),
                                          mul_cur=rng.choice([1, 11, 31]))
    if rng.random() < 0.6:
        raw["logit_softcap"] = rng.choice([2.0, 10.0, 25.0])
    return raw


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("seed", range(12))
def test_drawn_configuration(backend, seed):
    raw = draw_config(seed)
    cfg = H.lab.MinodraConfig.from_dict(raw)
    tensors = M.make_tensors(cfg, seed)
    seqs = {f"r{i}": M.random_ids(cfg, n, 100 * seed + i) for i, n in enumerate([3, 45, 70, 20])}
    want = {rid: M.plain_of(cfg.to_dict(), tensors, ids) for rid, ids in seqs.items()}
    for dtype in ("f32", "bf16"):
        kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=40,
                              max_requests=3, max_batch_tokens=128, max_seq_len=128, **kw)
        got = H.run_trace(engine, seqs, H.steps_mixed(seqs, seed=seed, max_live=3, budget=64))
        diff = torch.cat([got[rid].double() - want[rid] for rid in got])
        assert not torch.isnan(diff).any()
        size = max(1.0, float(torch.cat(list(want.values())).std()))
        if dtype == "f32":
            bad = H.first_wrong(got, want, 2e-4 * size)
            assert bad is None, f"{raw}\nfirst wrong logits at (request, position, error) = {bad}"
        else:
            # (a rounding may turn a router's close call at a few positions: see the 32-bit run)
            per_position = diff.pow(2).mean(-1).sqrt()
            assert float(per_position.median()) < 0.05 * size, (raw, float(per_position.median()))
            assert int((per_position > 0.2 * size).sum()) <= max(1, per_position.numel() // 20), raw
        engine.cache.check()
        assert engine.cache.metrics()["rows_used"] == 0


# Two configurations at the sizes of small real models (hundreds of channels, latents of the
# matrix-core attention kernels' widths, dozens of experts), with sequences of hundreds of tokens
# over pages of 64.
LARGER = {
    "X": dict(architecture="Minodra", vocab=701, width=384, norm=dict(eps=1e-6), canon=dict(taps=4),
              embedding=dict(scale=9.0, bigram=dict(buckets=4093, mul_prev=113, mul_cur=11)), logit_softcap=25.0,
              layers=[M.latent(6, 64, 64, 192, 128, 0.125, mlp=M.dense(1024)),
                      M.latent(12, 32, 48, 96, 256, 0.18, mlp=M.moe(96, 24, 6, shared=136)),
                      M.latent(3, 128, 64, 160, 64, 0.09, mlp=M.moe(104, 70, 3))]),
    "Y": dict(architecture="Minodra", vocab=330, width=192, norm=dict(eps=1e-5), canon=dict(taps=3),
              embedding=dict(scale=4.0), 
              layers=[M.latent(2, 112, 112, 64, 160, 0.1, mlp=M.dense(512)),
                      M.latent(16, 16, 16, 128, 96, 0.25, mlp=M.moe(32, 62, 5, shared=64)),
                      M.latent(4, 48, 80, 40, 224, 0.15, mlp=None)]),
}


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(LARGER))
def test_sizes_of_small_real_models(name):
    raw = LARGER[name]
    cfg = H.lab.MinodraConfig.from_dict(raw)
    tensors = M.make_tensors(cfg, 11)
    seqs = {f"r{i}": M.random_ids(cfg, n, 50 + i) for i, n in enumerate([420, 97, 333, 1])}
    want = {rid: M.plain_of(cfg.to_dict(), tensors, ids) for rid, ids in seqs.items()}
    size = max(1.0, float(torch.cat(list(want.values())).std()))
    for dtype in ("f32", "bf16"):
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=64, num_pages=16,
                              max_requests=3, max_batch_tokens=512, max_seq_len=512)
        for steps in (H.steps_prefill_then_decode(seqs, tail=40), H.steps_mixed(seqs, seed=1, max_live=3, budget=150)):
            got = H.run_trace(engine, seqs, steps)
            diff = torch.cat([got[rid].double() - want[rid] for rid in got])
            assert not torch.isnan(diff).any()
            if dtype == "f32":
                bad = H.first_wrong(got, want, 3e-4 * size)
                assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
            else:
                per_position = diff.pow(2).mean(-1).sqrt()
                assert float(per_position.median()) < 0.05 * size
                assert int((per_position > 0.2 * size).sum()) <= per_position.numel() // 20
            engine.cache.check()
            assert engine.cache.metrics()["rows_used"] == 0
