"""Ninisun as data: configuration -> ``ModelSpec``.

A stack of layers with a norm before and behind each sublayer and a learned scale on the
normed result: ``x += ls1 * norm1b(mixer(norm1(x)))``, then (where the layer has one) ``x +=
ls2 * norm2b(feed_forward(norm2(x)))``, all RMS norms.  The mixer is grouped-query attention
(neighbouring channels turned by position, a sliding window that keeps the first positions,
values mixed with the first such layer's), or a pair of mixers on one input: attention with sigmoid
weights and a gate per head, and a recurrent state under a generalised delta rule.  The
feed-forward is gated with the tanh form of gelu.  The head is the embedding table behind a
last norm.

Tensor names: ``embed``, ``final.norm``, and per layer ``l<i>.norm1``, ``.norm1b``, ``.norm2``,
``.norm2b``, ``.ls1``, ``.ls2``, ``l<i>.mix.<role>`` (``l<i>.mix.left.<role>`` / ``.right.<role>`` in a
parallel layer), ``l<i>.mlp.gate`` / ``.up`` / ``.down``.
"""
from __future__ import annotations

import dataclasses

from ..config.ninisun import NinisunConfig
from ..config.registry import register_architecture
from ..config.spec import BlockSpec, ModelSpec, PartSpec, ScheduleEntry


def _position(a):
    if a.rot is None or not a.rot.dims:
        return None
    scaling = dataclasses.asdict(a.rot.scaling) if a.rot.scaling is not None else None
    return PartSpec("rope_pairs", params=dict(dim=a.dim, rotary_dim=a.rot.dims, theta=a.rot.base, scaling=scaling))


def build_ninisun_spec(cfg: NinisunConfig) -> ModelSpec:
    w = cfg.width
    norm = lambda name: PartSpec("rmsnorm", params=dict(size=w, eps=cfg.norm_eps), tensors=dict(weight=name))
    mixing = cfg.value_mix_layers()
    blocks = []
    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        if l.type == "attention":
            a = l.attention
            names = dict(q_weight=p + "mix.q", k_weight=p + "mix.k", v_weight=p + "mix.v", o_weight=p + "mix.o")
            mix = None
            if i in mixing:
                mix = "first" if i == mixing[0] else "mix"
                if mix == "mix":
                    names["value_mix"] = p + "mix.vmix"
            mixer = PartSpec(
                "windowed_sink_attention",
                params=dict(hidden_size=w, num_heads=a.heads, num_kv_heads=a.kv_heads, key_dim=a.dim, value_dim=a.vdim,
                            scale=a.scale, window=a.window, keep_first=a.keep_first, sink=False, qk_norm=None,
                            position=_position(a), value_mix=mix),
                tensors=names)
        else:
            a, r, q = l.left, l.right, p + "mix.left."
            left = PartSpec(
                "windowed_sink_attention",
                params=dict(hidden_size=w, num_heads=a.heads, num_kv_heads=a.kv_heads, key_dim=a.dim, value_dim=a.vdim,
                            scale=a.scale, window=None, keep_first=0, sink=False, qk_norm=None, position=_position(a),
                            qkv_bias=True, weights="sigmoid", score_bias=True, output_gate="sigmoid"),
                tensors=dict(q_weight=q + "q", k_weight=q + "k", v_weight=q + "v", o_weight=q + "o", q_bias=q + "q.b",
                             k_bias=q + "k.b", v_bias=q + "v.b", score_bias=q + "pb", gate_weight=q + "g"))
            q = p + "mix.right."
            right = PartSpec(
                "delta_rule_attention",
                params=dict(hidden_size=w, num_heads=r.heads, key_dim=r.dim, decay_rank=None, norm_eps=cfg.norm_eps,
                            gate="sigmoid"),
                tensors=dict(r_weight=q + "r", k_weight=q + "k", v_weight=q + "v", gate_weight=q + "g",
                             rate_weight=q + "a", rate_bias=q + "a.b", decay_down=q + "w1", decay_up=q + "w2",
                             decay_bias=q + "w0", out_norm=q + "norm", o_weight=q + "o"))
            mixer = PartSpec("parallel", params=dict(left=left, right=right, left_scale=l.left_scale,
                                                     right_scale=l.right_scale))
        parts = dict(norm1=norm(p + "norm1"), mixer=mixer, post_norm1=norm(p + "norm1b"))
        tensors = dict(scale1=p + "ls1")
        if l.mlp is not None:
            parts.update(
                norm2=norm(p + "norm2"), post_norm2=norm(p + "norm2b"),
                feed_forward=PartSpec("swiglu", params=dict(hidden_size=w, intermediate_size=l.mlp.ff,
                                                            activation="gelu_tanh"),
                                      tensors=dict(gate_weight=p + "mlp.gate", up_weight=p + "mlp.up",
                                                   down_weight=p + "mlp.down")))
            tensors["scale2"] = p + "ls2"
        blocks.append(BlockSpec("sandwich_norm", parts=parts, params=dict(hidden_size=w, tensors=tensors)))
    sizes = dict(vocab_size=cfg.vocab, hidden_size=w)
    spec = ModelSpec(
        architecture=NinisunConfig.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=w,
        max_positions=NinisunConfig.MAX_POSITIONS,
        embedding=PartSpec("token_embedding", params=sizes, tensors=dict(weight="embed")),
        blocks=tuple(blocks), schedule=tuple(ScheduleEntry(i) for i in range(len(blocks))),
        final_norm=norm("final.norm"), head=PartSpec("linear_head", params=sizes, tensors=dict(weight="embed")),
        eos_token_ids=tuple(cfg.eos_token_ids))
    spec.validate()
    return spec


def ninisun_random_init(cfg: NinisunConfig, expected, seed: int, dtype):
    """Random-weights mode: a size that the configuration leaves to the tensors' shapes takes
    the configuration class's default."""
    from ..weights.random_init import random_tensors
    rank = NinisunConfig.DEFAULT_DECAY_RANK
    filled = {name: dataclasses.replace(s, shape=tuple(rank if d is None else d for d in s.shape))
              for name, s in expected.items()}
    return random_tensors(filled, seed, dtype)


register_architecture(NinisunConfig.ARCHITECTURE, NinisunConfig, build_ninisun_spec, random_init=ninisun_random_init,
                      replace=True)
