"""Minodra as data: configuration -> ``ModelSpec``.

A stack of pre-norm layers whose norms are RMS norms with a single number as their weight.  Every
sublayer reads its normed input through a short causal convolution over time (``h + conv(h)``) and
its result passes a sigmoid gate computed from the normed input before it joins the stream.  The
mixer is latent attention without positions: queries through a normed latent, keys and values
read out of one normed latent vector per token (the only thing cached), a learned extra term in
the softmax's denominator per head, one sigmoid gate per head.  The feed-forward is a gated one
(SiLU), a mixture of squared-ReLU experts behind a sigmoid router with a correction on the choice
and a gated shared expert, or absent.  The embedding adds a row of a hashed table of token pairs
to the scaled token vector and norms the sum; the logits pass a soft cap.

Tensor names: ``embed``, ``bigram``, ``embed.norm``, ``final.norm``, ``head``, and per layer
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.canon1``, ``l<i>.canon2``, ``l<i>.rg1``, ``l<i>.rg1.b``,
``l<i>.rg2``, ``l<i>.rg2.b``, ``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,sink,g,o}``,
``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,correction,e<j>.up,e<j>.down,shared.up,shared.down,shared.sg}``.
"""
from __future__ import annotations

from ..config.minodra import MinodraConfig
from ..config.registry import register_architecture
from ..config.spec import BlockSpec, ModelSpec, PartSpec, ScheduleEntry


def build_minodra_spec(cfg: MinodraConfig) -> ModelSpec:
    w = cfg.width
    norm = lambda name: PartSpec("rmsnorm", params=dict(size=w, eps=cfg.norm_eps, scalar=True), tensors=dict(weight=name))
    blocks = []
    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        m = p + "mix."
        mixer = PartSpec(
            "latent_attention",
            params=dict(hidden_size=w, num_heads=l.heads, head_dim=l.dim, value_dim=l.vdim, q_rank=l.q_rank,
                        kv_rank=l.kv_rank, scale=l.scale, norm_eps=cfg.norm_eps, sink=True, output_gate="sigmoid"),
            tensors=dict(dq_weight=m + "dq", dq_norm=m + "dq.norm", uq_weight=m + "uq", dkv_weight=m + "dkv",
                         dkv_norm=m + "dkv.norm", uk_weight=m + "uk", uv_weight=m + "uv", sink=m + "sink",
                         gate_weight=m + "g", o_weight=m + "o"))
        parts = dict(norm1=norm(p + "norm1"), mixer=mixer)
        f = l.mlp
        if f is not None and f.kind == "dense":
            parts.update(norm2=norm(p + "norm2"), feed_forward=PartSpec(
                "swiglu", params=dict(hidden_size=w, intermediate_size=f.ff, activation="silu"),
                tensors=dict(gate_weight=p + "mlp.gate", up_weight=p + "mlp.up", down_weight=p + "mlp.down")))
        elif f is not None:
            shared = None if f.shared_ff is None else PartSpec(
                "dense", params=dict(hidden_size=w, intermediate_size=f.shared_ff, activation="relu2"),
                tensors=dict(up_weight=p + "mlp.shared.up", down_weight=p + "mlp.shared.down"))
            tensors = dict(router=p + "mlp.router", correction=p + "mlp.correction", expert_up=p + "mlp.e{}.up",
                           expert_down=p + "mlp.e{}.down")
            if shared is not None:
                tensors["shared_gate"] = p + "mlp.shared.sg"
            parts.update(norm2=norm(p + "norm2"), feed_forward=PartSpec(
                "routed_experts",
                params=dict(hidden_size=w, expert_size=f.ff, num_experts=f.experts, top=f.top, correction=True,
                            scoring="sigmoid", expert_form="relu2", shared=shared, shared_gate=shared is not None),
                tensors=tensors))
        tensors = dict(conv1=p + "canon1", conv2=p + "canon2", gate1_weight=p + "rg1", gate1_bias=p + "rg1.b",
                       gate2_weight=p + "rg2", gate2_bias=p + "rg2.b")
        blocks.append(BlockSpec("gated_conv", parts=parts,
                                params=dict(hidden_size=w, conv_taps=cfg.canon_taps, residual_gate=True, tensors=tensors)))
    b = cfg.bigram
    embedding = PartSpec(
        "pair_hash_embedding",
        params=dict(vocab_size=cfg.vocab, hidden_size=w, scale=cfg.embedding_scale, buckets=b.buckets if b else 0,
                    mul_prev=b.mul_prev if b else 0, mul_cur=b.mul_cur if b else 0, norm=norm("embed.norm")),
        tensors=dict(weight="embed", pairs="bigram"))
    spec = ModelSpec(
        architecture=MinodraConfig.ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=w,
        max_positions=MinodraConfig.MAX_POSITIONS, embedding=embedding, blocks=tuple(blocks),
        schedule=tuple(ScheduleEntry(i) for i in range(len(blocks))), final_norm=norm("final.norm"),
        head=PartSpec("linear_head", params=dict(vocab_size=cfg.vocab, hidden_size=w, softcap=cfg.logit_softcap),
                      tensors=dict(weight="head")),
        eos_token_ids=tuple(cfg.eos_token_ids))
    spec.validate()
    return spec


register_architecture(MinodraConfig.ARCHITECTURE, MinodraConfig, build_minodra_spec, replace=True)
