"""A plain, slow Minodra in float64: whole sequences, one function per mechanism, no cache.

The oracle of the Minodra tests.  It shares nothing with the engine: it takes the raw
``config.json`` dictionary and the tensors by their file names, and computes every position of a
sequence from the sequence's start.

    x_0      = norm_s(embed[t] * scale + bigram[row(t_prev, t)], g_embed)
    per layer: h = norm_s(x, g1);  x += mixer(h + conv1(h)) * sigmoid(R1 h + b1)
               h = norm_s(x, g2);  x += ff(h + conv2(h))    * sigmoid(R2 h + b2)
    logits   = cap * tanh(head . norm_s(x, g_final) / cap)

``norm_s`` is the RMS norm with a single number as its weight.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    """``x / sqrt(mean(x^2) + eps)`` over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    return rms(x, eps) * g.to(F64).reshape(())


def vector_norm(x, w, eps):
    return rms(x, eps) * w.to(F64)


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """The bigram table's row for every position: the first token of a sequence takes the row
    behind the buckets."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((int(prev) * mul_prev + int(cur) * mul_cur) % buckets)
    return rows


def embed(tokens, cfg, w):
    e = cfg["embedding"]
    x = w["embed"].to(F64)[list(tokens)] * float(e.get("scale", 1.0))
    b = e.get("bigram")
    if b:
        x = x + w["bigram"].to(F64)[bigram_rows(list(tokens), b["buckets"], b["mul_prev"], b["mul_cur"])]
    return scalar_norm(x, w["embed.norm"], cfg["norm"]["eps"])


def causal_conv(h, taps_weight):
    """``out_t = sum_j w[:, j] h_(t - taps + 1 + j)``, nothing before the sequence's start."""
    n, _ = h.shape
    wt = taps_weight.to(F64)
    taps = wt.shape[1]
    out = torch.zeros_like(h)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += wt[:, j] * h[s]
    return out


def residual_gate(h, weight, bias):
    return torch.sigmoid(h @ weight.to(F64).T + bias.to(F64))


def latent_attention(h, m, w, p, eps):
    """``h [n, width]`` -> ``[n, width]``; ``m``: the mixer's sizes, ``p``: the tensors' prefix."""
    n = h.shape[0]
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    cq = vector_norm(h @ w[p + "dq"].to(F64).T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].to(F64).T).view(n, heads, dim)
    c = vector_norm(h @ w[p + "dkv"].to(F64).T, w[p + "dkv.norm"], eps)
    k = (c @ w[p + "uk"].to(F64).T).view(n, heads, dim)
    v = (c @ w[p + "uv"].to(F64).T).view(n, heads, vdim)
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).T)           # [n, heads]
    sink = w[p + "sink"].to(F64)
    out = torch.zeros(n, heads, vdim, dtype=F64)
    for i in range(n):
        for a in range(heads):
            s = (k[: i + 1, a] @ q[i, a]) * float(m["scale"])
            top = max(float(s.max()), float(sink[a]))
            e = torch.exp(s - top)
            den = e.sum() + math.exp(float(sink[a]) - top)
            out[i, a] = (e / den) @ v[: i + 1, a]
    out = out * gate[:, :, None]
    return out.reshape(n, heads * vdim) @ w[p + "o"].to(F64).T


def gated_ff(h, w, p):
    z = h @ w[p + "gate"].to(F64).T
    return (z * torch.sigmoid(z) * (h @ w[p + "up"].to(F64).T)) @ w[p + "down"].to(F64).T


def relu2_ff(h, w, p):
    z = torch.relu(h @ w[p + "up"].to(F64).T)
    return (z * z) @ w[p + "down"].to(F64).T


def route(h, w, p, top):
    """Chosen experts and their weights per row: sigmoid scores, the choice on score + correction
    (ties: the smaller index), the weights the scores themselves."""
    s = torch.sigmoid(h @ w[p + "router"].to(F64).T)
    choice = s + w[p + "correction"].to(F64) if (p + "correction") in w else s
    chosen = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
    return chosen, torch.gather(s, 1, chosen)


def mixture(h, mlp, w, p):
    chosen, weights = route(h, w, p, mlp["router"]["top"])
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for e, s in zip(chosen[r].tolist(), weights[r]):
            out[r] += s * relu2_ff(h[r:r + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + relu2_ff(h, w, p + "shared.") * torch.sigmoid(h @ w[p + "shared.sg"].to(F64).T)
    return out


def feed_forward(h, mlp, w, p):
    if mlp["kind"] == "dense":
        return gated_ff(h, w, p)
    if mlp["kind"] == "moe":
        return mixture(h, mlp, w, p)
    raise ValueError(mlp["kind"])


def layer(x, i, cfg, w):
    spec, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    canon = bool(cfg.get("canon"))
    if spec["type"] != "latent_attention":
        raise ValueError(spec["type"])
    h = scalar_norm(x, w[p + "norm1"], eps)
    hin = h + causal_conv(h, w[p + "canon1"]) if canon else h
    x = x + latent_attention(hin, spec["mixer"], w, p + "mix.", eps) * residual_gate(h, w[p + "rg1"], w[p + "rg1.b"])
    if spec.get("mlp"):
        h = scalar_norm(x, w[p + "norm2"], eps)
        hin = h + causal_conv(h, w[p + "canon2"]) if canon else h
        x = x + feed_forward(hin, spec["mlp"], w, p + "mlp.") * residual_gate(h, w[p + "rg2"], w[p + "rg2.b"])
    return x


def forward(tokens, cfg, w, layers_out=None):
    """Logits ``[n, vocab]`` of a whole sequence; ``layers_out``: a list that receives the stream
    after every layer."""
    x = embed(tokens, cfg, w)
    for i in range(len(cfg["layers"])):
        x = layer(x, i, cfg, w)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = scalar_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].to(F64).T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


def greedy(tokens, cfg, w, count):
    out = list(tokens)
    for _ in range(count):
        out.append(int(forward(out, cfg, w)[-1].argmax()))
    return out[len(tokens):]
