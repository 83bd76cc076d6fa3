"""A plain, slow implementation of the Ninisun decoder, one function per mechanism, in
float64 on the CPU.  It shares no code with the engine: tensors come as a dictionary by
file name, the configuration as the dictionary of ``config.json``.

Notation: ``h [T, W]`` the rows of one sequence at positions ``0 .. T-1``; ``H`` query
heads, ``G`` key/value heads, ``D`` the width of a query or key head, ``E`` of a value head.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gated_gelu_mlp(h, gate, up, down):
    return (gelu_tanh(h @ gate.T) * (h @ up.T)) @ down.T


# ------------------------------------------------------------------ rotation
def rotary_frequencies(rot):
    """``(f [dims/2], magnitude)``: ``f_i = base^(-2i/dims)``; with ``scaling`` the slow
    frequencies are divided by ``factor`` through a ramp over the pair index, and the sines
    and cosines are multiplied by ``0.1 ln(factor) + 1``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn_to_dim(t):
        return dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_to_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_to_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, rot):
    """``x [T, heads, D]``: channels ``2i`` and ``2i + 1`` (``i < dims/2``) of every head turn
    by ``position * f_i``; the channels from ``dims`` on pass unchanged."""
    f, mag = rotary_frequencies(rot)
    dims = int(rot["dims"])
    ang = torch.tensor(list(positions), dtype=F).unsqueeze(-1) * f            # [T, dims/2]
    cos, sin = (torch.cos(ang) * mag).unsqueeze(1), (torch.sin(ang) * mag).unsqueeze(1)
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ----------------------------------------------------------------- attention
def visible(i, j, size, keep_first):
    """Whether the query at position ``i`` sees the key at position ``j`` (``size`` None: no window)."""
    return j <= i and (size is None or i - j < size or j < keep_first)


def softmax_attention(q, k, v, scale, size=None, keep_first=0, q_positions=None):
    """``q [T, H, D]``, ``k [S, G, D]``, ``v [S, G, E]``; softmax over the visible keys."""
    T, H, _ = q.shape
    S, G, E = v.shape
    if q_positions is None:
        q_positions = list(range(S - T, S))
    out = torch.zeros(T, H, E, dtype=q.dtype)
    every = torch.arange(S)
    for t, i in enumerate(q_positions):
        # (the keys that ``visible`` admits, all at once)
        js = every[(every <= i) & ((i - every < (size if size is not None else S + 1)) | (every < keep_first))]
        for hd in range(H):
            g = hd // (H // G)
            s = (k[js, g] @ q[t, hd]) * scale
            p = torch.exp(s - s.max())
            out[t, hd] = (p / p.sum()) @ v[js, g]
    return out


def sigmoid_attention(q, k, v, scale, bias, q_positions=None):
    """Causal; the weight of a visible key is ``sigmoid(score + bias_h)``, not normalised."""
    T, H, _ = q.shape
    S, G, E = v.shape
    if q_positions is None:
        q_positions = list(range(S - T, S))
    out = torch.zeros(T, H, E, dtype=q.dtype)
    for t, i in enumerate(q_positions):
        for hd in range(H):
            g = hd // (H // G)
            s = (k[:i + 1, g] @ q[t, hd]) * scale + bias[hd]
            out[t, hd] = torch.sigmoid(s) @ v[:i + 1, g]
    return out


def windowed_mixer(h, p, m, v_first=None):
    """The 'attention' mixer.  Returns (output, the values it cached [T, G, E])."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ p["q"].T).view(T, H, D)
    k = (h @ p["k"].T).view(T, G, D)
    v = (h @ p["v"].T).view(T, G, E)
    if m.get("rot"):
        q, k = rotate_pairs(q, range(T), m["rot"]), rotate_pairs(k, range(T), m["rot"])
    if v_first is not None:
        lam = p["vmix"]
        v = (1.0 - lam) * v + lam * v_first
    mask = m.get("mask") or {}
    o = softmax_attention(q, k, v, m["scale"], mask.get("size"), mask.get("keep_first", 0))
    return o.reshape(T, H * E) @ p["o"].T, v


def gated_sigmoid_mixer(h, p, m):
    """The left half of the 'parallel' mixer."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ p["q"].T + p["q.b"]).view(T, H, D)
    k = (h @ p["k"].T + p["k.b"]).view(T, G, D)
    v = (h @ p["v"].T + p["v.b"]).view(T, G, E)
    if m.get("rot"):
        q, k = rotate_pairs(q, range(T), m["rot"]), rotate_pairs(k, range(T), m["rot"])
    o = sigmoid_attention(q, k, v, m["scale"], p["pb"])
    o = o * torch.sigmoid(h @ p["g"].T).unsqueeze(-1)
    return o.reshape(T, H * E) @ p["o"].T


# ---------------------------------------------------------------- delta rule
def delta_rule(r, k, v, w, a, state=None):
    """``r, k, v, w, a [T, H, D]``.  Per head, with the unit key ``u = k / sqrt(|k|^2 + 1e-6)``::

        S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T ;  o_t = S_t^T r_t

    Returns ``o [T, H, D]`` and the last state ``[H, D, D]``."""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=r.dtype) if state is None else state.clone()
    out = torch.zeros(T, H, D, dtype=r.dtype)
    for t in range(T):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + 1e-6)
        uS = torch.einsum("hd,hde->he", u, S)
        S = w[t].unsqueeze(-1) * S - (a[t] * u).unsqueeze(-1) * uS.unsqueeze(-2) + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = torch.einsum("hde,hd->he", S, r[t])
    return out, S


def delta_mixer(h, p, m, eps, state=None):
    """The right half of the 'parallel' mixer.  Returns (output, last state)."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ p["r"].T).view(T, H, D)
    k = (h @ p["k"].T).view(T, H, D)
    v = (h @ p["v"].T).view(T, H, D)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ p["w1"].T) @ p["w2"].T + p["w0"])).view(T, H, D)
    a = torch.sigmoid(h @ p["a"].T + p["a.b"]).view(T, H, D)
    o, S = delta_rule(r, k, v, w, a, state)
    o = unit_rms(o, eps).reshape(T, H * D) * p["norm"] * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T, S


# --------------------------------------------------------------------- model
def sub(tensors, prefix):
    return {n[len(prefix):]: t for n, t in tensors.items() if n.startswith(prefix)}


def forward(config, tensors, tokens, return_layers=False):
    """Logits ``[T, vocab]`` of one sequence (and the stream after every layer)."""
    t = {n: x.to(F) for n, x in tensors.items()}
    eps = float(config["norm"]["eps"])
    x = t["embed"][torch.tensor(list(tokens))]
    v_first = None
    after = []
    for i, layer in enumerate(config["layers"]):
        p = sub(t, f"l{i}.")
        m = layer["mixer"]
        h = rms_norm(x, p["norm1"], eps)
        if layer["type"] == "attention":
            mixing = bool(m.get("v_mix"))
            y, v = windowed_mixer(h, sub(p, "mix."), m, v_first if mixing else None)
            if mixing and v_first is None:
                v_first = v
        elif layer["type"] == "parallel":
            y = (m["left_scale"] * gated_sigmoid_mixer(h, sub(p, "mix.left."), m["left"])
                 + m["right_scale"] * delta_mixer(h, sub(p, "mix.right."), m["right"], eps)[0])
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, p["norm1b"], eps) * p["ls1"]
        if layer.get("mlp") is not None:
            h = rms_norm(x, p["norm2"], eps)
            y = gated_gelu_mlp(h, p["mlp.gate"], p["mlp.up"], p["mlp.down"])
            x = x + rms_norm(y, p["norm2b"], eps) * p["ls2"]
        after.append(x)
    logits = rms_norm(x, t["final.norm"], eps) @ t["embed"].T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy(config, tensors, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(forward(config, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
