"""Typed configuration of the Minodra decoder, read from ``config.json``.

The file lists the layers one by one (``layers``: ``type``, the mixer's sizes and constants in
``mixer``, the feed-forward in ``mlp`` or null for a layer with the mixer only).  Beside them:
``embedding`` (the scale of the token vectors and the hashed table of token pairs), ``canon`` (the
taps of the short convolution in front of every sublayer), ``norm.eps`` and ``logit_softcap``.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .qwen2 import _require, _typed


def _object(raw, key: str, at: str, required: bool = True):
    value = raw.get(key)
    if value is None and not required:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"{at}: key '{key}' must be an object")
    return value


@dataclasses.dataclass(frozen=True)
class MinodraFeedForward:
    """``kind`` "dense": one gated feed-forward ``ff`` wide.  ``kind`` "moe": ``experts`` experts
    ``ff`` wide of which a token takes ``top``, and a shared expert ``shared_ff`` wide (None: none)."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class MinodraLayer:
    """A latent attention layer: ``heads`` heads of ``dim`` query/key channels and ``vdim`` value
    channels, queries through a latent of ``q_rank``, keys and values out of one of ``kv_rank``."""

    type: str
    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    mlp: Optional[MinodraFeedForward] = None


@dataclasses.dataclass(frozen=True)
class MinodraBigram:
    buckets: int
    mul_prev: int
    mul_cur: int


def _feed_forward(mlp, at: str) -> Optional[MinodraFeedForward]:
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise ConfigError(f"{at}: 'mlp' is an object or null")
    kind = _require(mlp, "kind", str, at)
    if kind == "dense":
        return MinodraFeedForward("dense", _require(mlp, "ff", int, at))
    if kind != "moe":
        raise ConfigError(f"{at}: unknown feed-forward kind '{kind}' (known: dense, moe)")
    r = _object(mlp, "router", at)
    shared = _object(mlp, "shared", at, required=False)
    return MinodraFeedForward("moe", _require(_object(mlp, "expert", at), "ff", int, at + ".expert"),
                              experts=_require(r, "experts", int, at + ".router"),
                              top=_require(r, "top", int, at + ".router"),
                              shared_ff=None if shared is None else _require(shared, "ff", int, at + ".shared"))


@dataclasses.dataclass(frozen=True)
class MinodraConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[MinodraLayer, ...]
    embedding_scale: float = 1.0
    bigram: Optional[MinodraBigram] = None
    canon_taps: int = 0                      # 0: no convolution in front of the sublayers
    logit_softcap: Optional[float] = None
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Minodra"

    ARCHITECTURE = "Minodra"
    MAX_POSITIONS = 1 << 20          # the design has no position table: the engine's own bound

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "MinodraConfig":
        name = raw.get("architecture", (raw.get("architectures") or [cls.ARCHITECTURE])[0])
        if name != cls.ARCHITECTURE:
            raise ConfigError(f"{where}: architecture must be '{cls.ARCHITECTURE}', got {name!r}")
        norm = _object(raw, "norm", where)
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{where}: key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(listed):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{at} must be an object with 'type' and 'mixer'")
            kind, m = _require(entry, "type", str, at), _object(entry, "mixer", at)
            if kind != "latent_attention":
                raise ConfigError(f"{at}: unknown layer type '{kind}' (known: latent_attention)")
            dim = _require(m, "dim", int, at)
            layers.append(MinodraLayer(
                type=kind, heads=_require(m, "heads", int, at), dim=dim,
                vdim=_typed(m.get("vdim", dim), "vdim", int, at), q_rank=_require(m, "q_rank", int, at),
                kv_rank=_require(m, "kv_rank", int, at), scale=_require(m, "scale", float, at),
                mlp=_feed_forward(entry.get("mlp"), at + ".mlp")))
        emb = _object(raw, "embedding", where, required=False) or {}
        big = _object(emb, "bigram", where + ": embedding", required=False)
        if big is not None:
            big = MinodraBigram(*(_require(big, k, int, where + ": embedding.bigram")
                                  for k in ("buckets", "mul_prev", "mul_cur")))
        canon = _object(raw, "canon", where, required=False)
        cap = raw.get("logit_softcap")
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where)
                                               for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(norm, "eps", float, where + ": norm"), layers=tuple(layers),
                  embedding_scale=_typed(emb.get("scale", 1.0), "scale", float, where + ": embedding"),
                  bigram=big, canon_taps=0 if canon is None else _require(canon, "taps", int, where + ": canon"),
                  logit_softcap=None if cap is None else _typed(cap, "logit_softcap", float, where),
                  eos_token_ids=eos_ids)
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"{where}: 'vocab' and 'width' must be positive")
        if not (math.isfinite(self.norm_eps) and self.norm_eps > 0):
            raise ConfigError(f"{where}: norm.eps must be finite and > 0, got {self.norm_eps}")
        if not math.isfinite(self.embedding_scale):
            raise ConfigError(f"{where}: embedding.scale must be finite")
        if self.bigram is not None and (self.bigram.buckets <= 0 or self.bigram.mul_prev < 0 or self.bigram.mul_cur < 0):
            raise ConfigError(f"{where}: embedding.bigram needs buckets > 0 and multipliers >= 0")
        if self.canon_taps < 0 or self.canon_taps > 64:
            raise ConfigError(f"{where}: canon.taps must lie in 1 .. 64, got {self.canon_taps}")
        if self.logit_softcap is not None and not (math.isfinite(self.logit_softcap) and self.logit_softcap > 0):
            raise ConfigError(f"{where}: logit_softcap must be finite and > 0, got {self.logit_softcap}")
        for i, l in enumerate(self.layers):
            at = f"{where}: layers[{i}]"
            if min(l.heads, l.dim, l.vdim, l.q_rank, l.kv_rank) <= 0:
                raise ConfigError(f"{at}: heads, dim, vdim, q_rank and kv_rank must be positive")
            if not (math.isfinite(l.scale) and l.scale > 0):
                raise ConfigError(f"{at}: scale must be finite and > 0, got {l.scale}")
            f = l.mlp
            if f is None:
                continue
            if f.ff <= 0 or (f.shared_ff is not None and f.shared_ff <= 0):
                raise ConfigError(f"{at}: feed-forward widths must be positive")
            if f.kind == "moe" and not 0 < f.top <= f.experts:
                raise ConfigError(f"{at}: a router of {f.experts} experts cannot take the top {f.top}")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"{where}: eos_token_id {e} is outside the vocabulary")

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            mixer = dict(dim=l.dim, heads=l.heads, kv_rank=l.kv_rank, q_rank=l.q_rank, scale=l.scale, vdim=l.vdim)
            f, mlp = l.mlp, None
            if f is not None and f.kind == "dense":
                mlp = dict(ff=f.ff, kind="dense")
            elif f is not None:
                mlp = dict(expert=dict(ff=f.ff), kind="moe", router=dict(experts=f.experts, top=f.top))
                if f.shared_ff is not None:
                    mlp["shared"] = dict(ff=f.shared_ff)
            layers.append(dict(type=l.type, mixer=mixer, mlp=mlp))
        emb: Dict[str, Any] = dict(scale=self.embedding_scale)
        if self.bigram is not None:
            emb["bigram"] = dict(buckets=self.bigram.buckets, mul_cur=self.bigram.mul_cur, mul_prev=self.bigram.mul_prev)
        out: Dict[str, Any] = dict(architecture=self.architecture, embedding=emb, layers=layers,
                                   norm=dict(eps=self.norm_eps), vocab=self.vocab, width=self.width)
        if self.canon_taps:
            out["canon"] = dict(taps=self.canon_taps)
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
