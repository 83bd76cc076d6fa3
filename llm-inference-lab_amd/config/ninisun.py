"""Typed configuration of the Ninisun decoder, read from ``config.json``.

The file lists the layers one by one: each has a ``type`` (which mixer it has), the mixer's sizes
and constants (``mixer``), and its feed-forward (``mlp``, or null for a layer with the mixer
only).  ``attention``: grouped-query attention with a rotation of neighbouring channels, a
sliding window that keeps a sequence's first positions, and values that may be mixed with those
of the first such layer.  ``parallel``: a pair of mixers on one input, a ``left`` one (attention with
sigmoid weights, biases, a rotation with stretched frequencies and a gate per head) and a
``right`` one (a recurrent state under a generalised delta rule), summed with two fixed weights.
Sizes that the file does not name (the rank of the decay projection) are read off the tensors'
shapes when the weights are loaded.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .qwen2 import _require, _typed


@dataclasses.dataclass(frozen=True)
class NinisunFeedForward:
    kind: str
    ff: int


@dataclasses.dataclass(frozen=True)
class NinisunScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclasses.dataclass(frozen=True)
class NinisunRotation:
    dims: int
    base: float
    scaling: Optional[NinisunScaling] = None

    @classmethod
    def from_dict(cls, raw, at: str) -> Optional["NinisunRotation"]:
        if raw is None:
            return None
        if not isinstance(raw, dict):
            raise ConfigError(f"{at}: 'rot' is an object")
        sc = raw.get("scaling")
        if sc is not None:
            if not isinstance(sc, dict):
                raise ConfigError(f"{at}: 'rot.scaling' is an object")
            sc = NinisunScaling(*(_require(sc, k, float, at + ".rot.scaling") for k in ("factor", "original", "fast", "slow")))
        return cls(_require(raw, "dims", int, at + ".rot"), _require(raw, "base", float, at + ".rot"), sc)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = dict(base=self.base, dims=self.dims)
        if self.scaling is not None:
            out["scaling"] = dataclasses.asdict(self.scaling)
        return out

    def check(self, dim: int, at: str) -> None:
        if self.dims < 0 or self.dims % 2 or self.dims > dim:
            raise ConfigError(f"{at}: rot.dims {self.dims} must be even and at most the head's {dim} channels")
        if not (math.isfinite(self.base) and self.base > 0.0):
            raise ConfigError(f"{at}: rot.base must be finite and > 0, got {self.base}")
        s = self.scaling
        if s is not None and not (s.factor > 0 and s.original > 0 and s.fast > 0 and s.slow > 0 and self.base != 1.0):
            raise ConfigError(f"{at}: rot.scaling needs positive factor, original, fast and slow (and a base other "
                              f"than 1), got {s}")


@dataclasses.dataclass(frozen=True)
class NinisunAttention:
    """Sizes of an attention mixer: the ``attention`` layer's own, or the ``left`` half of a
    ``parallel`` one (which has no window, no kept prefix and no value mixing)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[NinisunRotation] = None
    window: Optional[int] = None
    keep_first: int = 0
    v_mix: bool = False

    @classmethod
    def from_dict(cls, m, at: str, masked: bool) -> "NinisunAttention":
        if not isinstance(m, dict):
            raise ConfigError(f"{at} must be an object")
        heads = _require(m, "heads", int, at)
        kv_heads = m.get("kv_heads")
        mask = (m.get("mask") or {}) if masked else {}
        if not isinstance(mask, dict):
            raise ConfigError(f"{at}: 'mask' is an object")
        window = mask.get("size")
        return cls(heads=heads, kv_heads=heads if kv_heads is None else _typed(kv_heads, "kv_heads", int, at),
                   dim=_require(m, "dim", int, at), vdim=_require(m, "vdim", int, at),
                   scale=_require(m, "scale", float, at), rot=NinisunRotation.from_dict(m.get("rot"), at),
                   window=None if window is None else _typed(window, "mask.size", int, at),
                   keep_first=_typed(mask.get("keep_first", 0), "mask.keep_first", int, at),
                   v_mix=_typed(m.get("v_mix", False), "v_mix", bool, at) if masked else False)

    def to_dict(self, masked: bool) -> Dict[str, Any]:
        out: Dict[str, Any] = dict(dim=self.dim, heads=self.heads, kv_heads=self.kv_heads, scale=self.scale,
                                   vdim=self.vdim)
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if masked:
            if self.window is not None or self.keep_first:
                out["mask"] = dict(keep_first=self.keep_first, size=self.window)
            out["v_mix"] = self.v_mix
        return out

    def check(self, at: str) -> None:
        if min(self.heads, self.kv_heads, self.dim, self.vdim) <= 0:
            raise ConfigError(f"{at}: heads, kv_heads, dim and vdim must be positive")
        if self.heads % self.kv_heads:
            raise ConfigError(f"{at}: heads {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        if not math.isfinite(self.scale):
            raise ConfigError(f"{at}: scale must be finite")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"{at}: mask.size must be positive, got {self.window}")
        if self.keep_first < 0:
            raise ConfigError(f"{at}: mask.keep_first must not be negative")
        if self.rot is not None:
            self.rot.check(self.dim, at)


@dataclasses.dataclass(frozen=True)
class NinisunRecurrent:
    heads: int
    dim: int


@dataclasses.dataclass(frozen=True)
class NinisunLayer:
    """``type`` "attention": ``attention``.  ``type`` "parallel": ``left``, ``right`` and the two weights."""

    type: str
    mlp: Optional[NinisunFeedForward] = None
    attention: Optional[NinisunAttention] = None
    left: Optional[NinisunAttention] = None
    right: Optional[NinisunRecurrent] = None
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclasses.dataclass(frozen=True)
class NinisunConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[NinisunLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Ninisun"

    ARCHITECTURE = "Ninisun"
    MAX_POSITIONS = 1 << 20          # the design has no position table: the engine's own bound
    DEFAULT_DECAY_RANK = 16          # random-weights mode: the configuration names no rank

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "NinisunConfig":
        name = raw.get("architecture", (raw.get("architectures") or [cls.ARCHITECTURE])[0])
        if name != cls.ARCHITECTURE:
            raise ConfigError(f"{where}: architecture must be '{cls.ARCHITECTURE}', got {name!r}")
        norm = raw.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError(f"{where}: required key 'norm' (with 'eps') is missing")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"{where}: key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(listed):
            at = f"{where}: layers[{i}]"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"{at} must be an object with 'type' and 'mixer'")
            kind, m = _require(entry, "type", str, at), entry["mixer"]
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict):
                    raise ConfigError(f"{at}: 'mlp' is an object or null")
                mlp = NinisunFeedForward(_typed(mlp.get("kind", "dense"), "mlp.kind", str, at),
                                         _require(mlp, "ff", int, at + ".mlp"))
            if kind == "attention":
                layers.append(NinisunLayer(kind, mlp, attention=NinisunAttention.from_dict(m, at, masked=True)))
            elif kind == "parallel":
                right = m.get("right")
                if not isinstance(right, dict):
                    raise ConfigError(f"{at}: 'mixer.right' must be an object")
                layers.append(NinisunLayer(
                    kind, mlp, left=NinisunAttention.from_dict(m.get("left"), at + ".left", masked=False),
                    right=NinisunRecurrent(_require(right, "heads", int, at + ".right"),
                                           _require(right, "dim", int, at + ".right")),
                    left_scale=_require(m, "left_scale", float, at), right_scale=_require(m, "right_scale", float, at)))
            else:
                raise ConfigError(f"{at}: unknown layer type '{kind}' (known: attention, parallel)")
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where)
                                               for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(norm, "eps", float, where + ": norm"), layers=tuple(layers),
                  eos_token_ids=eos_ids)
        cfg.validate(where)
        return cfg

    def value_mix_layers(self):
        """The layers whose values are mixed, in order: the first one gives, the others take."""
        return [i for i, l in enumerate(self.layers) if l.type == "attention" and l.attention.v_mix]

    def validate(self, where: str = "config") -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"{where}: 'vocab' and 'width' must be positive")
        if not (math.isfinite(self.norm_eps) and self.norm_eps > 0):
            raise ConfigError(f"{where}: norm.eps must be finite and > 0, got {self.norm_eps}")
        for i, l in enumerate(self.layers):
            at = f"{where}: layers[{i}]"
            if l.mlp is not None and (l.mlp.kind != "dense" or l.mlp.ff <= 0):
                raise ConfigError(f"{at}: the feed-forward is of kind 'dense' with a positive 'ff', got {l.mlp}")
            if l.type == "attention":
                l.attention.check(at)
            else:
                l.left.check(at + ".left")
                if min(l.right.heads, l.right.dim) <= 0:
                    raise ConfigError(f"{at}.right: heads and dim must be positive")
                if not (math.isfinite(l.left_scale) and math.isfinite(l.right_scale)):
                    raise ConfigError(f"{at}: left_scale and right_scale must be finite")
        mixing = self.value_mix_layers()
        for i in mixing[1:]:
            a, b = self.layers[mixing[0]].attention, self.layers[i].attention
            if (a.kv_heads, a.vdim) != (b.kv_heads, b.vdim):
                raise ConfigError(f"{where}: layers[{i}] mixes its values with those of layers[{mixing[0]}], so its "
                                  f"kv_heads and vdim must equal that layer's")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"{where}: eos_token_id {e} is outside the vocabulary")

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            if l.type == "attention":
                mixer = l.attention.to_dict(masked=True)
            else:
                mixer = dict(left=l.left.to_dict(masked=False), left_scale=l.left_scale,
                             right=dict(dim=l.right.dim, heads=l.right.heads), right_scale=l.right_scale)
            layers.append(dict(type=l.type, mixer=mixer,
                               mlp=None if l.mlp is None else dict(ff=l.mlp.ff, kind=l.mlp.kind)))
        out: Dict[str, Any] = dict(architecture=self.architecture, layers=layers, norm=dict(eps=self.norm_eps),
                                   vocab=self.vocab, width=self.width)
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
