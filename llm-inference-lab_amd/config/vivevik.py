"""Typed configuration of the Vivevik decoder, read from ``config.json``.

The file lists the layers one by one: each has a ``type`` (which mixer it has), the
mixer's sizes and constants (``mixer``), and its feed-forward (``mlp``, or null for a layer
with the mixer only).  Sizes that the file does not name (the rank of the decay projection
of a ``gla`` mixer) are read off the tensors' shapes when the weights are loaded.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .qwen2 import _require, _typed


@dataclasses.dataclass(frozen=True)
class VivevikFeedForward:
    kind: str
    ff: int


@dataclasses.dataclass(frozen=True)
class VivevikLayer:
    """One layer.  ``type`` "gla": ``heads, dim, vdim, tau`` (and ``rank``, or None to take it
    from the tensors).  ``type`` "attention": ``heads, kv_heads, dim, vdim, scale``, the mask
    (``window`` None: no window; ``keep_first``) and ``kv_from`` (the layer whose keys and
    values this one reads, or None if it has its own)."""

    type: str
    heads: int
    dim: int
    vdim: int
    mlp: Optional[VivevikFeedForward] = None
    tau: Optional[float] = None
    rank: Optional[int] = None
    kv_heads: Optional[int] = None
    scale: Optional[float] = None
    window: Optional[int] = None
    keep_first: int = 0
    kv_from: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class VivevikConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[VivevikLayer, ...]
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Vivevik"

    ARCHITECTURE = "Vivevik"
    MAX_POSITIONS = 1 << 20          # the design has no position table: the engine's own bound
    DEFAULT_DECAY_RANK = 32          # random-weights mode, when the configuration names no rank

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "VivevikConfig":
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
                mlp = VivevikFeedForward(_typed(mlp.get("kind", "dense"), "mlp.kind", str, at),
                                         _require(mlp, "ff", int, at + ".mlp"))
            common = dict(type=kind, heads=_require(m, "heads", int, at), dim=_require(m, "dim", int, at),
                          vdim=_require(m, "vdim", int, at), mlp=mlp)
            if kind == "gla":
                rank = m.get("rank")
                layers.append(VivevikLayer(tau=_require(m, "tau", float, at),
                                           rank=None if rank is None else _typed(rank, "rank", int, at), **common))
            elif kind == "attention":
                mask = m.get("mask") or {}
                if not isinstance(mask, dict):
                    raise ConfigError(f"{at}: 'mask' is an object")
                window, kv_from, kv_heads = mask.get("size"), m.get("kv_from"), m.get("kv_heads")
                layers.append(VivevikLayer(
                    kv_heads=common["heads"] if kv_heads is None else _typed(kv_heads, "kv_heads", int, at),
                    scale=_require(m, "scale", float, at),
                    window=None if window is None else _typed(window, "mask.size", int, at),
                    keep_first=_typed(mask.get("keep_first", 0), "mask.keep_first", int, at),
                    kv_from=None if kv_from is None else _typed(kv_from, "kv_from", int, at), **common))
            else:
                raise ConfigError(f"{at}: unknown layer type '{kind}' (known: gla, attention)")
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where)
                                               for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(norm, "eps", float, where + ": norm"), layers=tuple(layers),
                  eos_token_ids=eos_ids)
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError(f"{where}: 'vocab' and 'width' must be positive")
        if not (math.isfinite(self.norm_eps) and self.norm_eps > 0):
            raise ConfigError(f"{where}: norm.eps must be finite and > 0, got {self.norm_eps}")
        for i, l in enumerate(self.layers):
            at = f"{where}: layers[{i}]"
            if min(l.heads, l.dim, l.vdim) <= 0:
                raise ConfigError(f"{at}: heads, dim and vdim must be positive")
            if l.mlp is not None and (l.mlp.kind != "dense" or l.mlp.ff <= 0):
                raise ConfigError(f"{at}: the feed-forward is of kind 'dense' with a positive 'ff', got {l.mlp}")
            if l.type == "gla":
                if not (l.tau and math.isfinite(l.tau) and l.tau > 0):
                    raise ConfigError(f"{at}: tau must be finite and > 0, got {l.tau}")
                if l.rank is not None and l.rank <= 0:
                    raise ConfigError(f"{at}: rank must be positive")
            else:
                if l.kv_heads <= 0 or l.heads % l.kv_heads:
                    raise ConfigError(f"{at}: heads {l.heads} is not a multiple of kv_heads {l.kv_heads}")
                if l.window is not None and l.window <= 0:
                    raise ConfigError(f"{at}: mask.size must be positive, got {l.window}")
                if l.keep_first < 0:
                    raise ConfigError(f"{at}: mask.keep_first must not be negative")
                if l.kv_from is not None:
                    src = self.layers[l.kv_from] if 0 <= l.kv_from < i else None
                    if src is None or src.type != "attention" or src.kv_from is not None:
                        raise ConfigError(f"{at}: kv_from must name an earlier attention layer with keys and "
                                          f"values of its own, got {l.kv_from}")
                    if (src.kv_heads, src.dim, src.vdim) != (l.kv_heads, l.dim, l.vdim):
                        raise ConfigError(f"{at}: its kv_heads, dim and vdim must equal those of layer {l.kv_from}")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"{where}: eos_token_id {e} is outside the vocabulary")

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            if l.type == "gla":
                mixer: Dict[str, Any] = dict(dim=l.dim, heads=l.heads, tau=l.tau, vdim=l.vdim)
                if l.rank is not None:
                    mixer["rank"] = l.rank
            else:
                mixer = dict(dim=l.dim, heads=l.heads, kv_heads=l.kv_heads, scale=l.scale, vdim=l.vdim)
                if l.window is not None or l.keep_first:
                    mixer["mask"] = dict(keep_first=l.keep_first, size=l.window)
                if l.kv_from is not None:
                    mixer["kv_from"] = l.kv_from
            layers.append(dict(type=l.type, mixer=mixer,
                               mlp=None if l.mlp is None else dict(ff=l.mlp.ff, kind=l.mlp.kind)))
        out: Dict[str, Any] = dict(architecture=self.architecture, layers=layers, norm=dict(eps=self.norm_eps),
                                   vocab=self.vocab, width=self.width)
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
