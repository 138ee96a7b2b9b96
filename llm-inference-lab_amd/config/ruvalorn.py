"""Typed configuration of the Ruvalorn decoder, read from ``config.json``.

The file lists the layers one by one (``layers``: ``type``, the mixer's sizes and constants in
``mixer``, the feed-forward in ``mlp`` or null for a layer with the mixer only) and may name a
``loop``: the layers ``start .. stop-1`` run ``times`` times in a row with the same weights,
each pass with a cache of its own and a learned vector added to the stream before it.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Any, Dict, Optional, Tuple

from .errors import ConfigError
from .qwen2 import _require, _typed


@dataclasses.dataclass(frozen=True)
class RuvalornRouter:
    """The router of a mixture of experts: ``experts`` small feed-forwards and ``identity``
    outputs beyond them that stand for the layer's input itself; every token takes the ``top``
    best of them, out of the ``groups_keep`` best of ``groups`` equal groups of neighbours."""

    experts: int
    top: int
    scale: float
    identity: int = 0
    groups: int = 1
    groups_keep: int = 1


@dataclasses.dataclass(frozen=True)
class RuvalornFeedForward:
    """``kind`` "dense": one gated feed-forward ``ff`` wide.  ``kind`` "moe": experts ``ff`` wide
    each behind ``router``, and a shared expert ``shared_ff`` wide (None: none)."""

    kind: str
    ff: int
    router: Optional[RuvalornRouter] = None
    shared_ff: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class RuvalornLayer:
    """An attention layer: ``heads`` query heads on ``kv_heads`` key heads of ``dim`` channels; the
    values are the keys (``vdim == dim``); ``window`` None: every earlier position is read;
    ``rot_dims`` 0: no rotation."""

    type: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    mlp: Optional[RuvalornFeedForward] = None


@dataclasses.dataclass(frozen=True)
class RuvalornLoop:
    start: int
    stop: int
    times: int


def _object(raw, key: str, at: str, required: bool = True):
    value = raw.get(key)
    if value is None and not required:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"{at}: key '{key}' must be an object")
    return value


def _feed_forward(mlp, at: str) -> Optional[RuvalornFeedForward]:
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise ConfigError(f"{at}: 'mlp' is an object or null")
    kind = _require(mlp, "kind", str, at)
    if kind == "dense":
        return RuvalornFeedForward("dense", _require(mlp, "ff", int, at))
    if kind != "moe":
        raise ConfigError(f"{at}: unknown feed-forward kind '{kind}' (known: dense, moe)")
    r = _object(mlp, "router", at)
    groups = _object(r, "groups", at + ".router", required=False)
    router = RuvalornRouter(
        experts=_require(r, "experts", int, at + ".router"), top=_require(r, "top", int, at + ".router"),
        scale=_typed(r.get("scale", 1.0), "scale", float, at + ".router"),
        identity=_typed(r.get("identity", 0), "identity", int, at + ".router"),
        groups=1 if groups is None else _require(groups, "count", int, at + ".router.groups"),
        groups_keep=1 if groups is None else _require(groups, "keep", int, at + ".router.groups"))
    shared = _object(mlp, "shared", at, required=False)
    return RuvalornFeedForward("moe", _require(_object(mlp, "expert", at), "ff", int, at + ".expert"), router,
                               None if shared is None else _require(shared, "ff", int, at + ".shared"))


@dataclasses.dataclass(frozen=True)
class RuvalornConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[RuvalornLayer, ...]
    loop: Optional[RuvalornLoop] = None
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Ruvalorn"

    ARCHITECTURE = "Ruvalorn"
    MAX_POSITIONS = 1 << 20          # the design has no position table: the engine's own bound

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "RuvalornConfig":
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
            if kind != "attention":
                raise ConfigError(f"{at}: unknown layer type '{kind}' (known: attention)")
            heads, dim = _require(m, "heads", int, at), _require(m, "dim", int, at)
            mask, rot = _object(m, "mask", at, required=False), _object(m, "rot", at, required=False)
            kv_heads, window = m.get("kv_heads"), None if mask is None else mask.get("size")
            layers.append(RuvalornLayer(
                type=kind, heads=heads, dim=dim,
                kv_heads=heads if kv_heads is None else _typed(kv_heads, "kv_heads", int, at),
                vdim=_typed(m.get("vdim", dim), "vdim", int, at), scale=_require(m, "scale", float, at),
                window=None if window is None else _typed(window, "mask.size", int, at),
                rot_dims=0 if rot is None else _require(rot, "dims", int, at + ".rot"),
                rot_base=10000.0 if rot is None else _require(rot, "base", float, at + ".rot"),
                mlp=_feed_forward(entry.get("mlp"), at + ".mlp")))
        loop = _object(raw, "loop", where, required=False)
        if loop is not None:
            loop = RuvalornLoop(*(_require(loop, k, int, where + ": loop") for k in ("start", "stop", "times")))
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(_typed(e, "eos_token_id", int, where)
                                               for e in (eos if isinstance(eos, list) else [eos]))
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(norm, "eps", float, where + ": norm"), layers=tuple(layers), loop=loop,
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
            if min(l.heads, l.kv_heads, l.dim) <= 0 or l.heads % l.kv_heads:
                raise ConfigError(f"{at}: heads {l.heads} must be a positive multiple of kv_heads {l.kv_heads}")
            if l.vdim != l.dim:
                raise ConfigError(f"{at}: the values are the keys, so vdim {l.vdim} must equal dim {l.dim}")
            if not (math.isfinite(l.scale) and l.scale > 0):
                raise ConfigError(f"{at}: scale must be finite and > 0, got {l.scale}")
            if l.window is not None and l.window <= 0:
                raise ConfigError(f"{at}: mask.size must be positive, got {l.window}")
            if l.rot_dims < 0 or l.rot_dims % 2 or l.rot_dims > l.dim:
                raise ConfigError(f"{at}: rot.dims must be even and at most dim {l.dim}, got {l.rot_dims}")
            if l.rot_dims and not (math.isfinite(l.rot_base) and l.rot_base > 0):
                raise ConfigError(f"{at}: rot.base must be finite and > 0, got {l.rot_base}")
            f = l.mlp
            if f is None:
                continue
            if f.ff <= 0 or (f.shared_ff is not None and f.shared_ff <= 0):
                raise ConfigError(f"{at}: feed-forward widths must be positive")
            r = f.router
            if f.kind == "moe":
                total = r.experts + r.identity
                if r.experts < 0 or r.identity < 0 or total <= 0 or not 0 < r.top <= total:
                    raise ConfigError(f"{at}: the router has {r.experts} experts and {r.identity} identity outputs "
                                      f"and takes the top {r.top}")
                if r.groups <= 0 or total % r.groups or not 0 < r.groups_keep <= r.groups:
                    raise ConfigError(f"{at}: {total} router outputs do not form {r.groups} equal groups of which "
                                      f"{r.groups_keep} are kept")
                if r.groups_keep * (total // r.groups) < r.top:
                    raise ConfigError(f"{at}: the kept groups hold fewer than top = {r.top} outputs")
                if not math.isfinite(r.scale):
                    raise ConfigError(f"{at}: router.scale must be finite")
        if self.loop is not None:
            lo = self.loop
            if not 0 <= lo.start < lo.stop <= len(self.layers) or lo.times < 1:
                raise ConfigError(f"{where}: loop runs the layers start .. stop-1 ({lo.start} .. {lo.stop - 1}) "
                                  f"{lo.times} times: it needs 0 <= start < stop <= {len(self.layers)} and times >= 1")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"{where}: eos_token_id {e} is outside the vocabulary")

    def runs(self):
        """``(layer, pass)`` in the order the layers run; ``pass`` is None outside the loop."""
        n, lo = len(self.layers), self.loop
        if lo is None:
            return [(i, None) for i in range(n)]
        return ([(i, None) for i in range(lo.start)]
                + [(i, t) for t in range(lo.times) for i in range(lo.start, lo.stop)]
                + [(i, None) for i in range(lo.stop, n)])

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            mixer: Dict[str, Any] = dict(dim=l.dim, heads=l.heads, kv_heads=l.kv_heads, scale=l.scale, vdim=l.vdim)
            if l.window is not None:
                mixer["mask"] = dict(size=l.window)
            if l.rot_dims:
                mixer["rot"] = dict(base=l.rot_base, dims=l.rot_dims)
            f, mlp = l.mlp, None
            if f is not None and f.kind == "dense":
                mlp = dict(ff=f.ff, kind="dense")
            elif f is not None:
                r = f.router
                mlp = dict(expert=dict(ff=f.ff), kind="moe",
                           router=dict(experts=r.experts, groups=dict(count=r.groups, keep=r.groups_keep),
                                       identity=r.identity, scale=r.scale, top=r.top))
                if f.shared_ff is not None:
                    mlp["shared"] = dict(ff=f.shared_ff)
            layers.append(dict(type=l.type, mixer=mixer, mlp=mlp))
        out: Dict[str, Any] = dict(architecture=self.architecture, layers=layers, norm=dict(eps=self.norm_eps),
                                   vocab=self.vocab, width=self.width)
        if self.loop is not None:
            out["loop"] = dict(start=self.loop.start, stop=self.loop.stop, times=self.loop.times)
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
