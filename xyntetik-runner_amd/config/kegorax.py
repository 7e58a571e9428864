"""``KegoraxConfig``: the hyper-parameters of a Kegorax decoder, typed.

config.json of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``loop``
(``start``, ``stop``, ``times``: a span of layers that runs several times in a row) and a list ``layers``
whose entries name their mixer (``type``), the mixer's sizes (``mixer``) and the feed-forward (``mlp``, or
null for a layer without one).  Every size and constant that can differ between models is read here and
nowhere else; what the design fixes lives in the parts and in the builder.  Sizes that no key gives (the inner
widths of thin factor pairs) are read from the stored tensors when they are bound.

====================  =====================================================================
type                  keys of ``mixer``
====================  =====================================================================
parallel              left: heads, kv_heads, dim, vdim, scale, mask.size (a chunk's length), rot.base,
                      rot.dims (absent or 0: no rotation); right: heads, dim, vdim, tau
parallel_2            left: heads, kv_heads, dim, vdim, scale, mask.size (a window's length),
                      mask.keep_first; right: heads, dim, vdim, decay (a number a head);
                      left_scale, right_scale
channel_delta         heads, kv_heads, dim, vdim, conv (taps)
====================  =====================================================================

``mlp``: ``kind`` "dense" with ``ff``; or "moe" with ``expert.ff``, ``router.experts``, ``router.top``,
``router.scale``, ``router.groups.count`` and ``router.groups.keep`` (absent: one group).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, Fields

MIXERS = ("parallel", "parallel_2", "channel_delta")
MLPS = ("dense", "moe")


@dataclass(frozen=True)
class KegoraxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: int
    keep_first: int = 0
    rot_base: float = 0.0
    rot_dims: int = 0               # 0: no rotation


@dataclass(frozen=True)
class KegoraxRecurrent:
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0               # the delta rule's key heads
    tau: float = 1.0                # gated linear attention
    decay: Tuple[float, ...] = ()   # retention
    conv: int = 0                   # the delta rule's convolution taps


@dataclass(frozen=True)
class KegoraxMixer:
    kind: str
    left: Optional[KegoraxAttention] = None
    right: Optional[KegoraxRecurrent] = None
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass(frozen=True)
class KegoraxMLP:
    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1
    scale: float = 1.0


@dataclass(frozen=True)
class KegoraxLayer:
    mixer: KegoraxMixer
    mlp: Optional[KegoraxMLP]


@dataclass(frozen=True)
class KegoraxConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    layers: Tuple[KegoraxLayer, ...]
    loop: Optional[Tuple[int, int, int]]        # (start, stop, times)
    max_position: int

    def run_order(self) -> Tuple[Tuple[int, Optional[int]], ...]:
        """(layer, the number of the pass it begins or None) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, None) for i in range(n))
        a, b, times = self.loop
        out = [(i, None) for i in range(a)]
        for t in range(times):
            out += [(i, t if i == a else None) for i in range(a, b)]
        return tuple(out + [(i, None) for i in range(b, n)])

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "KegoraxConfig":
        f = Fields(raw)
        norm = f.mapping("norm")
        if norm is None:
            raise ConfigError("config.json: 'norm' is a required object")
        layers = []
        for lf in f.mappings("layers"):
            kind = lf.string("type", choices=MIXERS)
            mf = lf.mapping("mixer")
            if mf is None:
                raise ConfigError(f"{lf.where}: 'mixer' is required")
            layers.append(KegoraxLayer(_mixer(kind, mf), _mlp(lf)))
        emb = f.mapping("embedding")
        loop = None
        lp = f.mapping("loop")
        if lp is not None:
            start = lp.integer("start", lo=0, hi=len(layers))
            stop = lp.integer("stop", lo=start, hi=len(layers))
            loop = (start, stop, lp.integer("times", lo=1, hi=1 << 10))
            if stop == start:       # an empty span runs nothing, however often
                loop = None
        return KegoraxConfig(
            architecture="Kegorax", vocab=f.integer("vocab"), width=f.integer("width"), eps=norm.number("eps", lo=0.0),
            embedding_scale=emb.number("scale", default=1.0) if emb is not None else 1.0,
            layers=tuple(layers), loop=loop, max_position=f.integer("max_position", default=1 << 20, hi=1 << 30))


def _mlp(lf: Fields) -> Optional[KegoraxMLP]:
    mlp = lf.mapping("mlp")
    if mlp is None:
        return None
    kind = mlp.string("kind", choices=MLPS)
    if kind == "dense":
        return KegoraxMLP(kind, mlp.integer("ff"))
    ef, rf = mlp.mapping("expert"), mlp.mapping("router")
    if ef is None or rf is None:
        raise ConfigError(f"{mlp.where}: 'expert' and 'router' are required objects")
    experts = rf.integer("experts", hi=1 << 10)
    top = rf.integer("top", hi=experts)
    gf = rf.mapping("groups")
    groups = gf.integer("count", hi=experts) if gf is not None else 1
    keep = gf.integer("keep", hi=groups) if gf is not None else 1
    if experts % groups:
        raise ConfigError(f"{rf.where}: {experts} experts do not form {groups} equal groups")
    if top > keep * (experts // groups):
        raise ConfigError(f"{rf.where}: {keep} groups of {experts // groups} experts cannot give {top} choices")
    return KegoraxMLP(kind, ef.integer("ff"), experts=experts, top=top, groups=groups, keep_groups=keep,
                      scale=rf.number("scale", default=1.0, lo=0.0, lo_open=True))


def _attention(mf: Fields, keeps: bool, rotates: bool) -> KegoraxAttention:
    heads = mf.integer("heads")
    kv_heads = mf.integer("kv_heads", hi=heads)
    if heads % kv_heads:
        raise ConfigError(f"{mf.where}: {heads} heads are not a multiple of kv_heads = {kv_heads}")
    dim = mf.integer("dim")
    mask = mf.mapping("mask")
    if mask is None:
        raise ConfigError(f"{mf.where}: 'mask' is required")
    rot = mf.mapping("rot") if rotates else None
    dims = rot.integer("dims", default=0, lo=0, hi=dim) if rot is not None else 0
    if dims % 2:
        raise ConfigError(f"{mf.where}: rot.dims = {dims} must be even")
    return KegoraxAttention(heads, kv_heads, dim, mf.integer("vdim", default=dim), mf.number("scale"),
                            mask.integer("size", hi=1 << 30),
                            keep_first=mask.integer("keep_first", default=0, lo=0, hi=1 << 30) if keeps else 0,
                            rot_base=rot.number("base", lo=0.0, lo_open=True) if dims else 0.0, rot_dims=dims)


def _mixer(kind: str, mf: Fields) -> KegoraxMixer:
    if kind == "channel_delta":
        heads = mf.integer("heads")
        kv_heads = mf.integer("kv_heads", default=heads, hi=heads)
        if heads % kv_heads:
            raise ConfigError(f"{mf.where}: {heads} heads are not a multiple of kv_heads = {kv_heads}")
        dim = mf.integer("dim")
        return KegoraxMixer(kind, right=KegoraxRecurrent(heads, dim, mf.integer("vdim", default=dim), kv_heads=kv_heads,
                                                         conv=mf.integer("conv", lo=1, hi=16)))
    lf, rf = mf.mapping("left"), mf.mapping("right")
    if lf is None or rf is None:
        raise ConfigError(f"{mf.where}: 'left' and 'right' are required objects")
    heads, dim = rf.integer("heads"), rf.integer("dim")
    vdim = rf.integer("vdim", default=dim)
    if kind == "parallel":
        return KegoraxMixer(kind, _attention(lf, keeps=False, rotates=True),
                            KegoraxRecurrent(heads, dim, vdim, tau=rf.number("tau", lo=0.0, lo_open=True)))
    return KegoraxMixer(kind, _attention(lf, keeps=True, rotates=False),
                        KegoraxRecurrent(heads, dim, vdim, decay=rf.numbers("decay", count=heads, lo=0.0, hi=1.0)),
                        left_scale=mf.number("left_scale", default=1.0), right_scale=mf.number("right_scale", default=1.0))
