"""``DinasunConfig``: the hyper-parameters of a Dinasun decoder, typed.

config.json of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (the factor on
what every sublayer adds to the residual stream), ``embedding.scale``, ``loop`` (``start``, ``stop``,
``times``: a span of layers that runs several times in a row, every pass entered through the model's
input injection) and a list ``layers`` whose entries name their mixer (``type``), the mixer's sizes
(``mixer``) and the feed-forward (``mlp``, or null for a layer without one).  Every size and constant
that can differ between models is read here and nowhere else; what the design fixes lives in the
parts and in the builder.  A size that no key gives (the inner width of a time-mixing layer's decay
matrices) is read from the stored tensors when they are bound.

====================  =====================================================================
mixer                 keys of ``mixer``
====================  =====================================================================
wkv                   heads, dim
attention             heads, kv_heads, dim, vdim (the values are the keys: equal to dim), scale,
                      q_temp.coef, q_temp.every (absent: no query temperature)
====================  =====================================================================

``mlp``: ``kind`` "moe" with ``expert.ff``, ``router.experts``, ``router.top`` (the choice is a stored
table by token id, not a router's), ``shared.ff`` (absent: no shared expert).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, Fields

MIXERS = ("wkv", "attention")
MLPS = ("moe",)


@dataclass(frozen=True)
class DinasunMixer:
    kind: str
    heads: int
    dim: int
    kv_heads: int = 0                   # attention
    vdim: int = 0
    scale: float = 1.0
    temp_coef: float = 0.0              # query temperature; every 0: none
    temp_every: int = 0


@dataclass(frozen=True)
class DinasunMLP:
    kind: str
    ff: int
    experts: int
    top: int
    shared_ff: int = 0                  # 0: no shared expert


@dataclass(frozen=True)
class DinasunLayer:
    mixer: DinasunMixer
    mlp: Optional[DinasunMLP]


@dataclass(frozen=True)
class DinasunConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    residual_mult: float
    embedding_scale: float
    layers: Tuple[DinasunLayer, ...]
    loop: Optional[Tuple[int, int, int]]        # (start, stop, times)
    max_position: int

    def run_order(self) -> Tuple[Tuple[int, bool], ...]:
        """(layer, is it the first of a pass over the looped span?) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, False) for i in range(n))
        a, b, times = self.loop
        span = tuple((i, i == a) for i in range(a, b))
        return tuple((i, False) for i in range(a)) + span * times + tuple((i, False) for i in range(b, n))

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "DinasunConfig":
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
            layers.append(DinasunLayer(_mixer(kind, mf), _mlp(lf)))
        emb = f.mapping("embedding")
        loop = None
        lp = f.mapping("loop")
        if lp is not None:
            start = lp.integer("start", lo=0, hi=len(layers))
            stop = lp.integer("stop", lo=start, hi=len(layers))
            loop = (start, stop, lp.integer("times", lo=1, hi=1 << 10))
            if stop == start:       # an empty span runs nothing, however often
                loop = None
        return DinasunConfig(
            architecture="Dinasun", vocab=f.integer("vocab"), width=f.integer("width"), eps=norm.number("eps", lo=0.0),
            residual_mult=f.number("residual_mult", default=1.0),
            embedding_scale=emb.number("scale", default=1.0) if emb is not None else 1.0,
            layers=tuple(layers), loop=loop, max_position=f.integer("max_position", default=1 << 20, hi=1 << 30))


def _mlp(lf: Fields) -> Optional[DinasunMLP]:
    mlp = lf.mapping("mlp")
    if mlp is None:
        return None
    kind = mlp.string("kind", choices=MLPS)
    ef, rf = mlp.mapping("expert"), mlp.mapping("router")
    if ef is None or rf is None:
        raise ConfigError(f"{mlp.where}: 'expert' and 'router' are required objects")
    experts = rf.integer("experts", hi=1 << 12)
    sf = mlp.mapping("shared")
    return DinasunMLP(kind, ef.integer("ff"), experts=experts, top=rf.integer("top", hi=experts),
                      shared_ff=sf.integer("ff") if sf is not None else 0)


def _mixer(kind: str, mf: Fields) -> DinasunMixer:
    heads, dim = mf.integer("heads"), mf.integer("dim")
    if kind == "wkv":
        return DinasunMixer(kind, heads, dim)
    kv_heads = mf.integer("kv_heads", hi=heads)
    if heads % kv_heads:
        raise ConfigError(f"{mf.where}: {heads} heads are not a multiple of kv_heads = {kv_heads}")
    vdim = mf.integer("vdim", default=dim)
    if vdim != dim:
        raise ConfigError(f"{mf.where}: the values are the keys, so vdim = {vdim} must equal dim = {dim}")
    temp = mf.mapping("q_temp")
    return DinasunMixer(kind, heads, dim, kv_heads=kv_heads, vdim=vdim, scale=mf.number("scale"),
                        temp_coef=temp.number("coef") if temp is not None else 0.0,
                        temp_every=temp.integer("every", hi=1 << 30) if temp is not None else 0)
