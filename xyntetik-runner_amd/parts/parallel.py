"""Two mixers side by side: both read the same input, and their results meet in one sum.

``ParallelMixers``: ``y = a_left f(left(h)) + a_right f(right(h))`` with two numbers and ``f`` either the identity
or, with ``out_norm``, an RMS norm over the model's width with a weight of its own a side (the plain weight, eps
inside the root).  The two sides are mixers of any registered kind, built from their own ``PartSpec``; their
tensors lie under the prefixes ``left.`` and ``right.``.  At most one side keeps paged keys and values (it gets
the layer's pages); the sides' per-request state is kept under the side's name, and each side sees a view of the
layer's cache that holds what is its own (``SideCache``).  The results are 32-bit rows and the sum is made in 32 bits, straight
into the residual stream where the arrangement adds it there.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from dataclasses import dataclass, field

from .base import Mixer, ParamSpec, StateSpec, make_part, register_mixer


@dataclass
class SideCache:
    """What one side sees of the layer's cache: the fields of the layer's own record that a mixer reads."""
    group: int
    page_size: int
    owns: bool
    k: Optional[torch.Tensor]
    v: Optional[torch.Tensor]
    state: Optional[torch.Tensor] = None
    states: Dict[str, torch.Tensor] = field(default_factory=dict)

SIDES = ("left", "right")


class ParallelMixers(Mixer):
    def __init__(self, hidden_size: int, left, right, left_scale: float = 1.0, right_scale: float = 1.0,
                 out_norm: bool = False, eps: float = 0.0, left_norm_name: str = "left.out", right_norm_name: str = "right.out"):
        self.hidden_size = int(hidden_size)
        self.sides = {"left": make_part("mixer", left), "right": make_part("mixer", right)}
        self.scales = {"left": float(left_scale), "right": float(right_scale)}
        self.out_norm, self.eps = bool(out_norm), float(eps)
        self.norm_names = {"left": left_norm_name, "right": right_norm_name}
        self.norm_w: Dict[str, Optional[torch.Tensor]] = {"left": None, "right": None}
        if sum(1 for m in self.sides.values() if m.kv_spec() is not None) > 1:
            raise ValueError("parallel mixers: only one side can keep paged keys and values")

    @property
    def capturable(self) -> bool:
        return all(m.capturable for m in self.sides.values())

    def kv_spec(self):
        for m in self.sides.values():
            if m.kv_spec() is not None:
                return m.kv_spec()
        return None

    def state_spec(self):
        out: Dict[str, StateSpec] = {}
        for side, m in self.sides.items():
            st = m.state_spec()
            if isinstance(st, StateSpec):
                out[side] = st
            elif st:
                out.update({f"{side}.{name}": spec for name, spec in st.items()})
        return out or None

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {}
        for side, m in self.sides.items():
            specs.update({f"{side}.{name}": ps for name, ps in m.param_specs().items()})
            if self.out_norm:
                specs[self.norm_names[side]] = ParamSpec((self.hidden_size,), role="vector", init="ones_jitter")
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        for side, m in self.sides.items():
            m.bind({name: tensors[f"{side}.{name}"] for name in m.param_specs() if f"{side}.{name}" in tensors}, rt)
            if self.out_norm:
                self.norm_w[side] = tensors[self.norm_names[side]].float().contiguous()

    def _view(self, cache, side: str):
        """What ``side`` sees of the layer's cache: the pages if it keeps any, and its own state tensors under the
        names it gave them."""
        m = self.sides[side]
        pages = m.kv_spec() is not None
        own, single = {}, cache.states.get(f"mixer.{side}")
        if single is not None:
            own["mixer"] = single
        lead = f"mixer.{side}."
        own.update({"mixer." + name[len(lead):]: t for name, t in cache.states.items() if name.startswith(lead)})
        return SideCache(cache.group if pages else -1, cache.page_size, cache.owns, cache.k if pages else None,
                         cache.v if pages else None, single, own)

    def _results(self, ctx, cache, h):
        return [self.sides[side].forward_f32(ctx, self._view(cache, side), h) for side in SIDES]

    def forward_add(self, ctx, cache, h, residual) -> None:
        yl, yr = self._results(ctx, cache, h)
        self.rt.ops.pair_combine_(residual, yl.contiguous(), yr.contiguous(), self.scales["left"], self.scales["right"],
                                  self.norm_w["left"], self.norm_w["right"], self.eps)

    def forward_add_norm(self, ctx, cache, h, residual, norm, defer=False):
        """The sides' sum into the residual stream and ``norm`` of the updated rows in the same kernel, where
        ``norm`` is an RMS norm with a weight."""
        fold = norm.fold()
        if fold is None or fold[0] is None:
            return super().forward_add_norm(ctx, cache, h, residual, norm, defer)
        kept = getattr(norm, "_f32_weight", None)
        if kept is None or kept[0] is not fold[0]:
            kept = norm._f32_weight = (fold[0], fold[0].float().contiguous())
        yl, yr = self._results(ctx, cache, h)
        return self.rt.ops.pair_combine_(residual, yl.contiguous(), yr.contiguous(), self.scales["left"], self.scales["right"],
                                         self.norm_w["left"], self.norm_w["right"], self.eps,
                                         then_norm=(kept[1], fold[1]), out_dtype=self.rt.dtype)

    def forward_f32(self, ctx, cache, h):
        yl, yr = self._results(ctx, cache, h)
        out = torch.empty_like(yl)
        self.rt.ops.fill_rows_(out.view(1, -1), None, 1, 0)
        self.rt.ops.pair_combine_(out, yl.contiguous(), yr.contiguous(), self.scales["left"], self.scales["right"],
                                  self.norm_w["left"], self.norm_w["right"], self.eps)
        return out

    def forward(self, ctx, cache, h):
        return self.rt.ops.convert(self.forward_f32(ctx, cache, h), self.rt.dtype)


register_mixer("parallel_mixers", ParallelMixers)
