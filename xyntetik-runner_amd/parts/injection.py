"""Remaking the residual stream from itself and the embedding's rows.

``ConcatProjection``: ``x <- W [x; x0]`` with ``W [E, 2E]`` (the stream's columns first), ``x0`` the
embedding's rows as they left the embedding.  A model whose span of layers runs several times in a row
does this before the first layer of every pass, so that every pass sees the input again.  The two halves
of ``W`` are kept as two matrices: the product over the stream and the product over ``x0`` add up in
32 bits, and ``x0`` is rounded to the products' operand type once a step.

``StepAddition``: ``x <- x + [pass > 0] x0 + step[pass]`` with ``step [passes, E]``: every pass over the span begins
with a vector of its own added to every row, and every pass but the first sees the embedding's rows again.
Everything is 32-bit.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import Injection, ParamSpec, register_injection


class ConcatProjection(Injection):
    def __init__(self, hidden_size: int, weight_name: str = "weight"):
        self.hidden_size, self.weight_name = int(hidden_size), weight_name
        self.w_x = self.w_x0 = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        E = self.hidden_size
        # of the size that keeps a stream's scale: each half adds E terms
        return {self.weight_name: ParamSpec((E, 2 * E), init=f"normal:{(2 * E) ** -0.5:.6g}")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        E = self.hidden_size
        w = tensors[self.weight_name]
        self.w_x = rt.ops.pack_weight(w[:, :E].contiguous())
        self.w_x0 = rt.ops.pack_weight(w[:, E:].contiguous())

    def prepare(self, ctx, embedded: torch.Tensor):
        """The embedding's rows in the products' operand type (a copy: the layers change the stream in place)."""
        return self.rt.ops.convert(embedded, self.rt.dtype)

    def forward(self, ctx, x, x0, pass_index: int = 0):
        ops = self.rt.ops
        out = ops.linear(x if self.rt.is_fp32 else ops.convert(x, self.rt.dtype), self.w_x, out_dtype=torch.float32)
        ops.linear(x0, self.w_x0, out=out, accumulate=True)
        return out


class StepAddition(Injection):
    def __init__(self, hidden_size: int, passes: int, weight_name: str = "step"):
        if int(passes) < 1:
            raise ValueError(f"step addition: {passes} passes")
        self.hidden_size, self.passes, self.weight_name = int(hidden_size), int(passes), weight_name
        self.steps = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        # of the size of the stream's entries: a vector that is left out, or the wrong pass's, must show
        return {self.weight_name: ParamSpec((self.passes, self.hidden_size), role="vector", init="normal:0.5")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.steps = tensors[self.weight_name].float().contiguous()

    def prepare(self, ctx, embedded: torch.Tensor):
        """A copy of the embedding's rows (the layers change the stream in place); none if no pass needs it."""
        return self.rt.ops.convert(embedded, torch.float32) if self.passes > 1 else None

    def forward(self, ctx, x, x0, pass_index: int = 0):
        if not (0 <= pass_index < self.passes):
            raise ValueError(f"step addition: pass {pass_index} of {self.passes}")
        self.rt.ops.add_rows_(x, self.steps[pass_index], y=x0 if pass_index > 0 else None)
        return x


register_injection("concat_projection", ConcatProjection)
register_injection("step_addition", StepAddition)
