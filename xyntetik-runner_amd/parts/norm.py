"""Norms of the residual stream, in 32-bit.

RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w``
(src/model.c:3386-3392; kernel src/kernels.cu:32-48).
LayerNorm: ``y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w``, a weight and no bias.
DynamicTanh: ``y = tanh(alpha x) * w + b`` with one learned number ``alpha``: no mean and no variance,
so every element stands alone and a block may fold it into whatever pass touches the rows anyway.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    def __init__(self, size: int, eps: float, weight_name: str = "weight", has_weight: bool = True, optional: bool = False):
        self.size, self.eps = int(size), float(eps)
        self.weight_name, self.has_weight, self.optional = weight_name, has_weight, bool(optional)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if not self.has_weight:
            return {}
        return {self.weight_name: ParamSpec((self.size,), role="vector", init="ones_jitter", optional=self.optional)}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.weight = tensors.get(self.weight_name)

    def forward(self, ctx, x, rows=None):
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.rt.dtype, rows=rows)

    def fold(self):
        return (self.weight, self.eps) if self.weight is not None else None


class LayerNorm(Norm):
    """``out_dtype``: "compute" (the engine's dtype) or "float32", for a reader that wants the
    rows unrounded (a filter that carries them from token to token)."""

    def __init__(self, size: int, eps: float, weight_name: str = "weight", has_weight: bool = True,
                 out_dtype: str = "compute", optional: bool = False):
        if out_dtype not in ("compute", "float32"):
            raise ValueError(f"layer norm: out_dtype {out_dtype!r} (compute or float32)")
        self.size, self.eps = int(size), float(eps)
        self.weight_name, self.has_weight, self.out_dtype, self.optional = weight_name, has_weight, out_dtype, bool(optional)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if not self.has_weight:
            return {}
        return {self.weight_name: ParamSpec((self.size,), role="vector", init="ones_jitter", optional=self.optional)}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        w = tensors.get(self.weight_name)
        self.weight = w.float().contiguous() if w is not None else None

    def forward(self, ctx, x, rows=None):
        dt = torch.float32 if self.out_dtype == "float32" else self.rt.dtype
        return self.rt.ops.layernorm(x, self.weight, self.eps, dt, rows=rows)


class DynamicTanh(Norm):
    """Tensors: the weight ``[size]`` under ``weight_name``, and beside it ``<weight_name>.b`` (the bias) and
    ``<weight_name>.alpha`` (a scalar), unless named otherwise."""

    def __init__(self, size: int, weight_name: str = "weight", bias_name: Optional[str] = None,
                 alpha_name: Optional[str] = None, out_dtype: str = "compute", optional: bool = False):
        if out_dtype not in ("compute", "float32"):
            raise ValueError(f"dynamic tanh: out_dtype {out_dtype!r} (compute or float32)")
        self.size, self.out_dtype, self.optional = int(size), out_dtype, bool(optional)
        self.names = (weight_name, bias_name or weight_name + ".b", alpha_name or weight_name + ".alpha")
        self.weight = self.bias = None
        self.alpha = 1.0

    def param_specs(self) -> Dict[str, ParamSpec]:
        w, b, a = self.names
        # a bias and an alpha that a wrong reading would show: neither 0 nor 1
        return {w: ParamSpec((self.size,), role="vector", init="ones_jitter", optional=self.optional),
                b: ParamSpec((self.size,), role="vector", init="normal:0.1", optional=self.optional),
                a: ParamSpec((), role="vector", init="around:0.7:0.1", optional=self.optional)}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        w, b, a = self.names
        if w not in tensors:        # an optional norm the file leaves out is never run
            return
        self.weight = tensors[w].float().contiguous()
        self.bias = tensors[b].float().contiguous()
        self.alpha = float(tensors[a].float().item())

    def dyt(self):
        """(alpha, weight, bias) for a kernel that applies the norm itself."""
        return self.alpha, self.weight, self.bias

    def forward(self, ctx, x, rows=None):
        dt = torch.float32 if self.out_dtype == "float32" else self.rt.dtype
        return self.rt.ops.dyt(x, self.alpha, self.weight, self.bias, dt, rows=rows)


register_norm("dynamic_tanh", DynamicTanh)
register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
