"""Transforms of an attention's 32-bit queries and keys between their projection and the cache.

``HeadRMSNorm``: every query head and every key head is divided by its root mean square (eps inside
the root) and multiplied by a weight over the head's channels that all heads share (one for the
queries, one for the keys; the plain weight, not one plus it).  With ``temp_every`` the queries of the
token at position p are also multiplied by ``1 + temp_coef ln(floor((p + 1) / temp_every) + 1)``, which
sharpens the attention of tokens far into a sequence.
"""
from __future__ import annotations

from typing import Dict, Optional

from .base import ParamSpec, QKTransform, register_qk_transform


class HeadRMSNorm(QKTransform):
    def __init__(self, head_dim: int, eps: float, q_name: Optional[str] = "q_norm", k_name: Optional[str] = "k_norm",
                 temp_coef: float = 0.0, temp_every: int = 0):
        if temp_every < 0:
            raise ValueError(f"head norm: a query temperature every {temp_every} positions")
        self.head_dim, self.eps = int(head_dim), float(eps)
        self.q_name, self.k_name = q_name, k_name                   # None: that side is not normed
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.w_q = self.w_k = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        out = {}
        for name in (self.q_name, self.k_name):
            if name is not None:
                out[name] = ParamSpec((self.head_dim,), role="vector", init="ones_jitter")
        return out

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.w_q = tensors[self.q_name].float().contiguous() if self.q_name is not None else None
        self.w_k = tensors[self.k_name].float().contiguous() if self.k_name is not None else None

    def apply(self, ctx, q, k) -> None:
        self.rt.ops.head_rmsnorm_(q, k, self.w_q, self.w_k if k is not None else None, self.eps, ctx.positions,
                                  self.temp_coef, self.temp_every)


register_qk_transform("head_rmsnorm", HeadRMSNorm)
