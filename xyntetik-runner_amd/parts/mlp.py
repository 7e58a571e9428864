"""Gated feed-forward: ``down(act(gate(h)) * up(h))``; act = SiLU is the one activation the
reference has (src/model.c:6399-6407, ``gated_act`` :4451-4452); "clamped_swish" with a limit L
shapes both branches (``g' = min(g, L)``, ``u' = clamp(u, -L, L)``, ``g' sigmoid(1.702 g') (u' + 1)``).  The
products' epilogues apply either to their 32-bit sums.

``gate`` and ``up`` are kept as one ``[2F, E]`` matrix so that one product makes both;
the reference does the reverse for a checkpoint that stores them fused
(``slice_rows``, src/model.c:238-248).

Routed experts: ``n`` small feed-forwards ``down_e(relu(up_e(h))^2)`` of which every token uses ``top``,
chosen by a router (32-bit logits, a softmax over all experts, the largest of score + correction;
the weights are the chosen scores over their sum) and added up with those weights.  Options: experts that
are gated feed-forwards themselves, ``down_e(silu(gate_e(h)) * up_e(h))`` (``activation="swiglu"``); a choice
without a router, by a table ``[vocab, top]`` of expert numbers that the token's id indexes, every chosen
expert with the weight ``1 / top`` (``routing="table"``); a shared expert that runs for every token and is
added to the sum (``shared_size``: its inner width; a gated feed-forward with the SiLU gate); scores that are
the sigmoid of each expert's logit instead of a softmax over all (``scores="sigmoid"``); a choice limited to the best
groups (``groups`` equal groups of neighbouring experts, a group's score the sum of its two largest score +
correction, ``keep_groups`` groups whose experts can be chosen; the others count as minus infinity); weights that are
the chosen scores times a number (``weight_scale``) instead of their shares of their sum.

Dense feed-forward: ``down(act(up(h)))`` with an activation over the whole row.  "polynorm":
``a N(z) + b N(z^2) + c N(z^3) + e`` with four learned numbers, powers element by element and
``N(v) = v / sqrt(mean(v^2) + eps)`` over the row, in 32-bit.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import FeedForward, ParamSpec, register_feed_forward


class GatedMLP(FeedForward):
    takes_unscaled_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", bias: bool = False,
                 gate_name: str = "gate_proj", up_name: str = "up_proj", down_name: str = "down_proj",
                 activation_param: float = 0.0, weight_suffix: str = ".weight"):
        from ..csrc.ops import GATE_ACTIVATIONS
        if activation not in GATE_ACTIVATIONS:
            raise ValueError(f"gated feed-forward: activation {activation!r} is not built into the kernels "
                             f"(known: {sorted(GATE_ACTIVATIONS)})")
        self.activation, self.activation_param = activation, float(activation_param)
        self.suffix = weight_suffix
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.bias = bool(bias)
        self.names = (gate_name, up_name, down_name)
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, F = self.hidden_size, self.intermediate_size
        g, u, d = self.names
        sfx = self.suffix
        specs = {f"{g}{sfx}": ParamSpec((F, E)), f"{u}{sfx}": ParamSpec((F, E)),
                 f"{d}{sfx}": ParamSpec((E, F))}
        if self.bias:
            specs.update({f"{g}.bias": ParamSpec((F,), role="vector", init="normal"),
                          f"{u}.bias": ParamSpec((F,), role="vector", init="normal"),
                          f"{d}.bias": ParamSpec((E,), role="vector", init="normal")})
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        g, u, d = self.names
        sfx = self.suffix
        # gate rows then up rows, so that one product makes both; in the kernels' own order
        self.w_gate_up = rt.ops.pack_weight(
            torch.cat([tensors[f"{g}{sfx}"], tensors[f"{u}{sfx}"]], dim=0).contiguous(), gated=True)
        self.w_down = rt.ops.pack_weight(tensors[f"{d}{sfx}"])
        if self.bias:
            self.b_gate_up = torch.cat([tensors[f"{g}.bias"], tensors[f"{u}.bias"]]).float().contiguous()
            self.b_down = tensors[f"{d}.bias"].float().contiguous()

    def _hidden(self, ctx, h):
        return self.rt.ops.linear_gated(h, self.w_gate_up, bias=self.b_gate_up, activation=self.activation,
                                        param=self.activation_param)

    def forward(self, ctx, h):
        return self.rt.ops.linear(self._hidden(ctx, h), self.w_down, bias=self.b_down)

    def forward_f32(self, ctx, h):
        return self.rt.ops.linear(self._hidden(ctx, h), self.w_down, bias=self.b_down, out_dtype=torch.float32)

    def forward_add(self, ctx, h, residual) -> None:
        self.rt.ops.linear(self._hidden(ctx, h), self.w_down, bias=self.b_down, out=residual, accumulate=True)

    def forward_add_norm(self, ctx, h, residual, norm, defer=False):
        fold = norm.fold()
        if fold is None:
            return super().forward_add_norm(ctx, h, residual, norm, defer)
        return self.rt.ops.linear_add_rmsnorm(self._hidden(ctx, h), self.w_down, residual, fold[0], fold[1],
                                              self.rt.dtype, bias=self.b_down, defer=defer)


class DenseMLP(FeedForward):
    ACTIVATIONS = ("polynorm",)

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "polynorm", eps: float = 1e-5,
                 up_name: str = "up", down_name: str = "down", act_name: str = "act"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"dense feed-forward: activation {activation!r} is not built (known: {list(self.ACTIVATIONS)})")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation, self.eps = activation, float(eps)
        self.names = (up_name, down_name, act_name)
        self.w_up = self.w_down = self.coef = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, F = self.hidden_size, self.intermediate_size
        u, d, a = self.names
        return {u: ParamSpec((F, E)), d: ParamSpec((E, F)), a: ParamSpec((4,), role="vector", init="normal:0.5")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        u, d, a = self.names
        self.w_up = rt.ops.pack_weight(tensors[u])
        self.w_down = rt.ops.pack_weight(tensors[d])
        self.coef = tensors[a].float().contiguous()

    def _hidden(self, ctx, h):
        # the row's statistics are of the unrounded products
        z = self.rt.ops.linear(h, self.w_up, out_dtype=torch.float32)
        return self.rt.ops.polynorm(z, self.coef, self.eps, self.rt.dtype)

    def forward(self, ctx, h):
        return self.rt.ops.linear(self._hidden(ctx, h), self.w_down)

    def forward_add(self, ctx, h, residual) -> None:
        self.rt.ops.linear(self._hidden(ctx, h), self.w_down, out=residual, accumulate=True)


class RoutedExperts(FeedForward):
    """``n`` experts ``down_e(relu(up_e h)^2)`` without biases, ``top`` a token.  Tensors: ``router [n, E]``,
    ``correction [n]`` (added to the scores for the choice only), and per expert ``e<i>.up [F, E]``,
    ``e<i>.down [E, F]`` (gated experts: also ``e<i>.gate [F, E]``); with ``routing="table"`` no router but
    ``table [vocab, top]`` (integers); with a shared expert ``shared.gate``, ``shared.up``, ``shared.down``.
    Nothing here reads the choice on the host: the kernels find a token's
    experts on the device, so decode steps are recorded like any other."""
    ACTIVATIONS = ("relu2", "swiglu")
    ROUTINGS = ("router", "table")
    MAX_EXPERTS, MAX_TOP = 1024, 64     # MOE_MAX_EXPERTS, MOE_MAX_TOP of csrc/moe_kernels.hip

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int, activation: str = "relu2",
                 router_name: str = "router", correction_name: str = "correction", expert_prefix: str = "e",
                 up_name: str = "up", down_name: str = "down", gate_name: str = "gate", routing: str = "router",
                 vocab_size: int = 0, table_name: str = "table", shared_size: int = 0, shared_prefix: str = "shared.",
                 scores: str = "softmax", groups: int = 1, keep_groups: int = 1, weight_scale=None):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"routed experts: activation {activation!r} is not built (known: {list(self.ACTIVATIONS)})")
        if routing not in self.ROUTINGS:
            raise ValueError(f"routed experts: routing {routing!r} (known: {list(self.ROUTINGS)})")
        if routing == "table" and int(vocab_size) < 1:
            raise ValueError("routed experts: a table of experts by token id needs the vocabulary's size")
        self.activation, self.routing, self.vocab_size = activation, routing, int(vocab_size)
        self.gate_name, self.table_name = gate_name, table_name
        self.shared = (GatedMLP(hidden_size, int(shared_size), activation="silu", gate_name=shared_prefix + "gate",
                                up_name=shared_prefix + "up", down_name=shared_prefix + "down", weight_suffix="")
                       if int(shared_size) > 0 else None)
        if not (1 <= int(top) <= int(num_experts)):
            raise ValueError(f"routed experts: {top} of {num_experts} experts a token")
        if int(num_experts) > self.MAX_EXPERTS or int(top) > self.MAX_TOP:       # refused when the model is built, not at its first step
            raise ValueError(f"routed experts: the kernels take up to {self.MAX_EXPERTS} experts and {self.MAX_TOP} a token, "
                             f"not {num_experts} and {top}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.num_experts, self.top = int(num_experts), int(top)
        groups, keep_groups = int(groups), int(keep_groups)
        if scores not in ("softmax", "sigmoid"):
            raise ValueError(f"routed experts: scores {scores!r} (softmax or sigmoid)")
        if (groups < 1 or self.num_experts % groups or not (1 <= keep_groups <= groups)
                or self.top > keep_groups * (self.num_experts // groups)):
            raise ValueError(f"routed experts: {num_experts} experts in {groups} groups of which {keep_groups} are kept "
                             f"cannot give {top} choices a token")
        if weight_scale is not None and not float(weight_scale) > 0.0:
            raise ValueError(f"routed experts: weight scale {weight_scale} must be positive")
        self.how = dict(scores=scores, groups=groups, keep_groups=keep_groups,
                        weight_scale=float(weight_scale) if weight_scale is not None else None)
        self.names = (router_name, correction_name, expert_prefix, up_name, down_name)

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, F = self.hidden_size, self.intermediate_size
        r, c, p, u, d = self.names
        if self.routing == "table":
            specs = {self.table_name: ParamSpec((self.vocab_size, self.top), role="int", init=f"choice:{self.num_experts}")}
        else:
            # a router of N(0, 0.02) would score all experts alike; a correction that matters is as large as the scores differ
            specs = {r: ParamSpec((self.num_experts, E), init="normal:0.5"),
                     c: ParamSpec((self.num_experts,), role="vector", init="normal:0.1")}
        for e in range(self.num_experts):
            if self.activation == "swiglu":
                specs[f"{p}{e}.{self.gate_name}"] = ParamSpec((F, E))
            specs[f"{p}{e}.{u}"] = ParamSpec((F, E))
            specs[f"{p}{e}.{d}"] = ParamSpec((E, F))
        if self.shared is not None:
            specs.update(self.shared.param_specs())
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        r, c, p, u, d = self.names
        if self.routing == "table":
            self.table = tensors[self.table_name].to(torch.int32).contiguous()
        else:
            self.router = rt.ops.pack_weight(tensors[r])        # in the rows' dtype: the logits are a 32-bit product of the two
            self.correction = tensors[c].float().contiguous()
        if self.activation == "swiglu":     # an expert's gate rows before its up rows: one matrix [2F, E] an expert
            self.w_up = torch.stack([torch.cat([tensors[f"{p}{e}.{self.gate_name}"], tensors[f"{p}{e}.{u}"]], dim=0)
                                     for e in range(self.num_experts)]).contiguous()
        else:
            self.w_up = torch.stack([tensors[f"{p}{e}.{u}"] for e in range(self.num_experts)]).contiguous()
        self.w_down = torch.stack([tensors[f"{p}{e}.{d}"] for e in range(self.num_experts)]).contiguous()
        if self.shared is not None:
            self.shared.bind({name: tensors[name] for name in self.shared.param_specs()}, rt)

    def _run(self, ctx, h, out=None, accumulate=False):
        ops = self.rt.ops
        if self.routing == "table":
            idx, wts = ops.table_route(self.table, ctx.token_ids, self.num_experts)
        else:
            idx, wts = ops.moe_route(h, self.router, self.correction, self.top, **self.how)
        out = ops.moe_experts(h, self.w_up, self.w_down, idx, wts, out=out, accumulate=accumulate, activation=self.activation)
        if self.shared is not None:
            self.shared.forward_add(ctx, h, out)
        return out

    def forward(self, ctx, h):
        return self.rt.ops.convert(self._run(ctx, h), self.rt.dtype)

    def forward_f32(self, ctx, h):
        return self._run(ctx, h)

    def forward_add(self, ctx, h, residual) -> None:
        self._run(ctx, h, out=residual, accumulate=True)


register_feed_forward("gated_mlp", GatedMLP)
register_feed_forward("routed_experts", RoutedExperts)
register_feed_forward("dense_mlp", DenseMLP)
