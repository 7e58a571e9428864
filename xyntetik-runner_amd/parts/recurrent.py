"""Mixers whose memory is a matrix of state per request and head, carried from token to token
in 32-bit floats (``Ops.linear_recurrence``), read out as ``o = S^T q`` after the token's update.

``Retention``: linear attention with one fixed decay a head and neither softmax nor denominator.
``q = Wq h``, ``k = Wk h`` (H heads of D), ``v = Wv h`` (H heads of Dv); an optional rotation of the
first channels of q and k; k times ``D^-1/2`` after it; ``S <- decay_h S + k v^T``.  Every head's
read-out is divided by its root mean square, then times ``silu(Wg h)``, then ``Wo``.
Its options make the other members of the family: an activation on q, k and v (``qkv_activation``:
"silu"), another scale of the keys (``key_scale``; 1 for none), the read-outs of all heads normed
together instead of head by head (``norm_over``: "row") with a weight a channel (``norm_name``), and
another gate (``gate_activation``: "sigmoid").  "Lightning attention" is retention with
``q, k, v = silu(W h)``, no key scale, the joint norm with a weight, and the sigmoid gate.

``GatedDelta``: the gated delta rule.  ``q``, ``k`` (G heads of D; head h reads head ``h // (H / G)``)
and ``v`` (H heads of Dv) each pass a short causal convolution over time and SiLU; q and k become
unit vectors ``x / sqrt(sum(x^2) + 1e-6)``, q also times ``D^-1/2``; ``beta = sigmoid(Wb h)`` and
``g = exp(-exp(A_log_h) * softplus(Wa h + dt_bias_h))`` a head; ``S <- g S; u = beta (v - S^T k);
S <- S + k u^T``.  The read-out is divided by its root mean square, times a weight over Dv that
the heads share, times ``silu(Wg h)``, then ``Wo``.  Options: a decay a head *and key channel*
(``decay="channel"``: ``g = exp(-exp(A_log_h) * softplus(Wa2 (Wa1 h) + dt_bias))`` laid out heads x D, the decay's
projection in two thin factors whose inner width the stored tensors decide, ``dt_bias`` a number a channel); a gate
through two thin factors (``gate="low_rank"``: ``Wg2 (Wg1 h)``); the sigmoid instead of SiLU on the gate
(``gate_activation``).

``GatedLinearAttention``: linear attention with a decay a token, head and key channel.  ``q = Wq h * D^-1/2``,
``k = Wk h`` (H heads of D), ``v = Wv h`` (H heads of Dv); ``w = sigmoid(Wa2 (Wa1 h) + b)^(1/tau)`` laid out heads x D;
``S <- diag(w) S + k v^T``, read out after the update.  Every head's read-out is divided by its root mean square,
times a weight over Dv that the heads share, times ``silu(Wg h)``, then ``Wo``.

``TimeMixWKV``: time mixing with a decay a token, head and key channel.  Each of r, k, v, g and the
decay reads a mix of its own of the token's row and the row before, ``h + (h_before - h) mu_s`` (the row
before a sequence's first is zero; the last row of a step is state).  ``r, k, v = W h_s`` (H heads of D,
keys and values alike), ``w = exp(-exp(W2 tanh(W1 h_w) + w0))``; per head ``o = (S + diag(u) k v^T)^T r``
from the state before the token, with the bonus ``u`` for the token itself, then ``S <- diag(w) S + k v^T``.
Every head's read-out is divided by its root mean square, times a weight a channel of the row, times
``silu(Wg h_g)``, then ``Wo``.  The width of ``W1``/``W2``'s inner side is no constant of a configuration:
the stored tensors decide it.

All keep their projections in 32 bits from the product to the recurrence: what enters a
recurrence is not rounded on the way.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from .base import Mixer, ParamSpec, StateSpec, make_part, register_mixer

MAX_KEY_DIM = 256       # a column of the state is kept in the registers of four lanes


def _check_sizes(what: str, heads: int, kv_heads: int, dim: int, vdim: int) -> None:
    if heads < 1 or kv_heads < 1 or heads % kv_heads:
        raise ValueError(f"{what}: {heads} heads are not a multiple of {kv_heads} key heads")
    if not (1 <= dim <= MAX_KEY_DIM) or vdim < 1:
        raise ValueError(f"{what}: key size {dim} (1 to {MAX_KEY_DIM}), value size {vdim}")


class Retention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, decay: Sequence[float],
                 eps: float, position=None, q_name: str = "q", k_name: str = "k", v_name: str = "v",
                 g_name: str = "g", o_name: str = "o", qkv_activation: Optional[str] = None,
                 key_scale: Optional[float] = None, norm_over: str = "head", norm_name: Optional[str] = None,
                 gate_activation: str = "silu"):
        _check_sizes("retention", num_heads, num_heads, head_dim, v_head_dim)
        if len(decay) != num_heads:
            raise ValueError(f"retention: {len(decay)} decays for {num_heads} heads")
        if qkv_activation not in (None, "silu"):
            raise ValueError(f"retention: activation {qkv_activation!r} of q, k and v is not built (none, silu)")
        if norm_over not in ("head", "row"):
            raise ValueError(f"retention: the read-outs are normed over a 'head' or over the 'row', not {norm_over!r}")
        if gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"retention: gate activation {gate_activation!r} is not built (silu, sigmoid)")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.v_head_dim = int(head_dim), int(v_head_dim)
        self.decay_values, self.eps = [float(d) for d in decay], float(eps)
        self.position = make_part("position", position) if position is not None else None
        self.names = (q_name, k_name, v_name, g_name, o_name)
        self.qk_size, self.v_size = self.num_heads * self.head_dim, self.num_heads * self.v_head_dim
        self.qkv_activation, self.norm_over, self.norm_name = qkv_activation, norm_over, norm_name
        self.key_scale = float(key_scale) if key_scale is not None else self.head_dim ** -0.5
        self.gate_activation = gate_activation
        self.w_norm = None

    @property
    def capturable(self) -> bool:
        return self.position is None or self.position.capturable

    def state_spec(self):
        from ..csrc.ops import Ops
        return StateSpec(Ops.recurrence_state_shape(self.num_heads, self.head_dim, self.v_head_dim), torch.float32)

    def param_specs(self) -> Dict[str, ParamSpec]:
        E = self.hidden_size
        q, k, v, g, o = self.names
        specs = {q: ParamSpec((self.qk_size, E)), k: ParamSpec((self.qk_size, E)), v: ParamSpec((self.v_size, E)),
                 g: ParamSpec((self.v_size, E)), o: ParamSpec((E, self.v_size))}
        if self.norm_name is not None:
            width = self.v_size if self.norm_over == "row" else self.v_head_dim
            specs[self.norm_name] = ParamSpec((width,), role="vector", init="ones_jitter")
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        q, k, v, g, o = self.names
        self.w_in = rt.ops.pack_weight(torch.cat([tensors[q], tensors[k], tensors[v], tensors[g]], dim=0).contiguous())
        self.w_out = rt.ops.pack_weight(tensors[o])
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=rt.device)
        if self.norm_name is not None:
            self.w_norm = tensors[self.norm_name].float().contiguous()
        if self.position is not None:
            self.position.bind({}, rt)
            rot = self.position.rotary()
            if rot is None or rot.interleaved or rot.mscale != 1.0:
                raise ValueError("retention rotates channel j with j + dims/2 by a plain frequency table")

    def _read_out(self, ctx, cache, h):
        ops = self.rt.ops
        H, D, Dv, QK, V = self.num_heads, self.head_dim, self.v_head_dim, self.qk_size, self.v_size
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        q, k, v, gate = proj[:, :QK], proj[:, QK:2 * QK], proj[:, 2 * QK:2 * QK + V], proj[:, 2 * QK + V:]
        rot = self.position.rotary() if self.position is not None else None
        # a short portion's recurrence applies the activation as it reads (a kernel less in a decode step); a long
        # one, which runs in chunks and reads its rows twice, takes rows that passed it before
        fused_act = self.qkv_activation if (rot is None and self.key_scale == 1.0
                                            and ctx.max_q_len < ops.RETENTION_CHUNKED_FROM) else None
        if self.qkv_activation is not None and fused_act is None:
            ops.act_rows_(proj[:, :2 * QK + V], self.qkv_activation)
        if rot is not None:
            ops.rotate_rows_(q, ctx.positions, rot.inv_freq, H, D, rot.rotary_dim, 1.0)
        if rot is not None:
            ops.rotate_rows_(k, ctx.positions, rot.inv_freq, H, D, rot.rotary_dim, self.key_scale)
        # (without a rotation the keys' scale is applied as the recurrence fetches them: a kernel less)
        o = ops.linear_recurrence("retention", q, k, v, cache.state, ctx, H, H, D, Dv, decay=self.decay, activation=fused_act,
                                  k_scale=self.key_scale if rot is None else 1.0)
        if self.norm_over == "row":
            return ops.gated_rmsnorm(o, gate, self.w_norm, 1, V, self.eps, self.rt.dtype, gate_activation=self.gate_activation)
        return ops.gated_rmsnorm(o, gate, self.w_norm, H, Dv, self.eps, self.rt.dtype, gate_activation=self.gate_activation)

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out)

    def forward_f32(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out_dtype=torch.float32)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out=residual, accumulate=True)


def pad_inner(w1: torch.Tensor, w2: torch.Tensor):
    """Two thin factors ``w1 [r, E]`` and ``w2 [N, r]`` with the inner side in whole groups of 8 (what the matrix
    cores take): rows and columns of zeros, which add nothing."""
    r = int(w1.shape[0])
    if w2.shape[1] != r:
        raise ValueError(f"thin factors {tuple(w1.shape)} and {tuple(w2.shape)} do not meet")
    if r % 8:
        pad = 8 - r % 8
        w1 = torch.cat([w1, w1.new_zeros((pad, w1.shape[1]))], dim=0)
        w2 = torch.cat([w2, w2.new_zeros((w2.shape[0], pad))], dim=1)
    return w1.contiguous(), w2.contiguous()


def _random_rank(E: int) -> int:
    """The inner width the random-weights mode gives a pair of thin factors; a file may bring any."""
    return max(4, E // 16)


class GatedLinearAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, tau: float, eps: float,
                 q_name: str = "q", k_name: str = "k", v_name: str = "v", g_name: str = "g", o_name: str = "o",
                 a1_name: str = "a1", a2_name: str = "a2", a_bias_name: str = "a2.b", norm_name: str = "norm"):
        _check_sizes("gated linear attention", num_heads, num_heads, head_dim, v_head_dim)
        if not float(tau) > 0.0:
            raise ValueError(f"gated linear attention: tau {tau} must be positive")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.v_head_dim, self.tau, self.eps = int(head_dim), int(v_head_dim), float(tau), float(eps)
        self.names = dict(q=q_name, k=k_name, v=v_name, g=g_name, o=o_name, a1=a1_name, a2=a2_name, ab=a_bias_name, norm=norm_name)
        self.qk_size, self.v_size = self.num_heads * self.head_dim, self.num_heads * self.v_head_dim

    def state_spec(self):
        from ..csrc.ops import Ops
        return StateSpec(Ops.recurrence_state_shape(self.num_heads, self.head_dim, self.v_head_dim), torch.float32)

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, QK, V, n = self.hidden_size, self.qk_size, self.v_size, self.names
        rank = _random_rank(E)
        return {n["q"]: ParamSpec((QK, E)), n["k"]: ParamSpec((QK, E)), n["v"]: ParamSpec((V, E)), n["g"]: ParamSpec((V, E)),
                n["o"]: ParamSpec((E, V)),
                n["a1"]: ParamSpec((-1, E), random_shape=(rank, E)),
                n["a2"]: ParamSpec((QK, -1), init="normal:0.5", random_shape=(QK, rank)),
                # decays between a half and nearly one: a state that lasts tens of tokens, neither one nor all
                n["ab"]: ParamSpec((QK,), role="vector", init="around:2.0:1.5"),
                n["norm"]: ParamSpec((self.v_head_dim,), role="vector", init="ones_jitter")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        n = self.names
        self.w_in = rt.ops.pack_weight(torch.cat([tensors[n[key]] for key in ("q", "k", "v", "g")], dim=0).contiguous())
        w1, w2 = pad_inner(tensors[n["a1"]], tensors[n["a2"]])
        self.w_a1, self.w_a2 = rt.ops.pack_weight(w1), rt.ops.pack_weight(w2)
        self.b_a = tensors[n["ab"]].float().contiguous()
        self.w_norm = tensors[n["norm"]].float().contiguous()
        self.w_out = rt.ops.pack_weight(tensors[n["o"]])

    def _read_out(self, ctx, cache, h):
        ops = self.rt.ops
        H, D, Dv, QK, V = self.num_heads, self.head_dim, self.v_head_dim, self.qk_size, self.v_size
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        q, k, v, gate = proj[:, :QK], proj[:, QK:2 * QK], proj[:, 2 * QK:2 * QK + V], proj[:, 2 * QK + V:]
        w = ops.linear(ops.linear(h, self.w_a1), self.w_a2, bias=self.b_a, out_dtype=torch.float32)
        ops.decay_prepare_(w, H, D, "sigmoid_root", tau=self.tau)
        state = cache.state if cache.state is not None else cache.states["mixer"]
        o = ops.linear_recurrence("gla", q, k, v, state, ctx, H, H, D, Dv, gate=w, q_scale=D ** -0.5)
        return ops.gated_rmsnorm(o, gate, self.w_norm, H, Dv, self.eps, self.rt.dtype)

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out)

    def forward_f32(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out_dtype=torch.float32)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out=residual, accumulate=True)


class GatedDelta(Mixer):
    UNIT_EPS = 1e-6

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 conv_taps: int, eps: float, q_name: str = "q", k_name: str = "k", v_name: str = "v", b_name: str = "b",
                 a_name: str = "a", a_log_name: str = "A_log", dt_bias_name: str = "dt_bias", norm_name: str = "norm",
                 g_name: str = "g", o_name: str = "o", conv_suffix: str = ".conv", decay: str = "head",
                 gate: str = "full", gate_activation: str = "silu", a1_name: str = "a1", a2_name: str = "a2",
                 g1_name: str = "g1", g2_name: str = "g2"):
        _check_sizes("gated delta rule", num_heads, num_kv_heads, head_dim, v_head_dim)
        if decay not in ("head", "channel") or gate not in ("full", "low_rank") or gate_activation not in ("silu", "sigmoid"):
            raise ValueError(f"gated delta rule: decay {decay!r} (head, channel), gate {gate!r} (full, low_rank), "
                             f"gate activation {gate_activation!r} (silu, sigmoid)")
        self.decay_kind, self.gate_kind, self.gate_activation = decay, gate, gate_activation
        self.thin = dict(a1=a1_name, a2=a2_name, g1=g1_name, g2=g2_name)
        if not (0 <= int(conv_taps) <= 16):          # 0: no convolution (SiLU alone), and no tensors of one
            raise ValueError(f"gated delta rule: {conv_taps} convolution taps (0 to 16)")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.v_head_dim = int(head_dim), int(v_head_dim)
        self.conv_taps, self.eps = int(conv_taps), float(eps)
        self.names = dict(q=q_name, k=k_name, v=v_name, b=b_name, a=a_name, a_log=a_log_name, dt_bias=dt_bias_name,
                          norm=norm_name, g=g_name, o=o_name)
        self.conv_suffix = conv_suffix
        self.qk_size, self.v_size = self.num_kv_heads * self.head_dim, self.num_heads * self.v_head_dim
        self.conv_size = 2 * self.qk_size + self.v_size

    def state_spec(self):
        from ..csrc.ops import Ops
        out = {"S": StateSpec(Ops.recurrence_state_shape(self.num_heads, self.head_dim, self.v_head_dim), torch.float32)}
        if self.conv_taps > 1:
            out["conv"] = StateSpec((self.conv_taps - 1, self.conv_size), torch.float32)
        return out

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, H, n = self.hidden_size, self.num_heads, self.names
        specs = {}
        for key, rows in (("q", self.qk_size), ("k", self.qk_size), ("v", self.v_size)):
            specs[n[key]] = ParamSpec((rows, E))
            if self.conv_taps:
                specs[n[key] + self.conv_suffix] = ParamSpec((rows, self.conv_taps), role="vector", init="normal:0.6")
        specs[n["b"]] = ParamSpec((H, E))
        rank, t = _random_rank(E), self.thin
        if self.decay_kind == "channel":
            specs[t["a1"]] = ParamSpec((-1, E), random_shape=(rank, E))
            specs[t["a2"]] = ParamSpec((H * self.head_dim, -1), init="normal:0.5", random_shape=(H * self.head_dim, rank))
            specs[n["dt_bias"]] = ParamSpec((H * self.head_dim,), role="vector", init="normal:0.5")
        else:
            specs[n["a"]] = ParamSpec((H, E))
            specs[n["dt_bias"]] = ParamSpec((H,), role="vector", init="normal:0.5")
        specs[n["a_log"]] = ParamSpec((H,), role="vector", init="normal:0.5")
        specs[n["norm"]] = ParamSpec((self.v_head_dim,), role="vector", init="ones_jitter")
        if self.gate_kind == "low_rank":
            specs[t["g1"]] = ParamSpec((-1, E), random_shape=(rank, E))
            specs[t["g2"]] = ParamSpec((self.v_size, -1), init="normal:0.5", random_shape=(self.v_size, rank))
        else:
            specs[n["g"]] = ParamSpec((self.v_size, E))
        specs[n["o"]] = ParamSpec((E, self.v_size))
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        n = self.names
        # one product for everything of the full width: q, k, v first (the convolution's columns), then the
        # gate (if it is no pair of thin factors), the write strengths, the decays a head (if they are)
        fused = ["q", "k", "v"] + (["g"] if self.gate_kind == "full" else []) + ["b"] + (["a"] if self.decay_kind == "head" else [])
        self.w_in = rt.ops.pack_weight(torch.cat([tensors[n[key]] for key in fused], dim=0).contiguous())
        t = self.thin
        if self.decay_kind == "channel":
            w1, w2 = pad_inner(tensors[t["a1"]], tensors[t["a2"]])
            self.w_a1, self.w_a2 = rt.ops.pack_weight(w1), rt.ops.pack_weight(w2)
        if self.gate_kind == "low_rank":
            w1, w2 = pad_inner(tensors[t["g1"]], tensors[t["g2"]])
            self.w_g1, self.w_g2 = rt.ops.pack_weight(w1), rt.ops.pack_weight(w2)
        if self.conv_taps:
            self.w_conv = torch.cat([tensors[n[key] + self.conv_suffix].float() for key in ("q", "k", "v")], dim=0).contiguous()
        else:       # one tap of weight 1: the kernel's SiLU alone
            self.w_conv = torch.ones((self.conv_size, 1), dtype=torch.float32, device=rt.device)
        self.a_log = tensors[n["a_log"]].float().contiguous()
        self.dt_bias = tensors[n["dt_bias"]].float().contiguous()
        self.w_norm = tensors[n["norm"]].float().contiguous()
        self.w_out = rt.ops.pack_weight(tensors[n["o"]])

    def _read_out(self, ctx, cache, h):
        ops = self.rt.ops
        H, G, D, Dv, QK, V, C = (self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, self.qk_size,
                                 self.v_size, self.conv_size)
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        y = ops.causal_conv(proj[:, :C], self.w_conv, cache.states.get("mixer.conv"), ctx, torch.float32, activation="silu")
        q, k, v = y[:, :QK], y[:, QK:2 * QK], y[:, 2 * QK:]
        at = C
        if self.gate_kind == "full":
            gate = proj[:, at:at + V]
            at += V
        else:
            gate = ops.linear(ops.linear(h, self.w_g1), self.w_g2, out_dtype=torch.float32)
        b = proj[:, at:at + H]
        if self.decay_kind == "channel":
            w = ops.linear(ops.linear(h, self.w_a1), self.w_a2, out_dtype=torch.float32)
            ops.decay_prepare_(w, H, D, "exp_softplus", a_log=self.a_log, dt_bias=self.dt_bias)
            ops.delta_prepare_(q, k, b, None, None, None, G, H, D, D ** -0.5, self.UNIT_EPS)
            o = ops.linear_recurrence("delta_channel", q, k, v, cache.states["mixer.S"], ctx, H, G, D, Dv, beta=b, gate=w)
        else:
            a = proj[:, at + H:]
            ops.delta_prepare_(q, k, b, a, self.a_log, self.dt_bias, G, H, D, D ** -0.5, self.UNIT_EPS)
            o = ops.linear_recurrence("delta", q, k, v, cache.states["mixer.S"], ctx, H, G, D, Dv, beta=b, gate=a)
        return ops.gated_rmsnorm(o, gate, self.w_norm, H, Dv, self.eps, self.rt.dtype, gate_activation=self.gate_activation)

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out)

    def forward_f32(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out_dtype=torch.float32)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out=residual, accumulate=True)

    def forward_add_norm(self, ctx, cache, h, residual, norm, defer=False):
        fold = norm.fold()
        if fold is None:
            return super().forward_add_norm(ctx, cache, h, residual, norm, defer)
        return self.rt.ops.linear_add_rmsnorm(self._read_out(ctx, cache, h), self.w_out, residual, fold[0], fold[1],
                                              self.rt.dtype, defer=defer)


class TimeMixWKV(Mixer):
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, eps: float, mu_prefix: str = "mu.", r_name: str = "r",
                 k_name: str = "k", v_name: str = "v", g_name: str = "g", o_name: str = "o", w1_name: str = "w1",
                 w2_name: str = "w2", w0_name: str = "w0", u_name: str = "u", norm_name: str = "norm"):
        _check_sizes("wkv time mixing", num_heads, num_heads, head_dim, head_dim)
        self.hidden_size, self.num_heads, self.head_dim, self.eps = int(hidden_size), int(num_heads), int(head_dim), float(eps)
        self.size = self.num_heads * self.head_dim
        self.names = dict(mu=mu_prefix, r=r_name, k=k_name, v=v_name, g=g_name, o=o_name, w1=w1_name, w2=w2_name, w0=w0_name,
                          u=u_name, norm=norm_name)
        self.decay_rank = 0         # the inner width of the decay's two matrices: read from the tensors

    def state_spec(self):
        from ..csrc.ops import Ops
        D = self.head_dim
        return {"S": StateSpec(Ops.recurrence_state_shape(self.num_heads, D, D), torch.float32),
                "shift": StateSpec((self.hidden_size,), torch.float32)}

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, N, n = self.hidden_size, self.size, self.names
        rank = max(4, E // 10)      # what the random-weights mode writes; a file may bring any
        if rank >= 64:
            rank = rank // 64 * 64
        specs = {n["mu"] + s: ParamSpec((E,), role="vector", init="around:0.5:0.25") for s in self.MIXES}
        for key in ("r", "k", "v", "g"):
            specs[n[key]] = ParamSpec((N, E))
        specs[n["w1"]] = ParamSpec((-1, E), random_shape=(rank, E))
        specs[n["w2"]] = ParamSpec((N, -1), init="normal:0.3", random_shape=(N, rank))
        # decays between 0.2 and 0.95 or so: a state that is kept for some tens of tokens, not for one and not for ever
        specs[n["w0"]] = ParamSpec((N,), role="vector", init="around:-1.5:0.8")
        specs[n["u"]] = ParamSpec((self.num_heads, self.head_dim), role="vector", init="normal:0.5")
        specs[n["norm"]] = ParamSpec((N,), role="vector", init="ones_jitter")
        specs[n["o"]] = ParamSpec((E, N))
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        n = self.names
        w1, w2 = tensors[n["w1"]], tensors[n["w2"]]
        if w1.shape[0] != w2.shape[1]:
            raise ValueError(f"wkv time mixing: the decay's matrices {tuple(w1.shape)} and {tuple(w2.shape)} do not meet")
        self.decay_rank = rank = int(w1.shape[0])
        self.mu = torch.stack([tensors[n["mu"] + s].float() for s in self.MIXES]).contiguous()
        # r, k, v and the gate read a mix each: four products of the full width, each by the kernel a projection gets
        self.w_rkvg = [rt.ops.pack_weight(tensors[n[key]].contiguous()) for key in ("r", "k", "v", "g")]
        if rank % 8:        # the inner side in whole groups of 8 (what the matrix cores take): rows and columns of
            pad = 8 - rank % 8      # zeros, whose tanh is zero and adds nothing
            w1 = torch.cat([w1, w1.new_zeros((pad, w1.shape[1]))], dim=0)
            w2 = torch.cat([w2, w2.new_zeros((w2.shape[0], pad))], dim=1)
        self.w1, self.w2 = rt.ops.pack_weight(w1.contiguous()), rt.ops.pack_weight(w2.contiguous())
        self.w0 = tensors[n["w0"]].float().contiguous()
        self.u = tensors[n["u"]].float().contiguous()
        self.w_norm = tensors[n["norm"]].float().contiguous()
        self.w_out = rt.ops.pack_weight(tensors[n["o"]])

    def _read_out(self, ctx, cache, h):
        ops, dt = self.rt.ops, self.rt.dtype
        E, N, H, D = self.hidden_size, self.size, self.num_heads, self.head_dim
        if h.dtype != torch.float32:        # (a norm that rounds its rows: the mixes are then of the rounded rows)
            h = ops.convert(h.contiguous(), torch.float32)
        T = h.shape[0]
        mixes = ops.token_shift(h, self.mu, cache.states["mixer.shift"], ctx, dt)          # [T, 5 E]: r, k, v, g, w
        proj = torch.empty((T, 4 * N), dtype=torch.float32, device=h.device)
        for s, w in enumerate(self.w_rkvg):
            ops.linear(mixes[:, s * E:(s + 1) * E], w, out=proj[:, s * N:(s + 1) * N])
        r, k, v, gate = proj[:, :N], proj[:, N:2 * N], proj[:, 2 * N:3 * N], proj[:, 3 * N:]
        inner = ops.linear(mixes[:, 4 * E:], self.w1, out_dtype=torch.float32)
        x = ops.linear(ops.act_rows(inner, "tanh", dt), self.w2, bias=self.w0, out_dtype=torch.float32)
        o = ops.linear_recurrence("wkv", r, k, v, cache.states["mixer.S"], ctx, H, H, D, D, gate=x, decay=self.u)
        return ops.gated_rmsnorm(o, gate, self.w_norm, H, D, self.eps, dt)

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out)

    def forward_f32(self, ctx, cache, h):
        return self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out_dtype=torch.float32)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._read_out(ctx, cache, h), self.w_out, out=residual, accumulate=True)


register_mixer("retention", Retention)
register_mixer("wkv_time_mix", TimeMixWKV)
register_mixer("gated_delta", GatedDelta)
register_mixer("gated_linear_attention", GatedLinearAttention)
