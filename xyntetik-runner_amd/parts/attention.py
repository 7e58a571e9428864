"""Grouped-query attention over the paged cache.

Per token: ``q = Wq h``, ``k = Wk h``, ``v = Wv h`` (optional biases); the position
encoding rotates q and k; k and v go to the cache (k rotated, v as it is); query head
``h`` reads key/value head ``h // (H / Hk)``; scores are ``(q . k) * scale`` with
``scale = 1/sqrt(head_dim)`` unless given, causal by construction, limited to the last
``window`` keys if the layer has a window; softmax in 32-bit; ``a = Wo o``
(src/model.c:6243-6338, ``attn_heads`` :3548-3589, window bound :6326).

The three input projections are kept as one ``[Q + 2K, E]`` matrix.  A layer that
reads another layer's cache (``kv_shared``) has no key or value projection and writes
nothing (src/model.h:492-494).

Options that other designs bring: ``values="keys"``: there is no value projection and the values are the
keys as projected (before any transform of queries and keys: the cache then holds the transformed keys
and, as values, the untransformed ones); ``slopes``: one number a query head, ``slopes[h] * (i - j)`` is
taken off the score of query i and key j, a bias that grows with the distance and stands in for a position
encoding; ``weight_suffix`` / ``bias_suffix``: how a checkpoint names a projection's matrix and bias;
``v_head_dim``: values of another size than the keys; ``chunk``: instead of a window, a position reads the keys
of its own chunk of so many positions (chunks counted from position 0 of the sequence, whatever portions it was
run in); ``keep_first``: with a window, the first so many keys stay readable, at their true positions;
``sink``: the softmax's denominator holds one entry more, without key or value: "learned" (a score a head, the
tensor ``sink_name``, unscaled) or "zero" (the score 0: one is added to the denominator); ``gate_name``: a
projection ``[H, E]`` of the mixer's input whose sigmoid multiplies every head's output before the output
projection.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import KVSpec, Mixer, ParamSpec, make_part, register_mixer

MAX_HEAD_DIM = 256      # the attention and rotation kernels keep a head's channels in registers up to this size


class PagedAttention(Mixer):
    takes_unscaled_rows = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position=None, window: Optional[int] = None, scale: Optional[float] = None,
                 bias: bool = False, out_bias: Optional[bool] = None, kv_shared: bool = False, qk_transform=None,
                 q_name: str = "q_proj", k_name: str = "k_proj", v_name: str = "v_proj",
                 o_name: str = "o_proj", values: str = "projection", slopes=None, weight_suffix: str = ".weight",
                 bias_suffix: str = ".bias", v_head_dim: Optional[int] = None, chunk: Optional[int] = None,
                 keep_first: int = 0, sink: Optional[str] = None, sink_name: str = "sink", gate_name: Optional[str] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        if window is not None and window < 1:
            raise ValueError(f"attention window {window} must be at least 1")
        if not (1 <= int(head_dim) <= MAX_HEAD_DIM):
            # refused when the model is built, not at its first step
            raise ValueError(f"attention head size {head_dim} is outside what the attention kernels take (1 to {MAX_HEAD_DIM})")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.num_kv_heads, self.head_dim = int(num_kv_heads), int(head_dim)
        self.window = int(window) if window is not None else None
        self.chunk = int(chunk) if chunk is not None else None
        if self.chunk is not None and (self.chunk < 1 or self.window is not None):
            raise ValueError(f"attention: a chunk of {chunk} positions (at least 1, and no window beside it)")
        self.keep_first = int(keep_first)
        if self.keep_first < 0 or (self.keep_first and self.window is None):
            raise ValueError(f"attention: {keep_first} kept first keys need a window that would pass them")
        if sink not in (None, "learned", "zero"):
            raise ValueError(f"attention: sink {sink!r} (learned, zero or none)")
        self.sink, self.sink_name, self.gate_name = sink, sink_name, gate_name
        self.v_head_dim = int(v_head_dim) if v_head_dim is not None else int(head_dim)
        if not (1 <= self.v_head_dim <= MAX_HEAD_DIM):
            raise ValueError(f"attention value size {v_head_dim} is outside what the attention kernels take (1 to {MAX_HEAD_DIM})")
        if self.v_head_dim != int(head_dim) and values == "keys":
            raise ValueError("attention: values that are the keys have the keys' size")
        self.sinks = self.w_gate = None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.bias = bool(bias)
        self.out_bias = self.bias if out_bias is None else bool(out_bias)
        self.kv_shared = bool(kv_shared)
        if values not in ("projection", "keys"):
            raise ValueError(f"attention: values come from their 'projection' or are the 'keys', not {values!r}")
        self.values_are_keys = values == "keys"
        if slopes is not None and len(slopes) != int(num_heads):
            raise ValueError(f"attention: {len(slopes)} slopes for {num_heads} query heads")
        self.slope_values = [float(s) for s in slopes] if slopes is not None else None
        self.w_sfx, self.b_sfx = weight_suffix, bias_suffix
        self.slopes = None
        self.names = (q_name, k_name, v_name, o_name)
        self.position = make_part("position", position) if position is not None else None
        # applied to the 32-bit projections before the position encoding; with one, the projections
        # are written out and the kernels that rotate and cache their own result are not used
        self.qk_transform = make_part("qk_transform", qk_transform) if qk_transform is not None else None
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.v_size = self.num_kv_heads * self.v_head_dim
        self.w_in = self.b_in = self.w_out = self.b_out = None

    # what the cache manager must keep
    def kv_spec(self) -> Optional[KVSpec]:
        # a chunk never reaches further back than its length: its pages are kept as a window's of that length are
        reach = self.chunk if self.chunk is not None else self.window
        return KVSpec(self.num_kv_heads, self.head_dim, reach,
                      v_head_dim=self.v_head_dim if self.v_head_dim != self.head_dim else None, keep_first=self.keep_first)

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, Q, K, V = self.hidden_size, self.q_size, self.kv_size, self.v_size
        q, k, v, o = self.names
        ws, bs = self.w_sfx, self.b_sfx
        specs = {f"{q}{ws}": ParamSpec((Q, E)), f"{o}{ws}": ParamSpec((E, self.num_heads * self.v_head_dim))}
        if not self.kv_shared:
            specs[f"{k}{ws}"] = ParamSpec((K, E))
            if not self.values_are_keys:
                specs[f"{v}{ws}"] = ParamSpec((V, E))
        if self.bias:
            specs[f"{q}{bs}"] = ParamSpec((Q,), role="vector", init="normal")
            if not self.kv_shared:
                specs[f"{k}{bs}"] = ParamSpec((K,), role="vector", init="normal")
                if not self.values_are_keys:
                    specs[f"{v}{bs}"] = ParamSpec((V,), role="vector", init="normal")
        if self.sink == "learned":      # of the size of a score: a sink that no key outweighs, or that none feels, shows nothing
            specs[self.sink_name] = ParamSpec((self.num_heads,), role="vector", init="normal:1.0")
        if self.gate_name is not None:
            specs[f"{self.gate_name}{ws}"] = ParamSpec((self.num_heads, E), init="normal:0.1")
        if self.out_bias:
            specs[f"{o}{bs}"] = ParamSpec((E,), role="vector", init="normal")
        if self.qk_transform is not None:
            for name, ps in self.qk_transform.param_specs().items():
                if name in specs:
                    raise ValueError(f"the query/key transform names a tensor {name!r} that the attention has itself")
                specs[name] = ps
        return specs

    @property
    def capturable(self) -> bool:
        return ((self.position is None or self.position.capturable)
                and (self.qk_transform is None or self.qk_transform.capturable))

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        if self.position is not None:
            self.position.bind({}, rt)
        if self.qk_transform is not None:
            self.qk_transform.bind({n: tensors[n] for n in self.qk_transform.param_specs()}, rt)
        q, k, v, o = self.names
        H, Hk, D = self.num_heads, self.num_kv_heads, self.head_dim
        ws, bsf = self.w_sfx, self.b_sfx
        if self.values_are_keys:        # the value projection is the key projection: its rows stand twice in the one matrix
            v = k
        mats = [tensors[f"{q}{ws}"]]
        if not self.kv_shared:
            mats += [tensors[f"{k}{ws}"], tensors[f"{v}{ws}"]]
        w_in = torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else mats[0]
        b_in = None
        if self.bias:
            bs = [tensors[f"{q}{bsf}"]]
            if not self.kv_shared:
                bs += [tensors[f"{k}{bsf}"], tensors[f"{v}{bsf}"]]
            b_in = torch.cat([b.float() for b in bs]).contiguous()
        if self.slope_values is not None:
            self.slopes = torch.tensor(self.slope_values, dtype=torch.float32, device=rt.device)
        if self.sink == "learned":
            self.sinks = tensors[self.sink_name].float().contiguous()
        elif self.sink == "zero":
            self.sinks = torch.zeros((H,), dtype=torch.float32, device=rt.device)
        if self.gate_name is not None:
            self.w_gate = rt.ops.pack_weight(tensors[f"{self.gate_name}{ws}"].contiguous())
        # A rotation that pairs channel j with j + rot/2: the rows of every query and key head go
        # in paired order, so that the product's kernel has both halves of a pair at hand when
        # it rotates its own result (a few decoded tokens); the rotation kernel reads that order too.
        rot = self.position.rotary() if self.position is not None else None
        self.paired = (rot is not None and not rot.interleaved and rot.rotary_dim % 16 == 0 and D % 16 == 0
                       and self.qk_transform is None      # (a transform sees channels in the checkpoint's order)
                       and self.v_head_dim == D)          # (values of another size go through the plain store)
        if self.paired:
            from ..csrc.ops import paired_order
            order = paired_order(D, rot.rotary_dim)
            heads = H + (0 if self.kv_shared else Hk)
            rows = [h * D + c for h in range(heads) for c in order] + list(range(heads * D, w_in.shape[0]))
            index = torch.tensor(rows, dtype=torch.int64, device=w_in.device)
            w_in = w_in.index_select(0, index)
            if b_in is not None:
                b_in = b_in.index_select(0, index)
        self.w_in, self.b_in = rt.ops.pack_weight(w_in), b_in
        self.w_out = rt.ops.pack_weight(tensors[f"{o}{ws}"])
        if self.out_bias:
            self.b_out = tensors[f"{o}{bsf}"].float().contiguous()

    def _attend(self, ctx, cache, h):
        ops, rt = self.rt.ops, self.rt
        Q, K, H, Hk, D = self.q_size, self.kv_size, self.num_heads, self.num_kv_heads, self.head_dim
        Dv, V = self.v_head_dim, self.v_size
        T = h.shape[0]
        writes = not self.kv_shared and cache.owns
        rot = self.position.rotary() if self.position is not None else None
        table = ctx.block_table(cache.group)
        gate = ops.linear(h, self.w_gate, out_dtype=torch.float32) if self.w_gate is not None else None
        if Dv != D:
            # values of another size than the keys: the transforms and the rotation in place on the 32-bit
            # projections, then the store that takes both sizes
            if rot is not None and (rot.interleaved or rot.mscale != 1.0):
                raise ValueError("attention with values of another size rotates channel j with j + dims/2 by a plain table")
            proj = ops.linear(h, self.w_in, bias=self.b_in, out_dtype=torch.float32)
            q_in = proj[:, :Q]
            k_in = proj[:, Q:Q + K] if writes else None
            v_in = proj[:, Q + K:Q + K + V] if writes else None
            if self.qk_transform is not None:
                self.qk_transform.apply(ctx, q_in.unflatten(1, (H, D)), k_in.unflatten(1, (Hk, D)) if writes else None)
            if self.position is not None and rot is None:
                self.position.apply(ctx, q_in.unflatten(1, (H, D)), k_in.unflatten(1, (Hk, D)) if writes else None)
            if rot is not None:
                ops.rotate_rows_(q_in, ctx.positions, rot.inv_freq, H, D, rot.rotary_dim, 1.0)
                if writes:
                    ops.rotate_rows_(k_in, ctx.positions, rot.inv_freq, Hk, D, rot.rotary_dim, 1.0)
            q = ops.qkv_store(q_in, k_in, v_in, cache.k, cache.v, ctx, cache.group, H, Hk, D, Dv, cache.page_size, rt.dtype)
        elif (self.position is None or rot is not None) and writes == (not self.kv_shared) and self.qk_transform is None:
            q = ops.project_rope_kv_write(
                h, self.w_in, self.b_in, cache.k if writes else None, cache.v if writes else None, ctx.positions,
                ctx.req_of_token, table, rot.inv_freq if rot else None, H, Hk if writes else 0, D,
                rot.rotary_dim if rot else 0, rot.interleaved if rot else False, rot.mscale if rot else 1.0,
                cache.page_size, paired=self.paired, cs_table=(lambda: self._step_table(ctx, rot)) if rot else None)
        else:
            # a transform or a position encoding of its own works on the 32-bit queries and keys before
            # they are cached; or the keys and values this layer computes are another layer's to store
            proj = ops.linear(h, self.w_in, bias=self.b_in, out_dtype=torch.float32)
            q_in = proj[:, :Q]
            k_in = proj[:, Q:Q + K] if writes else None
            v_in = proj[:, Q + K:Q + 2 * K] if writes else None
            if self.qk_transform is not None:
                self.qk_transform.apply(ctx, q_in.unflatten(1, (H, D)), k_in.unflatten(1, (Hk, D)) if writes else None)
            if self.position is not None and rot is None:
                self.position.apply(ctx, q_in.unflatten(1, (H, D)), k_in.unflatten(1, (Hk, D)) if writes else None)
            q = torch.empty((T, Q), dtype=rt.dtype, device=h.device)
            ops.rope_kv_write(q_in, k_in, v_in, q, cache.k if writes else None, cache.v if writes else None,
                              ctx.positions, ctx.req_of_token, table,
                              rot.inv_freq if rot else None, H, Hk if writes else 0, D,
                              rot.rotary_dim if rot else 0, rot.interleaved if rot else False,
                              rot.mscale if rot else 1.0, cache.page_size, paired=self.paired)
        o = ops.attention(q, cache.k, cache.v, ctx, cache.group, H, Hk, D, cache.page_size, self.scale,
                          self.window, slopes=self.slopes, chunk=self.chunk, keep_first=self.keep_first, sinks=self.sinks,
                          v_head_dim=Dv)
        if gate is not None:
            ops.head_gate_(o, gate, H, Dv)
        return o

    def _step_table(self, ctx, rot):
        """The step's cosines and sines for this rotation, made once and shared by every layer
        that rotates by the same table (a step context keeps what its parts leave in ``shared``)."""
        shared = getattr(ctx, "shared", None)
        if shared is None:
            return self.rt.ops.rope_table(ctx.positions, rot.inv_freq, rot.mscale)
        key = ("rope_table", rot.table_key if rot.table_key is not None else rot.inv_freq.data_ptr(), rot.mscale)
        table = shared.get(key)
        if table is None:
            table = shared[key] = self.rt.ops.rope_table(ctx.positions, rot.inv_freq, rot.mscale)
        return table

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, bias=self.b_out)

    def forward_f32(self, ctx, cache, h):
        return self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, bias=self.b_out, out_dtype=torch.float32)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, bias=self.b_out, out=residual, accumulate=True)

    def forward_add_norm(self, ctx, cache, h, residual, norm, defer=False):
        fold = norm.fold()
        if fold is None:
            return super().forward_add_norm(ctx, cache, h, residual, norm, defer)
        return self.rt.ops.linear_add_rmsnorm(self._attend(ctx, cache, h), self.w_out, residual, fold[0], fold[1],
                                              self.rt.dtype, bias=self.b_out, defer=defer)


register_mixer("paged_attention", PagedAttention)
