"""Arrangements of a layer's parts around the 32-bit residual stream.

"prenorm": ``x += mixer(norm(x)); x += feed_forward(norm(x))`` — norm, projections,
rotation, cache write, attention, output, add, norm, feed-forward, add, every layer
alike (src/model.c:6168-6473).

"prenorm_filtered": the same, but what each sublayer reads goes through a sequence filter first:
``x += mixer(filter_m(norm(x))); x += feed_forward(filter_f(norm(x)))``.  A layer of it may come
without a feed-forward.

"prenorm_streams": the pre-norm layer over ``S`` copies ``x_1 .. x_S`` of the residual stream
("hyper-connections").  A sublayer with connection weights ``in [S]``, ``out [S]`` and ``mix [S, S]``
(indexed ``[from, to]``) reads ``u = sum_s in[s] x_s`` through its norm, and its result ``y`` goes back as
``x_t <- sum_s mix[s, t] x_s + out[t] y`` for all ``t`` at once, from the old copies.  ``x`` is then
``[S, T, E]``; the model makes the copies after the embedding and adds them up before the final norm.
The write of one sublayer and the read and norm of the next run in one kernel.

"sandwich": every sublayer is normed before and after, and what it adds is scaled:
``x += m post_m(mixer(pre_m(x))); x += m post_f(feed_forward(pre_f(x)))`` with one number ``m`` for the
layer.  A layer of it may come without a feed-forward.  Where all four norms are dynamic tanh, which
takes no statistic of a row, the second norm of one sublayer, the scaled sum and the first norm of
the next are one element-wise pass.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Block, Connection, ParamSpec, register_block, register_connection


def _takes_unscaled(part) -> bool:
    return bool(getattr(part, "takes_unscaled_rows", False))


class PreNormBlock(Block):
    chained = True
    norm_names = ("mixer_norm", "feed_forward_norm")

    @property
    def mixer_norm(self):
        return self.norms["mixer_norm"]

    @property
    def feed_forward_norm(self):
        return self.norms["feed_forward_norm"]

    def entry_norm(self):
        return self.mixer_norm, _takes_unscaled(self.mixer)

    def forward(self, ctx, cache, x, h=None, after=None):
        """``h``: the result of ``mixer_norm`` if the block before made it.  ``after``: the next
        block's ``entry_norm()``, whose result is then returned.  The parts' optional
        ``forward_add_norm`` is used where they have it."""
        if h is None:
            h = self.mixer_norm.forward(ctx, x)
        add_norm = getattr(self.mixer, "forward_add_norm", None)
        if add_norm is not None:
            h = add_norm(ctx, cache, h, x, self.feed_forward_norm, defer=_takes_unscaled(self.feed_forward))
        else:
            self.mixer.forward_add(ctx, cache, h, x)
            h = self.feed_forward_norm.forward(ctx, x)
        add_norm = getattr(self.feed_forward, "forward_add_norm", None)
        if after is None or add_norm is None:
            self.feed_forward.forward_add(ctx, h, x)
            return None
        next_norm, defer = after
        return add_norm(ctx, h, x, next_norm, defer=defer)


class PreNormOptionalBlock(PreNormBlock):
    """"prenorm" for a layer that may come without a feed-forward (its second norm then does nothing)."""
    needs_feed_forward = None

    def forward(self, ctx, cache, x, h=None, after=None):
        if self.feed_forward is not None:
            return super().forward(ctx, cache, x, h=h, after=after)
        if h is None:
            h = self.mixer_norm.forward(ctx, x)
        self.mixer.forward_add(ctx, cache, h, x)
        return None


class FilteredPreNormBlock(Block):
    norm_names = ("mixer_norm", "feed_forward_norm")
    filter_names = ("mixer_filter", "feed_forward_filter")
    needs_feed_forward = None       # with or without; the second norm and filter then do nothing

    def _read(self, ctx, cache, x, norm: str, flt: str):
        """What a sublayer reads: the norm of ``x`` through the filter, in one kernel if the filter has one."""
        f, state = self.filters[flt], cache.states.get(flt)
        fused = getattr(f, "forward_normed", None)
        h = fused(ctx, state, x, self.norms[norm]) if fused is not None else None
        if h is None:
            h = f.forward(ctx, state, self.norms[norm].forward(ctx, x))
        return h

    def forward(self, ctx, cache, x):
        self.mixer.forward_add(ctx, cache, self._read(ctx, cache, x, "mixer_norm", "mixer_filter"), x)
        if self.feed_forward is not None:
            self.feed_forward.forward_add(ctx, self._read(ctx, cache, x, "feed_forward_norm", "feed_forward_filter"), x)

    def state_specs(self):
        out = super().state_specs()
        if self.feed_forward is None:
            out.pop("feed_forward_filter", None)
        return out


class StreamConnection(Connection):
    """The weights by which one sublayer meets ``streams`` residual streams: ``in [S]``, ``out [S]``,
    ``mix [S, S]`` (``[from, to]``), kept in 32 bits.  With ``optional`` a file may leave them out, and
    the sublayer then reads and writes every stream alike (in = out = 1, mix = identity)."""

    def __init__(self, streams: int, in_name: str = "in", out_name: str = "out", mix_name: str = "mix", optional: bool = False):
        from ..csrc.ops import Ops
        if not (1 <= int(streams) <= Ops.MAX_STREAMS):
            raise ValueError(f"{streams} residual streams (the kernel takes 1 to {Ops.MAX_STREAMS})")
        self.streams, self.optional = int(streams), bool(optional)
        self.names = (in_name, out_name, mix_name)
        self.w_in = self.w_out = self.w_mix = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        S = self.streams
        i, o, m = self.names
        # of the size of 1, every entry its own: a weight that is transposed, swapped or left out must show
        return {i: ParamSpec((S,), role="vector", init="normal:0.7", optional=self.optional),
                o: ParamSpec((S,), role="vector", init="normal:0.7", optional=self.optional),
                m: ParamSpec((S, S), role="vector", init="normal:0.6", optional=self.optional)}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        S = self.streams
        i, o, m = self.names

        def take(name, default):
            t = tensors.get(name)
            return (t.float() if t is not None else default.to(rt.device)).contiguous()

        self.w_in = take(i, torch.ones(S))
        self.w_out = take(o, torch.ones(S))
        self.w_mix = take(m, torch.eye(S))


class StreamsEntry:
    """What the block before needs to make this block's first input: the first connection and norm."""

    def __init__(self, connection: StreamConnection, norm):
        self.connection, self.norm = connection, norm


class StreamsPreNormBlock(Block):
    chained = True
    norm_names = ("mixer_norm", "feed_forward_norm")
    connection_names = ("mixer_connection", "feed_forward_connection")
    needs_feed_forward = None       # with or without; the second norm and connection then do nothing

    def entry_norm(self):
        return StreamsEntry(self.connections["mixer_connection"], self.norms["mixer_norm"])

    def _norm_weight(self, norm):
        """(32-bit weight, eps) of an RMSNorm that the streams' kernel may apply itself; None for any other norm."""
        fold = norm.fold()
        if fold is None:
            return None
        cached = getattr(norm, "_f32_weight", None)
        if cached is None or cached[0] is not fold[0]:
            cached = norm._f32_weight = (fold[0], fold[0].float().contiguous())
        return cached[1], fold[1]

    def _step(self, ctx, xs, y, wrote: Optional[StreamConnection], reads: Optional[StreamConnection], norm):
        """Write ``y`` back through ``wrote`` and/or make the input of the sublayer behind ``reads`` and ``norm``."""
        ops, dt = ctx.ops, self.mixer.rt.dtype
        kw = {}
        if wrote is not None:
            kw.update(y=y, mix=wrote.w_mix, out_w=wrote.w_out)
        if reads is None:
            ops.streams_step(xs, **kw)
            return None
        fold = self._norm_weight(norm)
        if fold is not None:
            return ops.streams_step(xs, in_w=reads.w_in, norm_w=fold[0], eps=fold[1], h_dtype=dt, **kw)
        return norm.forward(ctx, ops.streams_step(xs, in_w=reads.w_in, **kw))

    def forward(self, ctx, cache, xs, h=None, after=None):
        """``xs [S, T, E]``; ``h``: this block's first input if the block before made it; ``after``: the
        next block's ``entry_norm()``, whose input is then returned."""
        c1, c2 = self.connections["mixer_connection"], self.connections["feed_forward_connection"]
        if xs.dim() != 3 or xs.shape[0] != c1.streams:
            raise ValueError(f"this layer mixes {c1.streams} residual streams, the model keeps {tuple(xs.shape)}")
        if h is None:
            h = self._step(ctx, xs, None, None, c1, self.norms["mixer_norm"])
        y = self.mixer.forward_f32(ctx, cache, h)
        last = c1
        if self.feed_forward is not None:
            h = self._step(ctx, xs, y, c1, c2, self.norms["feed_forward_norm"])
            y = self.feed_forward.forward_f32(ctx, h)
            last = c2
        if isinstance(after, StreamsEntry):
            return self._step(ctx, xs, y, last, after.connection, after.norm)
        self._step(ctx, xs, y, last, None, None)
        return None


class SandwichEntry:
    """What the block before needs to make this block's first input: its first norm."""

    def __init__(self, norm):
        self.norm = norm


class SandwichBlock(Block):
    chained = True
    norm_names = ("mixer_norm", "mixer_post_norm", "feed_forward_norm", "feed_forward_post_norm")
    needs_feed_forward = None       # with or without; the feed-forward's two norms then do nothing

    def __init__(self, mixer, feed_forward, norms, filters=None, connections=None, residual_mult: float = 1.0):
        super().__init__(mixer, feed_forward, norms, filters, connections)
        self.residual_mult = float(residual_mult)

    def entry_norm(self):
        return SandwichEntry(self.norms["mixer_norm"])

    def _add(self, ctx, x, y, post, nxt):
        """``x += m post(y)``, then ``nxt`` of the updated rows (None: nothing comes back).  ``y`` is 32-bit."""
        ops = ctx.ops
        if hasattr(post, "dyt") and (nxt is None or hasattr(nxt, "dyt")):
            dt = None
            if nxt is not None:
                dt = torch.float32 if getattr(nxt, "out_dtype", "compute") == "float32" else self.mixer.rt.dtype
            return ops.dyt_step(x, y=y, post=post.dyt(), mult=self.residual_mult, norm=nxt.dyt() if nxt is not None else None,
                                out_dtype=dt)
        ops.add_(x, post.forward(ctx, y).contiguous(), scale=self.residual_mult)
        return nxt.forward(ctx, x) if nxt is not None else None

    def forward(self, ctx, cache, x, h=None, after=None):
        """``h``: the result of ``mixer_norm`` if the block before made it.  ``after``: the next block's
        ``entry_norm()``; if that block is of this arrangement too, its first input is returned."""
        nxt = after.norm if isinstance(after, SandwichEntry) else None
        if h is None:
            h = self.norms["mixer_norm"].forward(ctx, x)
        y = self.mixer.forward_f32(ctx, cache, h)
        if self.feed_forward is None:
            return self._add(ctx, x, y, self.norms["mixer_post_norm"], nxt)
        h = self._add(ctx, x, y, self.norms["mixer_post_norm"], self.norms["feed_forward_norm"])
        y = self.feed_forward.forward_f32(ctx, h)
        return self._add(ctx, x, y, self.norms["feed_forward_post_norm"], nxt)


register_connection("stream_connection", StreamConnection)
register_block("sandwich", SandwichBlock)
register_block("prenorm_streams", StreamsPreNormBlock)
register_block("prenorm", PreNormBlock)
register_block("prenorm_optional", PreNormOptionalBlock)
register_block("prenorm_filtered", FilteredPreNormBlock)
