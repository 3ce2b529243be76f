"""Arrangement of a layer: pre-norm residual block
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
(reference: src/graph_builder.cpp:1195, :1366-1374, :1396, :1443). Each
residual add is carried as pending and fused into the next norm, or, with few
rows, done by the last product of the mixer / feed-forward, which then also prepares
the rows of the norm that follows (parts.base.ResidualSink).

residual_scale m (1 unless given): x = x + m * mixer(norm1(x)); x = x + m * feed_forward(norm2(x)).
A layer without a feed-forward (feed_forward None) is the first line alone.

The "post_norm" block norms what a branch returns and nothing it reads:
    x = x + m * norm1(mixer(x));  x = x + m * norm2(feed_forward(x))."""
from __future__ import annotations

import torch

from .base import (Block, BuildEnv, LayerCache, PartSpec, ResidualStream, StepContext,
                   build_part, param, register_part)


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        names = param(params, "names", dict)
        self.mixer_norm = build_part("norm", param(params, "mixer_norm", PartSpec),
                                     prefix + names["mixer_norm"] + ".", env)
        self.mixer = build_part("mixer", param(params, "mixer", PartSpec),
                                prefix + names["mixer"] + ".", env)
        self.residual_scale = param(params, "residual_scale", float, 1.0)
        self.ff_norm = self.feed_forward = None
        if param(params, "feed_forward", PartSpec, None) is not None:
            self.ff_norm = build_part("norm", param(params, "feed_forward_norm", PartSpec),
                                      prefix + names["feed_forward_norm"] + ".", env)
            self.feed_forward = build_part("feed_forward", param(params, "feed_forward", PartSpec),
                                           prefix + names["feed_forward"] + ".", env)

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward) if p is not None]

    def first_norm(self):
        return self.mixer_norm

    def tensor_specs(self):
        specs = {}
        for c in self.children():
            specs.update(c.tensor_specs())
        return specs

    def bind(self, tensors):
        for c in self.children():
            c.bind(tensors)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        after = ctx.next_norm                  # reads the stream once this block is done
        m = self.residual_scale
        n = stream.normed(self.mixer_norm, ctx, self.mixer.accepts_normed_rows)
        ctx.sink = stream.sink_for(self.ff_norm if self.feed_forward is not None else after, ctx, m)
        delta = self.mixer.forward(n, ctx, cache)
        ctx.sink = None
        stream.add(delta, ctx, m)
        if self.feed_forward is None:
            return
        n = stream.normed(self.ff_norm, ctx, self.feed_forward.accepts_normed_rows)
        ctx.sink = stream.sink_for(after, ctx, m)
        delta = self.feed_forward.forward(n, ctx)
        ctx.sink = None
        stream.add(delta, ctx, m)


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    """A layer whose branches are normed on both sides of the residual sum:
        x = x + post1(mixer(pre1(x)));  x = x + post2(feed_forward(pre2(x)))
    and, where the layer has one, a token input behind them: x = x + postT(token_input(x, token)),
    which reads the stream itself (in the activation dtype) and not a norm of it. A layer without a
    feed-forward is the first line (and the token input) alone.

    Every sum is one launch where the norms around it are RMS norms with a gain: the branch output
    is normed and added in fp32, and the same launch forms what the next reader wants of the new
    stream (the next pre-norm, the plain rows for the token input, or the first norm of the block
    that follows). Other norms go through their own add_norm on a 32-bit copy of the branch output.

    names: mixer_norm, mixer_post_norm, mixer, feed_forward_norm, feed_forward_post_norm,
    feed_forward, token_input (suffixes of the parts' prefixes)."""

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        names = param(params, "names", dict)

        def norm(key):
            return build_part("norm", param(params, key, PartSpec), prefix + names[key] + ".", env)

        self.mixer_norm = norm("mixer_norm")
        self.mixer_post = norm("mixer_post_norm")
        self.mixer = build_part("mixer", param(params, "mixer", PartSpec), prefix + names["mixer"] + ".", env)
        self.ff_norm = self.ff_post = self.feed_forward = self.token_input = None
        if param(params, "feed_forward", PartSpec, None) is not None:
            self.ff_norm = norm("feed_forward_norm")
            self.ff_post = norm("feed_forward_post_norm")
            self.feed_forward = build_part("feed_forward", param(params, "feed_forward", PartSpec),
                                           prefix + names["feed_forward"] + ".", env)
        if param(params, "token_input", PartSpec, None) is not None:
            self.token_input = build_part("token_input", param(params, "token_input", PartSpec),
                                          prefix + names["token_input"] + ".", env)

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_post, self.ff_norm, self.feed_forward,
                            self.ff_post, self.token_input) if p is not None]

    def first_norm(self):
        return self.mixer_norm

    def tensor_specs(self):
        specs = {}
        for c in self.children():
            specs.update(c.tensor_specs())
        return specs

    def bind(self, tensors):
        for c in self.children():
            c.bind(tensors)

    @staticmethod
    def _rms(norm):
        """(gain, eps) of a norm that is a plain RMS norm with a gain, else None."""
        c = norm.carried() if norm is not None else None
        return c if c is not None and len(c) == 2 else None

    def _join(self, stream: ResidualStream, delta, post, reader, ctx: StepContext):
        """stream += post(delta); returns what `reader` wants of the new stream: reader a Norm -> its
        normed rows, "rows" -> the stream in the activation dtype, None -> nothing."""
        from ..kernels import ops
        rows = stream.rows
        resid = stream.materialize(ctx)
        stream.prepared = stream.ready = None
        post_c = post if isinstance(post, tuple) else self._rms(post)
        read_c = self._rms(reader) if reader is not None and reader != "rows" else None
        if post_c is not None and (reader is None or reader == "rows" or read_c is not None):
            out = None if reader is None else ctx.alloc((rows, resid.shape[-1]))
            ops.add_normed(resid, delta, post_c[0], post_c[1], read_c[0] if read_c else None,
                           read_c[1] if read_c else 0.0, out, rows)
            return out
        # any other norm: the branch output through the norm's own kernel on a 32-bit copy, then the sum
        copy = ctx.alloc((rows, resid.shape[-1]), torch.float32)
        copy[:rows].copy_(delta[:rows])
        normed = post.add_norm(copy, None, rows, ctx)
        ops.residual_add(resid, normed, rows)
        if reader is None:
            return None
        if reader == "rows":
            out = ctx.alloc((rows, resid.shape[-1]))
            out[:rows].copy_(resid[:rows])
            return out
        return reader.add_norm(resid, None, rows, ctx)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        after = ctx.next_norm                  # reads the stream once this block is done
        ctx.sink = None
        n = stream.normed(self.mixer_norm, ctx)
        delta = self.mixer.forward(n, ctx, cache)
        # who reads the stream after each sum
        tail = "rows" if self.token_input is not None else after
        n = self._join(stream, delta, self.mixer_post, self.ff_norm if self.feed_forward is not None else tail, ctx)
        if self.feed_forward is not None:
            delta = self.feed_forward.forward(n, ctx)
            n = self._join(stream, delta, self.ff_post, tail, ctx)
        if self.token_input is not None:
            delta = self.token_input.forward(n, ctx)
            post = self.token_input.post_norm()
            if post is None:
                stream.add(delta, ctx)
                return
            n = self._join(stream, delta, post, after, ctx)
        if after is not None and n is not None:
            stream.ready = (after, n)


@register_part("block", "post_norm")
class PostNormBlock(Block):
    """A layer whose branches read the stream itself (in the activation dtype) and are normed on their way
    back into it:  x = x + m * norm1(mixer(x));  x = x + m * norm2(feed_forward(x)), with m = residual_scale
    (1 unless given). A layer without a feed-forward is the first line alone.

    Each sum is one launch where the norm has add_normed_delta (the grouped RMS norm): the branch output is
    normed and added in fp32, and the same launch writes the new stream's rows in the activation dtype for the
    branch that reads them next. Other norms go through their own add_norm on a 32-bit copy of the branch output.
    names: mixer_norm, mixer, feed_forward_norm, feed_forward (suffixes of the parts' prefixes)."""

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        names = param(params, "names", dict)
        self.mixer_norm = build_part("norm", param(params, "mixer_norm", PartSpec),
                                     prefix + names["mixer_norm"] + ".", env)
        self.mixer = build_part("mixer", param(params, "mixer", PartSpec), prefix + names["mixer"] + ".", env)
        self.residual_scale = param(params, "residual_scale", float, 1.0)
        self.ff_norm = self.feed_forward = None
        if param(params, "feed_forward", PartSpec, None) is not None:
            self.ff_norm = build_part("norm", param(params, "feed_forward_norm", PartSpec),
                                      prefix + names["feed_forward_norm"] + ".", env)
            self.feed_forward = build_part("feed_forward", param(params, "feed_forward", PartSpec),
                                           prefix + names["feed_forward"] + ".", env)

    def children(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward) if p is not None]

    def tensor_specs(self):
        specs = {}
        for c in self.children():
            specs.update(c.tensor_specs())
        return specs

    def bind(self, tensors):
        for c in self.children():
            c.bind(tensors)

    def _rows(self, stream: ResidualStream, ctx: StepContext):
        """The stream as it stands, in the activation dtype."""
        from ..kernels import ops
        resid = stream.materialize(ctx)
        out = ctx.alloc((stream.rows, resid.shape[-1]))
        ops.add_group_normed(resid, None, None, 1, 0.0, 1.0, out, stream.rows)
        return out

    def _join(self, stream: ResidualStream, delta, norm, want_rows: bool, ctx: StepContext):
        """stream += m * norm(delta); returns the new stream's rows in the activation dtype when asked."""
        from ..kernels import ops
        rows = stream.rows
        resid = stream.materialize(ctx)
        stream.prepared = stream.ready = None
        out = ctx.alloc((rows, resid.shape[-1])) if want_rows else None
        if hasattr(norm, "add_normed_delta"):
            norm.add_normed_delta(resid, delta, rows, self.residual_scale, out)
            return out
        copy = ctx.alloc((rows, resid.shape[-1]), torch.float32)
        copy[:rows].copy_(delta[:rows])
        normed = norm.add_norm(copy, None, rows, ctx)
        ops.residual_add(resid, normed, rows, self.residual_scale)
        if want_rows:
            out[:rows].copy_(resid[:rows])
        return out

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        ctx.sink = None
        delta = self.mixer.forward(self._rows(stream, ctx), ctx, cache)
        x = self._join(stream, delta, self.mixer_norm, self.feed_forward is not None, ctx)
        if self.feed_forward is not None:
            delta = self.feed_forward.forward(x, ctx)
            self._join(stream, delta, self.ff_norm, False, ctx)
