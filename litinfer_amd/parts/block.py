"""The pre-norm arrangement of a layer's parts
(src/llaisys/models/qwen2.cpp:272-317): x += mixer(norm1(x)); x += ffn(norm2(x)).
A layer may lack the feed-forward (and its norm).  The residual stream x is float32; mixer and feed-forward add into it through
the `ResidualStream` they are given."""
from __future__ import annotations

import torch

from .base import Block, build_part, register_part


class PreNormBlock(Block):
    def __init__(self, spec, rt, parts):
        super().__init__(spec, rt)
        self.norm1 = build_part("norm", parts["norm1"], rt)
        self.mixer = build_part("mixer", parts["mixer"], rt)
        self.norm2 = self.ffn = None
        if parts.get("feed_forward") is not None:
            self.norm2 = build_part("norm", parts["norm2"], rt)
            self.ffn = build_part("feed_forward", parts["feed_forward"], rt)
        self._all = tuple(p for p in (self.norm1, self.mixer, self.norm2, self.ffn) if p is not None)

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._all)

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_needs(self):
        needs = super().batch_needs()
        for p in self._all:
            needs = needs.merged(p.batch_needs())
        return needs

    def expected_params(self):
        e = {}
        for p in self._all:
            e.update(p.expected_params())
        return e

    def load_params(self, get):
        for p in self._all:
            p.load_params(get)

    def first_norm(self):
        return self.norm1

    def forward(self, stream, ctx, cache):
        xn = ctx.ws.buffer("block.xn", stream.shape, self.rt.dtype)
        after = stream.next_norm                   # the norm that reads the stream after this block
        stream.next_norm = self.norm2 if self.ffn is not None else after
        self.mixer.forward_prenorm(self.norm1, stream, xn, ctx, cache)
        if self.ffn is not None:
            stream.next_norm = after
            self.ffn.forward_prenorm(self.norm2, stream, xn, ctx)
        stream.next_norm = None


class SandwichBlock(Block):
    """A norm before AND behind each sublayer: x += norm1b(mixer(norm1(x))), then, if the layer has a
    feed-forward, x += norm2b(ffn(norm2(x))), then, if it has one, the layer's token input
    (`parts/token_side.py`).  A sublayer writes into a branch buffer; the kernel that norms and adds it
    also leaves the norm through which the stream is read next, where that is known.
    The norms BEFORE the sublayers may be absent (no `norm1` / `norm2` among the parts): x += norm1b(mixer(x)),
    x += norm2b(ffn(x)); the sublayers then read the stream itself, rounded to the parts' dtype."""

    def __init__(self, spec, rt, parts):
        super().__init__(spec, rt)
        self.norm1 = build_part("norm", parts["norm1"], rt) if parts.get("norm1") is not None else None
        self.mixer = build_part("mixer", parts["mixer"], rt)
        self.norm1b = build_part("norm", parts["norm1b"], rt)
        self.ffn = self.norm2 = self.norm2b = self.token_input = None
        if parts.get("feed_forward") is not None:
            self.norm2 = build_part("norm", parts["norm2"], rt) if parts.get("norm2") is not None else None
            self.ffn = build_part("feed_forward", parts["feed_forward"], rt)
            self.norm2b = build_part("norm", parts["norm2b"], rt)
        if parts.get("token_input") is not None:
            self.token_input = build_part("token_input", parts["token_input"], rt)
        self._all = tuple(p for p in (self.norm1, self.mixer, self.norm1b, self.norm2, self.ffn, self.norm2b,
                                      self.token_input) if p is not None)

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._all)

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_needs(self):
        needs = super().batch_needs()
        for p in self._all:
            needs = needs.merged(p.batch_needs())
        return needs

    def expected_params(self):
        e = {}
        for p in self._all:
            e.update(p.expected_params())
        return e

    def load_params(self, get):
        for p in self._all:
            p.load_params(get)

    def first_norm(self):
        return self.norm1

    @property
    def reads_stream_itself(self):
        """True if the block's first reader takes the residual sum without a norm."""
        return self.norm1 is None

    def _read(self, stream, norm, ctx):
        buf = ctx.ws.buffer("block.xn", stream.shape, self.rt.dtype)
        return stream.normed(norm, buf) if norm is not None else stream.rounded(buf)

    def forward(self, stream, ctx, cache):
        from .stream import BranchStream
        after, after_plain = stream.next_norm, stream.next_plain      # who reads the stream after this block
        stream.next_norm, stream.next_plain = None, False
        xn = self._read(stream, self.norm1, ctx)
        y = ctx.ws.buffer("block.branch", stream.shape, torch.float32)
        branch = BranchStream(y, ctx.ws)
        self.mixer.forward(xn, branch, ctx, cache)
        last = self.ffn is None and self.token_input is None
        if self.ffn is not None:
            stream.add_normed(self.norm1b, branch, self.norm2, next_plain=self.norm2 is None)
            xn = self._read(stream, self.norm2, ctx)
            branch = BranchStream(y, ctx.ws)
            self.ffn.forward(xn, branch, ctx)
            last = self.token_input is None
            stream.add_normed(self.norm2b, branch, after if last else None, next_plain=last and after_plain)
        else:
            stream.add_normed(self.norm1b, branch, after if last else None, next_plain=last and after_plain)
        if self.token_input is not None:
            self.token_input.forward(stream, ctx, after)


class ParallelBlock(Block):
    """One norm, two readers: with h = norm1(x), x += mixer(h) + ffn(h).  Both sublayers add into the stream through
    their last product (32-bit adds); a layer may lack the feed-forward."""

    def __init__(self, spec, rt, parts):
        super().__init__(spec, rt)
        self.norm1 = build_part("norm", parts["norm1"], rt)
        self.mixer = build_part("mixer", parts["mixer"], rt)
        self.ffn = build_part("feed_forward", parts["feed_forward"], rt) if parts.get("feed_forward") is not None else None
        self._all = tuple(p for p in (self.norm1, self.mixer, self.ffn) if p is not None)

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._all)

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_needs(self):
        needs = super().batch_needs()
        for p in self._all:
            needs = needs.merged(p.batch_needs())
        return needs

    def expected_params(self):
        e = {}
        for p in self._all:
            e.update(p.expected_params())
        return e

    def load_params(self, get):
        for p in self._all:
            p.load_params(get)

    def first_norm(self):
        return self.norm1

    def forward(self, stream, ctx, cache):
        after = stream.next_norm                   # the norm that reads the stream after this block
        stream.next_norm = None                    # (between the two sublayers nobody reads the sum)
        # the normed rows must outlive the mixer: the feed-forward reads them too
        h = stream.normed(self.norm1, ctx.ws.buffer("block.xn", stream.shape, self.rt.dtype))
        self.mixer.forward(h, stream, ctx, cache)
        if self.ffn is not None:
            stream.next_norm = after
            self.ffn.forward(h, stream, ctx)
        stream.next_norm = None


register_part("block", "prenorm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "sandwich", SandwichBlock)
