"""The residual stream of a step: a float32 tensor [T, H] that the parts of a
layer add into, in 32-bit.

Parts do not add by themselves; they ask the stream: `add_linear(linear, h)`
adds `h W^T + b` (the product kernel's epilogue does the add in 32-bit, so no
separate pass reads and writes the stream: src/llaisys/models/qwen2.cpp:287-290
does linear and add as two), `normed(norm, out)` gives the norm of the current
sum, and `tensor()` gives the sum itself for a part that adds in its own way.

Whoever knows which norm reads the stream next says so in `next_norm`.  Then
`add_linear` may, for the few rows of a decoding step, have its kernel leave the
sum times that norm's weights and the rows' sums of squares beside the sum
itself, and the part behind the norm finds them under `scaled_rows(norm)`: the
norm costs no pass of its own.  Any other write to the stream forgets them.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import ScaledRows


_PLAIN = object()         # in place of a norm: "the sum itself, in the parts' dtype"


class ResidualStream:
    def __init__(self, x: torch.Tensor, ws):
        self.x = x
        self.ws = ws
        self.next_norm = None                 # the norm through which the stream is read next, if known
        self.next_plain = False               # the next reader takes the sum itself, without a norm (known like next_norm)
        self._scaled = None                   # (norm, ScaledRows) left by the last add_linear
        self._normed = None                   # (norm, its result) left by the last add_linear
        self.ws_dtype = torch.bfloat16        # the dtype in which normed rows are handed to the parts (the model sets it)

    @property
    def shape(self):
        return self.x.shape

    def tensor(self) -> torch.Tensor:
        """The sum so far (whoever takes it may write to it)."""
        self._scaled = self._normed = None
        return self.x

    def add_linear(self, linear, h: torch.Tensor) -> None:
        """x += h W^T + b."""
        norm, self._scaled, self._normed = self.next_norm, None, None
        scaling = norm.as_scaling() if norm is not None else None
        if scaling is not None and linear.takes_scaling(h, self.x):
            rows = self.ws.buffer("stream.scaled_rows", self.x.shape, h.dtype)
            self._scaled = (norm, ScaledRows(rows, linear.add_with_scaling(h, self.x, scaling, rows, self.ws)))
            return
        if scaling is not None:
            # some more rows: where the product is cut along K, the kernel that adds the parts up norms as well
            rows = self.ws.buffer("stream.normed_rows", self.x.shape, h.dtype)
            if linear.add_then_norm(h, self.x, scaling, rows, self.ws):
                self._normed = (norm, rows)
                return
        linear(h, self.x, accumulate=True, ws=self.ws)

    def scaled_rows(self, norm) -> Optional[ScaledRows]:
        """What the last addition left for this norm's reader, if it did."""
        if self._scaled is not None and self._scaled[0] is norm:
            return self._scaled[1]
        return None

    def normed(self, norm, out: torch.Tensor) -> torch.Tensor:
        """norm(x): in `out`, or in the tensor that the last addition already left."""
        if self._normed is not None and self._normed[0] is norm:
            return self._normed[1]
        norm.forward(self.x, out)
        return out

    def rounded(self, out: torch.Tensor) -> torch.Tensor:
        """The sum itself as a sublayer without a norm of its own reads it: in the parts' dtype (in `out`, or in the
        tensor that the last addition already left); in a 32-bit engine the stream's own tensor, which a reader must
        not write to."""
        if self._normed is not None and self._normed[0] is _PLAIN:
            return self._normed[1]
        if out.dtype is self.x.dtype:
            return self.x
        from ..kernels import ops
        ops.cast(self.x, out)
        return out

    def add_normed(self, norm, y, next_norm=None, next_plain: bool = False) -> None:
        """x += norm(y) for the output y [T, H] (float32) of a sublayer that is normed BEFORE it joins the
        stream; y may be the sublayer's `BranchStream`, which can hold two outputs and their factors (the norm then
        sees factor0 * y0 + factor1 * y1).  `next_norm`: the norm through which the stream is read next, if the
        caller knows it; the same kernel then leaves that norm of the new sum, and `normed(next_norm, ...)` hands it
        out.  `next_plain`: the next reader takes the sum itself; the kernel leaves it in the parts' dtype for `rounded`."""
        from ..kernels import ops
        scaling = norm.as_scaling()
        if scaling is None:
            raise NotImplementedError("add_normed: the norm behind a sublayer must be an RMS norm with weights")
        y2, factors = None, (1.0, 1.0)
        if isinstance(y, BranchStream):
            y, y2, factors = y.outputs()
        self._scaled = self._normed = None
        nxt = next_norm.as_scaling() if next_norm is not None else None
        if nxt is None and not (next_plain and self.ws_dtype is not self.x.dtype):
            ops.rmsnorm_add(y, scaling.weight, scaling.eps, self.x, y2=y2, factors=factors)
            return
        rows = self.ws.buffer("stream.normed_rows", self.x.shape, self.ws_dtype)
        if nxt is None:
            ops.rmsnorm_add(y, scaling.weight, scaling.eps, self.x, None, 0.0, rows, y2=y2, factors=factors)
            self._normed = (_PLAIN, rows)
            return
        ops.rmsnorm_add(y, scaling.weight, scaling.eps, self.x, nxt.weight, nxt.eps, rows, y2=y2, factors=factors)
        self._normed = (next_norm, rows)


class BranchStream(ResidualStream):
    """What ONE sublayer puts out, for arrangements that treat it (norm it, gate it) before it joins the
    residual stream: the mixer or feed-forward is handed this in the stream's place, and its first
    `add_linear` writes instead of adding."""

    def __init__(self, y: torch.Tensor, ws):
        super().__init__(y, ws)
        self._fresh = True
        self.factor = 1.0                    # what this output is multiplied by when it joins
        self.second = None                   # a second output beside this one (a BranchStream with a factor of its own)

    def fork(self, name: str) -> "BranchStream":
        """A second output beside this one, for a sublayer made of two that are added with factors."""
        if self.second is not None:
            raise NotImplementedError("a branch holds at most two outputs")
        self.second = BranchStream(self.ws.buffer(name, self.x.shape, torch.float32), self.ws)
        return self.second

    def outputs(self):
        """(first output, second output or None, (factor of the first, factor of the second))."""
        if self.second is None:
            if self.factor != 1.0:
                return self.result(), self.result(), (self.factor, 0.0)
            return self.result(), None, (1.0, 1.0)
        return self.result(), self.second.result(), (self.factor, self.second.factor)

    def tensor(self) -> torch.Tensor:
        if self._fresh:
            self.x.zero_()
            self._fresh = False
        return self.x

    def add_linear(self, linear, h: torch.Tensor) -> None:
        linear(h, self.x, accumulate=not self._fresh, ws=self.ws)
        self._fresh = False

    def result(self) -> torch.Tensor:
        return self.tensor()
