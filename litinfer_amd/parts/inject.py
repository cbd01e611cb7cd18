"""Additions to the residual stream BETWEEN layers, named by entries of the execution order.

`LoopEntry`: where a run of layers is passed several times with the same weights, the stream takes, right
before the first layer of pass t, the embedding output again (not before the first pass) and the t-th row
of a table [passes, width].  The embedding output is gathered again from the table rather than kept.

`LoopMix`: before every pass the stream becomes a product of one matrix with the stream and the embedding output
side by side."""
from __future__ import annotations

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Part, register_part


class LoopEntry(Part):
    category = "injection"
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.times = int(spec.args["times"])
        self.hidden = int(spec.args["hidden_size"])
        self.param = self.prefix + str(spec.args.get("param", "step"))
        self.add_embedding = bool(spec.args.get("add_embedding", True))
        self.steps = None

    def expected_params(self):
        return {self.param: ParamSpec((self.times, self.hidden))}

    def load_params(self, get):
        self.steps = self.rt.vector(get(self.param))

    def forward(self, stream, ctx, index: int, embedding) -> None:
        if not 0 <= index < self.times:
            raise IndexError(f"loop entry: pass {index} of {self.times}")
        x = stream.tensor()
        table = embedding.table if (self.add_embedding and index > 0) else None
        ops.embedding_add(x, ctx.ids, table, self.steps[index], ctx.id_src, ctx.feedback)


class LoopMix(Part):
    """Before every pass of a repeated run of layers (the first too) the stream becomes W [x ; x0]: a product of
    the matrix `param` [width, 2 width] with the stream and the embedding output side by side (the stream first).
    The model keeps the embedding output for it (`keeps_embedding_output`).  The two halves are rounded to the
    engine's dtype side by side in one buffer, the product writes the float32 stream."""
    category = "injection"
    graph_safe = True
    keeps_embedding_output = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.times = int(spec.args["times"])
        self.hidden = int(spec.args["hidden_size"])
        self.param = self.prefix + str(spec.args.get("param", "in"))
        self.proj = None

    def expected_params(self):
        return {self.param: ParamSpec((self.hidden, 2 * self.hidden))}

    def load_params(self, get):
        from .linear import Linear
        self.proj = Linear(self.rt, get(self.param))

    def batch_needs(self):
        from .base import BatchNeeds
        return BatchNeeds(row_tile=self.proj.row_tile() if self.proj is not None else 1)

    def forward(self, stream, ctx, index: int, embedding) -> None:
        if not 0 <= index < self.times:
            raise IndexError(f"loop entry: pass {index} of {self.times}")
        if ctx.embedding_out is None:
            raise ValueError("loop entry: the model has not kept the embedding output")
        x = stream.tensor()
        both = ctx.ws.buffer("loop.both", (x.shape[0], 2 * self.hidden), self.rt.dtype)
        ops.concat_rows(x, ctx.embedding_out, both)
        self.proj(both, x, ws=ctx.ws)


register_part("injection", "loop_entry", LoopEntry)
register_part("injection", "loop_mix", LoopMix)
