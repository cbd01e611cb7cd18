"""Token embedding and the output head.

Embedding: x[t, :] = E[ids[t], :], a row copy without scaling
(src/ops/embedding/op.cpp:32-40), written into the float32 residual stream.
Head: logits = xf Wout^T without bias (src/llaisys/models/qwen2.cpp:337), as
float32; when tied, Wout is the embedding table itself (one buffer), and so it
is when the configuration says untied but the checkpoint holds no head matrix
(python/llaisys/models/qwen2.py:196-199).

Options that other designs use: the embedding may add a sinusoidal position vector
(`sinusoid_base` b: column 2i gets sin(p b^(-2i/H)), column 2i+1 the cosine of the same
angle; the frequencies are worked out once in float64 and rounded to float32, the angle is
float(p) * f in float32); the head may scale its logits (`logit_scale`) and cap them
(`softcap` c: c * tanh(logits / c)), in that order.  `PairHashEmbedding` adds a row of a second, hashed table
that the token and its predecessor choose together."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Part, register_part
from .linear import Linear


class TokenEmbedding(Part):
    graph_safe = True

    category = "embedding"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab = int(spec.args["vocab_size"])
        self.hidden = int(spec.args["hidden_size"])
        self.param = self.prefix + str(spec.args.get("param", "weight"))
        self.sinusoid_base = float(spec.args.get("sinusoid_base") or 0.0)
        if self.sinusoid_base < 0:
            raise ValueError("embedding: the base of the position vector must be positive")
        self.table = None
        self.freq = None

    def expected_params(self):
        return {self.param: ParamSpec((self.vocab, self.hidden))}

    def load_params(self, get):
        self.table = self.rt.matrix(get(self.param))
        if self.sinusoid_base:
            i = torch.arange((self.hidden + 1) // 2, dtype=torch.float64)
            self.freq = self.rt.vector(torch.pow(torch.tensor(self.sinusoid_base, dtype=torch.float64), -2.0 * i / self.hidden))

    def cache_need(self):
        """Per-request state that the embedding keeps (none here); see `Mixer.cache_need`."""
        return None

    def forward(self, ids, out, id_src=None, feedback=None, positions=None, ctx=None, cache=None):
        ops.embedding(ids, self.table, out, id_src, feedback)
        if self.freq is not None:
            if positions is None:
                raise ValueError("embedding: the position vector needs the tokens' positions")
            ops.sinusoid_add(out, positions, self.freq)
        return out


class PairHashEmbedding(TokenEmbedding):
    """The token's row plus a row of a second table that is chosen by the token AND the one before it in its
    request: row (previous * mul_prev + token * mul_cur) mod buckets of `pair_param` [buckets + 1, hidden], and the
    table's last row for a request's first token.  The token before a step's first one is per-request state: one
    int32 a state slot, kept up to date by the kernel that gathers (so tokens chosen on the device count too)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.buckets, self.mul_prev, self.mul_cur = int(a["buckets"]), int(a["mul_prev"]), int(a["mul_cur"])
        if self.buckets <= 0 or self.mul_prev < 0 or self.mul_cur < 0:
            raise ValueError("pair embedding: buckets must be positive and the multipliers not negative")
        if (self.vocab - 1) * (self.mul_prev + self.mul_cur) >= 1 << 62:
            raise ValueError("pair embedding: the multipliers are too large for 64-bit sums")
        self.pair_param = self.prefix + str(a.get("pair_param", "bigram"))
        self.pair = None

    def cache_need(self):
        from .base import StateNeed
        return StateNeed((1,), torch.int32, "last_token")

    def expected_params(self):
        return {**super().expected_params(), self.pair_param: ParamSpec((self.buckets + 1, self.hidden))}

    def load_params(self, get):
        super().load_params(get)
        self.pair = self.rt.matrix(get(self.pair_param))
        if self.pair.dtype is not self.table.dtype:
            self.pair = self.pair.to(self.table.dtype)

    def forward(self, ids, out, id_src=None, feedback=None, positions=None, ctx=None, cache=None):
        if ctx is None or cache is None or cache.state is None:
            raise ValueError("pair embedding: needs the step's segments and its state (the requests' last tokens)")
        ops.pair_embedding(ids, self.table, self.pair, out, ctx.positions, ctx.seg_of_token, ctx.q_start, ctx.q_len,
                           ctx.state_slots, cache.state.view(-1), self.buckets, self.mul_prev, self.mul_cur, id_src, feedback)
        if self.freq is not None:
            ops.sinusoid_add(out, ctx.positions, self.freq)
        return out


class LinearHead(Part):
    graph_safe = True

    category = "head"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab = int(spec.args["vocab_size"])
        self.hidden = int(spec.args["hidden_size"])
        self.tied_to = spec.args.get("tied_to")
        # untied by the configuration, but no matrix stored: use the table, as the reference does
        self.tie_if_absent = bool(spec.args.get("tie_if_absent", False))
        self.param = self.prefix + str(spec.args.get("param", "weight"))
        self.logit_scale = float(spec.args.get("logit_scale") if spec.args.get("logit_scale") is not None else 1.0)
        self.softcap = float(spec.args.get("softcap") or 0.0)
        if self.softcap < 0:
            raise ValueError("head: the cap of the logits must not be negative")
        self.proj = None

    def expected_params(self):
        if self.tied_to:
            return {}
        return {self.param: ParamSpec((self.vocab, self.hidden), required=not self.tie_if_absent)}

    def load_params(self, get, tied_table=None):
        """`tied_table` is the embedding's table as the model holds it."""
        w = None if self.tied_to else get(self.param)
        if w is None:
            if tied_table is None:
                raise ValueError("head: tied to the embedding, but no table was given")
            if not self.tied_to and hasattr(get, "note"):
                get.note(f"{self.param} is not stored: the head uses the embedding table")
            self.proj = Linear(self.rt, tied_table)
        else:
            self.proj = Linear(self.rt, w)

    def forward(self, xn, out, ws):
        self.proj(xn, out, ws=ws)
        if self.logit_scale != 1.0 or self.softcap:
            ops.scale_softcap(out, self.logit_scale, self.softcap)
        return out


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("embedding", "pair_hash_embedding", PairHashEmbedding)
register_part("head", "linear_head", LinearHead)
