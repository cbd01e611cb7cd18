"""Two attention mixers over the paged cache that share one attention kernel (`ops.masked_attention`):
a window beside which a number of first positions stay visible, scores capped by a tanh, keys and
values of unequal sizes.

`MaskedAttention`: grouped-query attention.  q = xn Wq^T, k = xn Wk^T, v = xn Wv^T (one packed
product, left in float32); optionally an RMS norm over the WHOLE of q and the whole of k (all heads
at once, before the split into heads); the position encoding on the first columns of every query and
key head; score = (q . k) * scale, then cap * tanh(score / cap) where a cap is given; the query at
position p sees the keys j <= p with p - j < window (0: all) or j < keep_first; softmax; Wo on the
heads side by side.  Options: biases on q, k and v (`bias`; the tensor's name with `bias_suffix` added); a SINK a
head (`sink`): the softmax's denominator also holds exp(sink_h), a learned number without key or value; a sigmoid
gate a head (`head_gate`): head h's output is multiplied by sigmoid(Wg xn)_h before Wo; the position part says how
it pairs columns (`layout`: neighbouring ones, or column i with column i + rotary_dim/2).

`LatentAttention`: keys and values are expanded from one latent vector c per token, c = the RMS
norm of the first `rank` rows of Wd xn; the other `rot_dim` rows of Wd xn, rotated, are a key part
that all heads share.  Head h has key [Wuk_h c | shared part] and value Wuv_h c, and a query of
`dim` plain and `rot_dim` rotated columns.  Only c and the shared part are cached.  The expansion is
never carried out per key: q_h . (Wuk_h c) = (Wuk_h^T q_h) . c, and sum_j p_j Wuv_h c_j =
Wuv_h (sum_j p_j c_j), so the attention runs over the cached rows themselves, one kv head of
rank + rot_dim key columns whose first `rank` are also the value, with a per-head product before
(queries into the latent space) and one after it (the summed latent into the head's value space).
Options: the queries may go through a latent of their own (`q_rank` > 0: c_q = RMS norm of Wdq xn with weights
`q_down_norm`, q = Wuq c_q); every head's output may be multiplied by a sigmoid gate of the mixer's input
(`head_gate`: sigmoid(Wg xn)_h, one row of Wg a head); the position part says how it pairs columns (`layout`:
neighbouring ones, or column i with column i + rot_dim/2).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, Mixer, PagedNeed, PagedTensor, build_part, register_part
from .linear import Linear


class MaskedAttention(Mixer):

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.nh = int(a["num_heads"])
        self.nkv = int(a.get("num_kv_heads") or self.nh)
        self.dk = int(a["head_dim"])
        self.dv = int(a.get("value_dim") or self.dk)
        self.window = int(a.get("window") or 0)
        self.keep_first = int(a.get("keep_first") or 0) if self.window else 0
        self.softcap = float(a.get("softcap") or 0.0)
        self.scale = float(a["scale"]) if a.get("scale") is not None else self.dk ** -0.5
        self.qk_norm = bool(a.get("qk_norm", False))
        self.eps = float(a.get("eps", 1e-6))
        self.bias = bool(a.get("bias", False))
        self.has_sink = bool(a.get("sink", False))
        self.head_gate = bool(a.get("head_gate", False))
        self.gate_cols = -(-int(a["num_heads"]) // 4) * 4 if self.head_gate else 0
        if self.nh <= 0 or self.nkv <= 0 or self.nh % self.nkv:
            raise ValueError(f"attention: {self.nh} heads are not a multiple of {self.nkv} kv heads")
        if self.softcap < 0 or self.window < 0 or self.keep_first < 0:
            raise ValueError("attention: the cap, the window and the kept first positions must not be negative")
        self.position = build_part("position", a["position"], rt) if a.get("position") else None
        self.rotary_dim = int(getattr(self.position, "rotary_dim", 0)) if self.position is not None else 0
        self.half_split = getattr(self.position, "layout", "pairs") == "half"
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "bias_suffix": ".b",
                      "sink": "sink", "gate": "g", **(a.get("names") or {})}
        self.n_q, self.n_k, self.n_v = self.nh * self.dk, self.nkv * self.dk, self.nkv * self.dv
        self.qkv = self.out = self.wq = self.wk = self.sink = None

    @property
    def graph_safe(self):
        return self.position is None or self.position.graph_safe

    def cache_need(self):
        return PagedNeed((PagedTensor("k", (self.nkv, self.dk)), PagedTensor("v", (self.nkv, self.dv))),
                         self.window, self.keep_first)

    def batch_needs(self):
        # the kernels take single-token segments and the others (tiles of queries) apart
        return BatchNeeds(tile_rows=ops.MASKED_TILE_ROWS, token_kinds=True,
                          row_tile=self.qkv.row_tile() if self.qkv is not None else 1)

    def expected_params(self):
        p, n = self.prefix, self.names
        e = {p + n["q"]: ParamSpec((self.n_q, self.hidden)), p + n["k"]: ParamSpec((self.n_k, self.hidden)),
             p + n["v"]: ParamSpec((self.n_v, self.hidden)), p + n["o"]: ParamSpec((self.hidden, self.nh * self.dv))}
        if self.qk_norm:
            e[p + n["q_norm"]] = ParamSpec((self.n_q,), init="one_plus_normal")
            e[p + n["k_norm"]] = ParamSpec((self.n_k,), init="one_plus_normal")
        if self.bias:
            for x, size in (("q", self.n_q), ("k", self.n_k), ("v", self.n_v)):
                e[p + n[x] + n["bias_suffix"]] = ParamSpec((size,), init="normal")
        if self.has_sink:
            e[p + n["sink"]] = ParamSpec((self.nh,), init="normal")
        if self.head_gate:
            e[p + n["gate"]] = ParamSpec((self.nh, self.hidden))
        return e

    def load_params(self, get):
        p, n = self.prefix, self.names
        ws = [get(p + n[x]) for x in "qkv"]
        if self.head_gate:                  # the gates' rows ride behind q, k and v in the one packed product
            g = get(p + n["gate"])         # (with rows of zeros up to a multiple of four, so that a token's row keeps 16-byte pieces)
            ws.append(torch.cat([g, g.new_zeros(self.gate_cols - self.nh, self.hidden)], dim=0))
        dt = torch.float32 if any(w.dtype is torch.float32 for w in ws) else ws[0].dtype
        bias = None
        if self.bias:
            bs = [get(p + n[x] + n["bias_suffix"]).to(torch.float32) for x in "qkv"]
            bias = torch.cat(bs + ([bs[0].new_zeros(self.gate_cols)] if self.head_gate else []))
        self.qkv = Linear(self.rt, torch.cat([w.to(dt) for w in ws], dim=0), bias)
        self.out = Linear(self.rt, get(p + n["o"]))
        if self.has_sink:
            self.sink = self.rt.vector(get(p + n["sink"]))
        if self.qk_norm:
            self.wq, self.wk = self.rt.vector(get(p + n["q_norm"])), self.rt.vector(get(p + n["k_norm"]))

    def forward(self, xn, residual, ctx, cache):
        t = xn.shape[0]
        n_qkv = self.n_q + self.n_k + self.n_v
        qkv = ctx.ws.buffer("attn.qkv32", (t, n_qkv + self.gate_cols), torch.float32)
        self.qkv(xn, qkv, ws=ctx.ws)
        if self.position is not None:
            cos, sin = self.position.tables(ctx)
        else:
            cos = sin = ctx.ws.buffer("attn.no_tables", (t, 0), torch.float32)
        # norm over the whole projections, rotation, and the write of keys and values to their pages: one kernel
        ops.qk_norm_pairs_store(qkv, self.nh, self.nkv, self.dk, self.dv, self.rotary_dim, self.wq, self.wk, self.eps,
                                cos, sin, ctx.slot_map(cache.group) if cache.owned else None,
                                cache.k if cache.owned else None, cache.v if cache.owned else None, cache.page_size,
                                half_split=self.half_split)
        attn = ctx.ws.buffer("attn.out", (t, self.nh * self.dv), self.rt.dtype)
        ops.masked_attention(qkv, qkv.stride(0), self.dk, attn, cache.k, cache.v, ctx.attention_meta(cache.group),
                             self.nh, self.nkv, self.dk, self.dv, cache.page_size, self.window, self.keep_first,
                             self.softcap, self.scale, ws=ctx.ws, sink=self.sink,
                             head_gate=qkv[:, n_qkv:n_qkv + self.nh] if self.head_gate else None)
        residual.add_linear(self.out, attn)


class LatentAttention(Mixer):

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.nh = int(a["num_heads"])
        self.dn = int(a["head_dim"])                 # plain (unrotated) query/key columns of a head
        self.dr = int(a["rot_dim"])                  # rotated columns
        self.dv = int(a.get("value_dim") or self.dn)
        self.rank = int(a["kv_rank"])
        self.q_rank = int(a.get("q_rank") or 0)      # 0: the queries are one product of the input
        self.head_gate = bool(a.get("head_gate", False))
        self.window = int(a.get("window") or 0)
        self.keep_first = int(a.get("keep_first") or 0) if self.window else 0
        self.softcap = float(a.get("softcap") or 0.0)
        self.scale = float(a["scale"]) if a.get("scale") is not None else (self.dn + self.dr) ** -0.5
        self.eps = float(a.get("eps", 1e-6))
        if min(self.nh, self.dn, self.dv, self.rank) <= 0 or self.dr <= 0 or self.dr % 2 or self.q_rank < 0:
            raise ValueError("latent attention: sizes must be positive and the rotated size even")
        self.position = build_part("position", a["position"], rt)
        if int(getattr(self.position, "rotary_dim", self.dr)) != self.dr:
            raise ValueError("latent attention: the position encoding must rotate the whole rotated part")
        self.half_split = getattr(self.position, "layout", "pairs") == "half"
        self.names = {"q": "q", "q_down": "dq", "q_down_norm": "dq.norm", "q_up": "uq", "down": "dkv", "down_norm": "dkv.norm",
                      "up_k": "uk", "up_v": "uv", "gate": "g", "o": "o", **(a.get("names") or {})}
        self.n_q = self.nh * (self.dn + self.dr)
        self.q_down = self.q_up = self.out = self.wc = self.wq = self.to_latent = self.from_latent = None

    @property
    def graph_safe(self):
        return self.position.graph_safe

    def cache_need(self):
        # one row a token: the latent, then the shared rotated key part
        return PagedNeed((PagedTensor("latent", (1, self.rank + self.dr)),), self.window, self.keep_first)

    def batch_needs(self):
        return BatchNeeds(tile_rows=ops.MASKED_TILE_ROWS, token_kinds=True,
                          row_tile=self.q_down.row_tile() if self.q_down is not None else 1)

    def expected_params(self):
        p, n = self.prefix, self.names
        e = {p + n["down"]: ParamSpec((self.rank + self.dr, self.hidden)),
             p + n["down_norm"]: ParamSpec((self.rank,), init="one_plus_normal"),
             p + n["up_k"]: ParamSpec((self.nh * self.dn, self.rank)),
             p + n["up_v"]: ParamSpec((self.nh * self.dv, self.rank)),
             p + n["o"]: ParamSpec((self.hidden, self.nh * self.dv))}
        if self.q_rank:
            e[p + n["q_down"]] = ParamSpec((self.q_rank, self.hidden))
            e[p + n["q_down_norm"]] = ParamSpec((self.q_rank,), init="one_plus_normal")
            e[p + n["q_up"]] = ParamSpec((self.n_q, self.q_rank))
        else:
            e[p + n["q"]] = ParamSpec((self.n_q, self.hidden))
        if self.head_gate:
            e[p + n["gate"]] = ParamSpec((self.nh, self.hidden))
        return e

    def load_params(self, get):
        p, n = self.prefix, self.names
        # ONE product of the mixer's input: [queries, or their latent | latent and shared key part | gates]
        first = [get(p + n["q_down"] if self.q_rank else p + n["q"]), get(p + n["down"])]
        if self.head_gate:
            first.append(get(p + n["gate"]))
        dt = torch.float32 if any(w.dtype is torch.float32 for w in first) else first[0].dtype
        self.q_down = Linear(self.rt, torch.cat([w.to(dt) for w in first], dim=0))
        if self.q_rank:
            self.wq = self.rt.vector(get(p + n["q_down_norm"]))
            self.q_up = Linear(self.rt, get(p + n["q_up"]))
        self.wc = self.rt.vector(get(p + n["down_norm"]))
        # per head: queries into the latent space (Wuk_h^T, [rank, dn]) and the summed latent out of it (Wuv_h, [dv, rank])
        uk = get(p + n["up_k"]).reshape(self.nh, self.dn, self.rank).transpose(1, 2).contiguous()
        self.to_latent = self.rt.matrix(uk)
        self.from_latent = self.rt.matrix(get(p + n["up_v"]).reshape(self.nh, self.dv, self.rank).contiguous())
        self.out = Linear(self.rt, get(p + n["o"]))

    def forward(self, xn, residual, ctx, cache):
        t, nh, dn, dr, rank = xn.shape[0], self.nh, self.dn, self.dr, self.rank
        n_first = self.q_rank or self.n_q
        qd = ctx.ws.buffer("latent.qd32", (t, n_first + rank + dr + (nh if self.head_gate else 0)), torch.float32)
        self.q_down(xn, qd, ws=ctx.ws)
        cos, sin = self.position.tables(ctx)
        rows = cache.tensors["latent"]
        slots = ctx.slot_map(cache.group) if cache.owned else None
        qfull = ctx.ws.buffer("latent.q", (t, nh, rank + dr), torch.float32)
        down = qd[:, n_first:n_first + rank + dr]
        if self.q_rank:
            # the norm of the queries' latent, the norm of the keys' latent, the rotation of the shared key part and the
            # page write: one kernel; then the queries themselves, whose rotated parts the per-head product rotates
            # on their way behind its outputs
            cq = ctx.ws.buffer("latent.cq", (t, self.q_rank), self.rt.dtype)
            ops.latent_norm_pairs_store(None, 0, dn, dr, rank, self.wc, self.eps, cos, sin, slots, rows if cache.owned else None,
                                        None, down=down, half_split=self.half_split, q_latent=qd[:, :self.q_rank], wq=self.wq, cq=cq)
            q = ctx.ws.buffer("latent.q32", (t, self.n_q), torch.float32)
            self.q_up(cq, q, ws=ctx.ws)
            ops.headwise_linear(q, q.stride(0), dn + dr, self.to_latent, qfull, nh * (rank + dr), rank + dr, t,
                                rotate_tail=(dr, cos, sin, self.half_split))
        else:
            q = qd
            ops.latent_norm_pairs_store(qd, nh, dn, dr, rank, self.wc, self.eps, cos, sin, slots, rows if cache.owned else None,
                                        qfull, half_split=self.half_split)
            ops.headwise_linear(q, q.stride(0), dn + dr, self.to_latent, qfull, nh * (rank + dr), rank + dr, t)
        summed = ctx.ws.buffer("latent.summed", (t, nh * rank), self.rt.dtype)
        ops.masked_attention(qfull, nh * (rank + dr), rank + dr, summed, rows, rows, ctx.attention_meta(cache.group),
                             nh, 1, rank + dr, rank, cache.page_size, self.window, self.keep_first, self.softcap, self.scale,
                             ws=ctx.ws)
        heads = ctx.ws.buffer("attn.out", (t, nh * self.dv), self.rt.dtype)
        gate = qd[:, n_first + rank + dr:] if self.head_gate else None
        ops.headwise_linear(summed, nh * rank, rank, self.from_latent, heads, nh * self.dv, self.dv, t, gate=gate)
        residual.add_linear(self.out, heads)


register_part("mixer", "masked_attention", MaskedAttention)
register_part("mixer", "latent_attention", LatentAttention)
