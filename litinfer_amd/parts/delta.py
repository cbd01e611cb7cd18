"""A gated delta-rule mixer: a matrix state of fixed size per request that every token first decays, then corrects
towards its own value, then reads.

With H heads of `vdim` columns and G groups of q/k heads of `dim` columns (head h uses group h // (H / G)):
q = Wq xn and k = Wk xn (G x dim), v = Wv xn (H x vdim), no biases.  Each of q, k, v passes a causal convolution per
channel over the last `conv` tokens (no bias, zeros before a request's start), then silu.  q and k become unit vectors
per head (x / sqrt(sum x^2 + 1e-6)); q is also multiplied by dim^(-1/2).  beta = sigmoid(Wb xn) and
g = exp(-exp(A_log) * softplus(Wa xn + dt_bias)), one number a head each.  Per head, with S of dim x vdim values:
    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q      (the read-out sees the token's own write).
Each head's o is RMS-normed over vdim (weights `norm` [vdim], shared by the heads), multiplied by silu(Wg xn) and
projected back by Wo.

A request keeps two states in its slot, both float32 and zero at admission: the dim x vdim matrices of all heads, and
the last conv - 1 inputs of the convolution.  The projections run in the engine's dtype with a float32 result; the
convolution, the unit vectors, beta, the decays, the recurrence and the norm are float32 in both engine dtypes.
One packed product gives a token's row [gate: H vdim | v: H vdim | k: G dim | q: G dim | b: H | a: H].
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, Mixer, StateNeed, register_part
from .linear import Linear


class GatedDeltaMixer(Mixer):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.heads = int(a["num_heads"])
        self.groups = int(a.get("num_kv_heads") or self.heads)
        self.dim = int(a["head_dim"])
        self.vdim = int(a.get("value_dim") or self.dim)
        self.taps = int(a.get("conv") or 1)
        self.eps = float(a.get("eps", 1e-6))
        if min(self.heads, self.groups, self.dim, self.vdim, self.taps) <= 0:
            raise ValueError("gated delta: sizes must be positive")
        if self.heads % self.groups:
            raise ValueError(f"gated delta: {self.heads} heads are not a multiple of {self.groups} q/k heads")
        if self.dim > 256 or self.taps > 64:
            raise ValueError("gated delta: the kernels take states of at most 256 values a column and at most 64 taps")
        self.inner = self.heads * self.vdim
        self.n_qk = self.groups * self.dim
        self.channels = self.inner + 2 * self.n_qk                       # what passes the convolution: v, k, q
        self.n_proj = 2 * self.inner + 2 * self.n_qk + 2 * self.heads
        self.names = {"q": "q", "k": "k", "v": "v", "conv_suffix": ".conv", "beta": "b", "a": "a", "a_log": "A_log",
                      "dt_bias": "dt_bias", "norm": "norm", "gate": "g", "out": "o", **(a.get("names") or {})}
        self.proj = self.out = self.conv_w = self.dt_bias = self.a_log = self.norm_w = None

    def cache_need(self):
        need = [StateNeed((self.heads, self.dim, self.vdim), torch.float32, name="delta")]
        if self.taps > 1:
            need.append(StateNeed((self.taps - 1, self.channels), torch.float32, name="conv"))
        return tuple(need)

    def batch_needs(self):
        return BatchNeeds(row_tile=self.proj.row_tile() if self.proj is not None else 1)

    def expected_params(self):
        p, n = self.prefix, self.names
        e = {p + n["gate"]: ParamSpec((self.inner, self.hidden)), p + n["out"]: ParamSpec((self.hidden, self.inner)),
             p + n["beta"]: ParamSpec((self.heads, self.hidden)), p + n["a"]: ParamSpec((self.heads, self.hidden)),
             p + n["a_log"]: ParamSpec((self.heads,)), p + n["dt_bias"]: ParamSpec((self.heads,)),
             p + n["norm"]: ParamSpec((self.vdim,), init="one_plus_normal")}
        for x, rows in (("q", self.n_qk), ("k", self.n_qk), ("v", self.inner)):
            e[p + n[x]] = ParamSpec((rows, self.hidden))
            e[p + n[x] + n["conv_suffix"]] = ParamSpec((rows, self.taps))
        return e

    def load_params(self, get):
        p, n = self.prefix, self.names
        ws = [get(p + n[x]) for x in ("gate", "v", "k", "q", "beta", "a")]
        dt = torch.float32 if any(w.dtype is torch.float32 for w in ws) else ws[0].dtype
        self.proj = Linear(self.rt, torch.cat([w.to(dt) for w in ws], dim=0))
        self.out = Linear(self.rt, get(p + n["out"]))
        self.conv_w = self.rt.vector(torch.cat([get(p + n[x] + n["conv_suffix"]).to(torch.float32) for x in ("v", "k", "q")], dim=0))
        self.dt_bias = self.rt.vector(get(p + n["dt_bias"]))
        self.a_log = self.rt.vector(get(p + n["a_log"]))
        self.norm_w = self.rt.vector(get(p + n["norm"]).to(torch.float32).repeat(self.heads))      # the same weights for every head

    def forward(self, xn, residual, ctx, cache):
        t, inner = xn.shape[0], self.inner
        proj = ctx.ws.buffer("delta.proj32", (t, self.n_proj), torch.float32)
        self.proj(xn, proj, ws=ctx.ws)
        state = cache.states["delta"]
        vkq = ctx.ws.buffer("delta.vkq", (t, self.channels), torch.float32)
        tail = cache.states["conv"] if self.taps > 1 else state.view(state.shape[0], 1, -1)
        ops.causal_conv_silu(proj[:, inner:inner + self.channels], self.conv_w, None, tail, ctx, vkq)
        y = ctx.ws.buffer("delta.y", (t, inner), torch.float32)
        ops.delta_scan(vkq, proj[:, inner + self.channels:], self.dt_bias, self.a_log, state, ctx, y, self.heads, self.vdim,
                       self.dim, self.groups, self.dim ** -0.5, ws=ctx.ws)
        g = ctx.ws.buffer("delta.gated", (t, inner), self.rt.dtype)
        ops.gated_group_norm(y, proj[:, :inner], self.norm_w, self.eps, self.heads, g, gate_after=True)
        residual.add_linear(self.out, g)


register_part("mixer", "gated_delta", GatedDeltaMixer)
