"""A retention mixer: linear attention with a fixed decay a head, no softmax and no denominator, whose state has a
fixed size per request.

q = Wq xn and k = Wk xn (heads x dim), v = Wv xn (heads x vdim), no biases.  q and k are encoded by the position part
(v is not); k is multiplied by dim^(-1/2) after that.  Per head, with S of dim x vdim values:
    S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
with decay_h from the list `decay`.  Each head's o is divided by its root mean square (no weights), the heads side by
side are multiplied by silu(Wg xn) and projected back by Wo.

A request keeps the dim x vdim matrices of all heads in its slot, float32 and zero at admission.  The projections run in
the engine's dtype with a float32 result; the rotation, the recurrence and the norm are float32 in both engine dtypes.
The recurrence is the state-space recurrence's kernel with the same decay and the same step (dim^(-1/2)) for every
token: k is its B, q its C, v its x.  One packed product gives a token's row [gate: H vdim | v: H vdim | k: H dim | q: H dim].
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, Mixer, StateNeed, build_part, register_part
from .linear import Linear


class RetentionMixer(Mixer):

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.heads = int(a["num_heads"])
        self.dim = int(a["head_dim"])
        self.vdim = int(a.get("value_dim") or self.dim)
        self.eps = float(a.get("eps", 1e-6))
        self.decay = tuple(float(d) for d in a["decay"])
        if min(self.heads, self.dim, self.vdim) <= 0:
            raise ValueError("retention: sizes must be positive")
        if len(self.decay) != self.heads:
            raise ValueError(f"retention: {len(self.decay)} decays for {self.heads} heads")
        if self.dim > 256:
            raise ValueError("retention: the kernels take states of at most 256 values a column")
        self.position = build_part("position", a["position"], rt) if a.get("position") else None
        self.state_name = str(a.get("state_name") or "retention")
        self.inner = self.heads * self.vdim
        self.n_qk = self.heads * self.dim
        self.n_proj = 2 * self.inner + 2 * self.n_qk
        self.names = {"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", **(a.get("names") or {})}
        self.proj = self.out = self.decay_dev = None

    @property
    def graph_safe(self):
        return self.position is None or self.position.graph_safe

    def cache_need(self):
        return StateNeed((self.heads, self.dim, self.vdim), torch.float32, name=self.state_name)

    def batch_needs(self):
        return BatchNeeds(row_tile=self.proj.row_tile() if self.proj is not None else 1)

    def expected_params(self):
        p, n = self.prefix, self.names
        return {p + n["q"]: ParamSpec((self.n_qk, self.hidden)), p + n["k"]: ParamSpec((self.n_qk, self.hidden)),
                p + n["v"]: ParamSpec((self.inner, self.hidden)), p + n["gate"]: ParamSpec((self.inner, self.hidden)),
                p + n["out"]: ParamSpec((self.hidden, self.inner))}

    def load_params(self, get):
        p, n = self.prefix, self.names
        ws = [get(p + n[x]) for x in ("gate", "v", "k", "q")]
        dt = torch.float32 if any(w.dtype is torch.float32 for w in ws) else ws[0].dtype
        self.proj = Linear(self.rt, torch.cat([w.to(dt) for w in ws], dim=0))
        self.out = Linear(self.rt, get(p + n["out"]))
        self.decay_dev = self.rt.vector(torch.tensor(self.decay, dtype=torch.float32))

    def forward(self, xn, residual, ctx, cache):
        t, inner = xn.shape[0], self.inner
        proj = ctx.ws.buffer("retention.proj32", (t, self.n_proj), torch.float32)
        self.proj(xn, proj, ws=ctx.ws)
        if self.position is not None:
            self.position.apply(proj[:, 2 * inner:], 2 * self.heads, self.dim, ctx)       # k and q heads, in place
        y = ctx.ws.buffer("retention.y", (t, inner), torch.float32)
        ops.ssm_scan(proj[:, inner:], None, None, None, None, cache.states[self.state_name], ctx, y, self.heads, self.vdim,
                     self.dim, self.heads, ctx.ws, fixed_decay=self.decay_dev, fixed_step=self.dim ** -0.5)
        g = ctx.ws.buffer("retention.gated", (t, inner), self.rt.dtype)
        ops.gated_group_norm(y, proj[:, :inner], None, self.eps, self.heads, g, gate_after=True)
        residual.add_linear(self.out, g)


register_part("mixer", "retention", RetentionMixer)
