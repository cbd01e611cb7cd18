"""Dense SwiGLU feed-forward: y = (up * gate / (1 + exp(-gate))) Wd^T with
gate = xn Wg^T, up = xn Wu^T, no biases (src/llaisys/models/qwen2.cpp:744-759,
src/ops/swiglu/op.cpp:19-22).  Gate and up are one product with the packed
matrix [Wg; Wu]; the result is added to the residual stream.  With `activation` = "gelu_tanh" the gate passes the
tanh form of GELU instead: y = (up * gelu_tanh(gate)) Wd^T; the tensors' names behind the prefix are parameters
(`names`)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, FeedForward, register_part
from .linear import Linear


class SwiGLUMLP(FeedForward):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec.args["hidden_size"])
        self.inter = int(spec.args["intermediate_size"])
        self.activation = str(spec.args.get("activation") or "silu")
        if self.activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"gated feed-forward: activation {self.activation!r} (silu or gelu_tanh)")
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight", **(spec.args.get("names") or {})}
        self.gate_up = None
        self.down = None

    def expected_params(self):
        p, n = self.prefix, self.names
        return {p + n["gate"]: ParamSpec((self.inter, self.hidden)),
                p + n["up"]: ParamSpec((self.inter, self.hidden)),
                p + n["down"]: ParamSpec((self.hidden, self.inter))}

    def batch_needs(self):
        return BatchNeeds(row_tile=self.down.row_tile() if self.down is not None else 1)

    def load_params(self, get):
        p, n = self.prefix, self.names
        g, u = get(p + n["gate"]), get(p + n["up"])
        dt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        self.gate_up = Linear(self.rt, torch.cat([g.to(dt), u.to(dt)], dim=0))
        self.down = Linear(self.rt, get(p + n["down"]))

    def forward_prenorm(self, norm, residual, xn, ctx):
        # few rows (decoding): the product before the norm may have left its rows scaled by the
        # norm's weights; the gate/up product then applies the rows' factors with its activation
        sc = residual.scaled_rows(norm) if self.activation == "silu" else None
        if sc is not None and self.gate_up.takes_swiglu(sc.rows):
            h = ctx.ws.buffer("mlp.h", (sc.rows.shape[0], self.inter), self.rt.dtype)
            self.gate_up(sc.rows, h, ws=ctx.ws, swiglu=True, row_scale=sc.scale)
            return residual.add_linear(self.down, h)
        self.forward(residual.normed(norm, xn), residual, ctx)

    def forward(self, xn, residual, ctx):
        t = xn.shape[0]
        h = ctx.ws.buffer("mlp.h", (t, self.inter), self.rt.dtype)
        if self.activation == "silu" and self.gate_up.takes_swiglu(xn):
            self.gate_up(xn, h, ws=ctx.ws, swiglu=True)        # few rows: the activation is the epilogue
        else:
            if self.activation == "silu":
                gu = ctx.ws.buffer("mlp.gate_up", (t, 2 * self.inter), self.rt.dtype)
                self.gate_up(xn, gu, ws=ctx.ws)
                ops.swiglu(gu, h)
            else:                                              # the product is left in float32 and the activation rounds once
                gu = ctx.ws.buffer("mlp.gate_up32", (t, 2 * self.inter), torch.float32)
                self.gate_up(xn, gu, ws=ctx.ws)
                ops.gated_act(gu, h, self.activation)
        residual.add_linear(self.down, h)


register_part("feed_forward", "swiglu_mlp", SwiGLUMLP)
register_part("feed_forward", "gated_mlp", SwiGLUMLP)


class ReluSquaredMLP(FeedForward):
    """Dense feed-forward with a squared ReLU: y = max(xn Wu^T, 0)^2 Wd^T, no biases.  The first product is
    left in float32 and the activation rounds once to the engine's dtype."""
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec.args["hidden_size"])
        self.inter = int(spec.args["intermediate_size"])
        self.names = {"up": "up", "down": "down", **(spec.args.get("names") or {})}
        self.up = None
        self.down = None

    def expected_params(self):
        p = self.prefix
        return {p + self.names["up"]: ParamSpec((self.inter, self.hidden)),
                p + self.names["down"]: ParamSpec((self.hidden, self.inter))}

    def batch_needs(self):
        return BatchNeeds(row_tile=self.down.row_tile() if self.down is not None else 1)

    def load_params(self, get):
        self.up = Linear(self.rt, get(self.prefix + self.names["up"]))
        self.down = Linear(self.rt, get(self.prefix + self.names["down"]))

    def forward(self, xn, residual, ctx):
        t = xn.shape[0]
        u = ctx.ws.buffer("mlp.up32", (t, self.inter), torch.float32)
        self.up(xn, u, ws=ctx.ws)
        h = ctx.ws.buffer("mlp.h", (t, self.inter), self.rt.dtype)
        ops.relu_squared(u, h)
        residual.add_linear(self.down, h)


register_part("feed_forward", "relu2_mlp", ReluSquaredMLP)


class GeluMLP(FeedForward):
    """Dense feed-forward with the tanh form of GELU and biases on both products:
    y = gelu_tanh(xn Wu^T + bu) Wd^T + bd.  The first product is left in float32 and the activation rounds once."""
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec.args["hidden_size"])
        self.inter = int(spec.args["intermediate_size"])
        self.biases = bool(spec.args.get("biases", True))
        self.names = {"up": "up", "down": "down", "bias_suffix": ".b", **(spec.args.get("names") or {})}
        self.up = None
        self.down = None

    def expected_params(self):
        p, n = self.prefix, self.names
        e = {p + n["up"]: ParamSpec((self.inter, self.hidden)), p + n["down"]: ParamSpec((self.hidden, self.inter))}
        if self.biases:
            e[p + n["up"] + n["bias_suffix"]] = ParamSpec((self.inter,), init="normal")
            e[p + n["down"] + n["bias_suffix"]] = ParamSpec((self.hidden,), init="normal")
        return e

    def batch_needs(self):
        return BatchNeeds(row_tile=self.down.row_tile() if self.down is not None else 1)

    def load_params(self, get):
        p, n = self.prefix, self.names
        self.up = Linear(self.rt, get(p + n["up"]), get(p + n["up"] + n["bias_suffix"]) if self.biases else None)
        self.down = Linear(self.rt, get(p + n["down"]), get(p + n["down"] + n["bias_suffix"]) if self.biases else None)

    def forward(self, xn, residual, ctx):
        t = xn.shape[0]
        u = ctx.ws.buffer("mlp.up32", (t, self.inter), torch.float32)
        self.up(xn, u, ws=ctx.ws)
        h = ctx.ws.buffer("mlp.h", (t, self.inter), self.rt.dtype)
        ops.gelu_tanh(u, h)
        residual.add_linear(self.down, h)


register_part("feed_forward", "gelu_mlp", GeluMLP)
