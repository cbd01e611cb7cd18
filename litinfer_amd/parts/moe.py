"""A routed feed-forward: `experts` small feed-forwards of which every token uses `top`, and an optional shared
one that every token uses.

Router: logits = xn Wr^T (+ br) in float32.  `scores` = "softmax_chosen": the `top` largest logits are chosen (the
lower index wins a tie) and weighted by the softmax over the chosen logits alone.  `scores` = "sigmoid": an
expert's score is sigmoid(logit); the choice goes by score + correction (a stored vector, one number an expert,
that the weights do not see), and, where the experts form `groups` groups of neighbours, only among the experts of
the `keep_groups` groups whose two largest choice values have the largest sum; the weights are the chosen scores
divided by their sum.  `scores` = "softmax": the same with an expert's score = the softmax over ALL router outputs.
`group_score` = "max": a group's score is its largest choice value (default: the sum of its two largest);
`normalize` False: the weights are the chosen scores as they are.  `identity` > 0: the router has that many outputs
more than there are experts; the last `identity` of them are identity experts, which have no tensors and whose output
is the feed-forward's input itself (times the weight); groups are formed over all router outputs.
An expert (`activation`): "relu2" is Wdown max(Wup xn, 0)^2; "swiglu" is Wdown (silu(Wgate xn) * (Wup xn));
"clamped_swiglu" is Wdown (g sigmoid(1.702 g) (u + 1)) with g = min(Wgate xn, limit), u = clamp(Wup xn, -limit, limit).  No
biases.  The shared expert (relu2 only) has a width of its own; its output is multiplied by sigmoid(wg . xn), one
number a token, where a gate row is given.  The output is the weighted sum, added to the stream in float32.

On the device: one kernel routes (logits, choice, weights and the shared gate), one sorts the step's (token,
choice) pairs by expert and cuts them into tiles of rows, the two products run tile by tile against the
tile's expert (the activation is the first one's epilogue; gate and up are ONE product whose matrix holds an
expert's gate and up rows in turn, so that a thread of the product ends with both factors of an output), and one
kernel adds the weighted rows and the gated shared output into the stream, in the order of the choices.  No number
returns to the host, so a decoding step can be recorded.  The experts' matrices are bound as two tensors
[experts, ff (or 2 ff), hidden] and [experts, hidden, ff].
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, FeedForward, register_part
from .linear import Linear


class RoutedMLP(FeedForward):
    graph_safe = True
    default_activation = "swiglu"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.experts = int(a["experts"])
        self.top = int(a["top"])
        self.inter = int(a["intermediate_size"])
        self.activation = str(a.get("activation") or self.default_activation)
        self.scores = str(a.get("scores") or "softmax_chosen")
        self.groups = int(a.get("groups") or 1)
        self.keep_groups = int(a.get("keep_groups") or self.groups)
        self.has_correction = bool(a.get("correction", False))
        self.has_router_bias = bool(a.get("router_bias", self.scores == "softmax_chosen"))
        self.identity = int(a.get("identity") or 0)
        self.n_router = self.experts + self.identity             # the router's outputs
        self.group_score = str(a.get("group_score") or "top2_sum")
        self.normalize = bool(a.get("normalize", True))
        self.limit = float(a.get("limit") or 0.0)
        self.shared_inter = int(a.get("shared_intermediate_size") or 0)
        self.shared_gate = bool(a.get("shared_gate", True)) and self.shared_inter > 0
        if min(self.hidden, self.experts, self.top, self.inter) <= 0 or self.identity < 0 or self.top > self.n_router:
            raise ValueError(f"routed feed-forward: {self.top} of {self.experts} experts of width {self.inter}")
        if self.top > 64:
            raise ValueError("routed feed-forward: the router kernel picks at most 64 experts a token")
        if (self.activation not in ("relu2", "swiglu", "clamped_swiglu") or self.scores not in ("softmax_chosen", "sigmoid", "softmax")
                or self.group_score not in ("top2_sum", "max")):
            raise ValueError(f"routed feed-forward: activation {self.activation!r}, scores {self.scores!r}, group score {self.group_score!r}")
        if self.activation == "clamped_swiglu" and self.limit <= 0:
            raise ValueError("routed feed-forward: the clamped activation needs a positive limit")
        if self.scores == "softmax_chosen" and (self.groups != 1 or self.has_correction or self.identity):
            raise ValueError("routed feed-forward: groups, a correction of the choice and identity experts belong to "
                             "scores over all router outputs (sigmoid, softmax)")
        if not 1 <= self.keep_groups <= self.groups or self.n_router % self.groups:
            raise ValueError(f"routed feed-forward: {self.n_router} router outputs in {self.groups} groups of which {self.keep_groups} are kept")
        if self.top > self.keep_groups * (self.n_router // self.groups):
            raise ValueError(f"routed feed-forward: {self.top} choices, but the kept groups hold "
                             f"{self.keep_groups * (self.n_router // self.groups)} experts")
        if self.shared_inter and self.activation != "relu2":
            raise ValueError("routed feed-forward: the shared expert is a squared-ReLU one")
        self.names = {"expert": "e{}.", "up": "up", "gate": "gate", "down": "down", "router": "router", "router_bias": "router.b",
                      "correction": "correction", "shared": "shared.", "shared_gate": "sg", **(a.get("names") or {})}
        self.gated = self.activation in ("swiglu", "clamped_swiglu")
        self.w_up = self.w_down = self.router = self.router_b = self.correction = None
        self.gate_row = self.shared_up = self.shared_down = None

    def _expert(self, e: int, which: str) -> str:
        return self.prefix + self.names["expert"].format(e) + self.names[which]

    def expected_params(self):
        p, n = self.prefix, self.names
        out = {p + n["router"]: ParamSpec((self.n_router, self.hidden))}
        if self.has_router_bias:
            out[p + n["router_bias"]] = ParamSpec((self.n_router,), init="zeros")
        if self.has_correction:
            out[p + n["correction"]] = ParamSpec((self.n_router,), init="normal")
        for e in range(self.experts):
            if self.gated:
                out[self._expert(e, "gate")] = ParamSpec((self.inter, self.hidden))
            out[self._expert(e, "up")] = ParamSpec((self.inter, self.hidden))
            out[self._expert(e, "down")] = ParamSpec((self.hidden, self.inter))
        if self.shared_inter:
            s = p + n["shared"]
            out[s + n["up"]] = ParamSpec((self.shared_inter, self.hidden))
            out[s + n["down"]] = ParamSpec((self.hidden, self.shared_inter))
            if self.shared_gate:
                out[s + n["shared_gate"]] = ParamSpec((1, self.hidden))
        return out

    def batch_needs(self):
        return BatchNeeds(row_tile=self.shared_down.row_tile() if self.shared_down is not None else 1)

    def load_params(self, get):
        p, n = self.prefix, self.names
        if self.gated:                       # an expert's gate and up rows in turn: one product, the activation its epilogue
            first = [torch.stack([get(self._expert(e, "gate")), get(self._expert(e, "up"))], dim=1).reshape(2 * self.inter, self.hidden)
                     for e in range(self.experts)]
        else:
            first = [get(self._expert(e, "up")) for e in range(self.experts)]
        self.w_up = self.rt.matrix(torch.stack(first))
        self.w_down = self.rt.matrix(torch.stack([get(self._expert(e, "down")) for e in range(self.experts)]))
        self.router = self.rt.matrix(get(p + n["router"]))
        self.router_b = self.rt.vector(get(p + n["router_bias"])) if self.has_router_bias else None
        self.correction = self.rt.vector(get(p + n["correction"])) if self.has_correction else None
        if self.shared_inter:
            s = p + n["shared"]
            self.shared_up = Linear(self.rt, get(s + n["up"]))
            self.shared_down = Linear(self.rt, get(s + n["down"]))
            if self.shared_gate:
                self.gate_row = self.rt.matrix(get(s + n["shared_gate"]).reshape(-1))

    def forward(self, xn, residual, ctx):
        t, top, ws = xn.shape[0], self.top, ctx.ws
        pairs = t * top
        idx = ws.buffer("moe.idx", (t, top), torch.int32)
        wt = ws.buffer("moe.wt", (t, top), torch.float32)
        gate = ws.buffer("moe.gate", (t,), torch.float32) if self.gate_row is not None else None
        ops.moe_route(xn, self.router, self.router_b, self.gate_row, idx, wt, gate, scores=self.scores,
                      correction=self.correction, groups=self.groups, keep_groups=self.keep_groups,
                      group_score=self.group_score, normalize=self.normalize)
        # (a prompt's portion gives every expert hundreds of rows: larger tiles then, for the kernel that stages them in LDS)
        n_first = self.w_up.shape[1]
        rows_a_tile = ops.moe_tile_rows(t, top, self.experts, xn.dtype, self.w_up.dtype,
                                        ((n_first, self.hidden), (self.hidden, self.inter)))
        max_tiles = ops.moe_max_tiles(t, top, self.experts, rows_a_tile)
        plan = ws.buffer("moe.plan", (4 + 4 * max_tiles,), torch.int32)
        row_token = ws.buffer("moe.row_token", (pairs,), torch.int32)
        pair_row = ws.buffer("moe.pair_row", (pairs,), torch.int32)
        ops.moe_plan(idx, self.experts, plan, row_token, pair_row, rows_a_tile)
        h = ws.buffer("moe.h", (pairs, self.inter), self.rt.dtype)
        ops.moe_linear(xn, row_token, self.w_up, plan, max_tiles, h, pairs, act={"relu2": 1, "swiglu": 2, "clamped_swiglu": 3}[self.activation],
                       tile_rows=rows_a_tile, limit=self.limit)
        yrows = ws.buffer("moe.y", (pairs, self.hidden), torch.float32)
        ops.moe_linear(h, None, self.w_down, plan, max_tiles, yrows, pairs, tile_rows=rows_a_tile)
        shared = None
        if self.shared_inter:
            u = ws.buffer("mlp.up32", (t, self.shared_inter), torch.float32)
            self.shared_up(xn, u, ws=ws)
            hs = ws.buffer("mlp.h", (t, self.shared_inter), self.rt.dtype)
            ops.relu_squared(u, hs)
            shared = ws.buffer("moe.shared", (t, self.hidden), torch.float32)
            self.shared_down(hs, shared, ws=ws)
        # (a pair whose choice is an identity expert has no row in the plan: the sum takes the token's input for it)
        ops.moe_combine(residual.tensor(), yrows, pair_row, wt, gate, shared, idx=idx if self.identity else None,
                        experts=self.experts, identity_rows=xn if self.identity else None)


class RoutedReluSquaredMLP(RoutedMLP):
    """Squared-ReLU experts behind a router with bias and a softmax over the chosen logits, plus a gated shared expert."""
    default_activation = "relu2"


register_part("feed_forward", "routed_relu2", RoutedReluSquaredMLP)
register_part("feed_forward", "routed_mlp", RoutedMLP)
