"""Norms of the residual stream.

RMSNorm: y = w * x / sqrt(mean(x^2) + eps), computed in 32-bit
(src/ops/rms_norm/op.cpp:13-23: eps inside the root, the weight multiplies
directly).  With `offset` (an argument, default 0) the stored tensor lies around
zero and the weight is offset + stored: y = (offset + w) * x / sqrt(...); the sum
is made once, in float32, when the tensor is bound."""
from __future__ import annotations

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Norm, RmsScaling, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.size = int(spec.args["size"])
        self.eps = float(spec.args["eps"])
        if self.eps < 0:
            raise ValueError(f"rmsnorm: eps must not be negative, found {self.eps}")
        self.param = self.prefix + str(spec.args.get("param", "weight"))     # the tensor's name behind the prefix
        self.offset = float(spec.args.get("offset") or 0.0)
        self.weight = None

    def expected_params(self):
        return {self.param: ParamSpec((self.size,), init="normal" if self.offset else "one_plus_normal")}

    def load_params(self, get):
        self.weight = self.rt.vector(get(self.param))
        if self.offset:
            self.weight = (self.weight + self.offset).contiguous()

    def forward(self, x, out):
        ops.rmsnorm(x, self.weight, self.eps, out)
        return out

    def as_scaling(self):
        return RmsScaling(self.weight, self.eps)


class LayerNorm(Norm):
    """Layer norm with weight and, unless `bias` is False, bias: y = (x - mean) / sqrt(var + eps) * w + b, var the mean
    of the squared deviations from the mean, all in 32-bit.  The bias is the tensor named like the weight with
    `bias_suffix` (default ".b") added."""
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.size = int(spec.args["size"])
        self.eps = float(spec.args["eps"])
        if self.eps < 0:
            raise ValueError(f"layernorm: eps must not be negative, found {self.eps}")
        self.param = self.prefix + str(spec.args.get("param", "weight"))
        self.has_bias = bool(spec.args.get("bias", True))
        self.bias_param = self.param + str(spec.args.get("bias_suffix", ".b"))
        self.weight = self.bias = None

    def expected_params(self):
        e = {self.param: ParamSpec((self.size,), init="one_plus_normal")}
        if self.has_bias:
            e[self.bias_param] = ParamSpec((self.size,), init="normal")
        return e

    def load_params(self, get):
        self.weight = self.rt.vector(get(self.param))
        self.bias = self.rt.vector(get(self.bias_param)) if self.has_bias else None

    def forward(self, x, out):
        ops.layernorm(x, self.weight, self.bias, self.eps, out)
        return out


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
