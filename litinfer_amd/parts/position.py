"""Position encodings of a mixer's queries and keys.

Interface: `tables(ctx)` prepares what depends on the step's positions only
(cached in the step context under `key()`, so every layer with the same
constants shares it); `encode_and_store(qkv, ...)` encodes queries and keys in
place inside the packed projection output and, if the cache is owned, writes
keys and values into their pages.  The default does it in two steps
(`apply` + the plain store kernel); an encoding with a fused kernel overrides it.
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part, register_part


class Position(Part):
    category = "position"

    def key(self):
        return (type(self).__name__,)

    def tables(self, ctx):
        return None

    def apply(self, qkv, n_heads_total, head_dim, ctx) -> None:
        """Encode heads 0..n_heads_total-1 of qkv [T, *] (head h at columns
        h*head_dim..) in place."""
        raise NotImplementedError

    def project_encode_store(self, proj, xn, qkv, num_heads, num_kv_heads, head_dim, ctx, cache,
                             row_scale=None) -> bool:
        """An encoding that has the packed projection, the encoding and the page
        write in ONE kernel for this batch does all three and returns True; the
        default has none, and the mixer then projects and calls `encode_and_store`.
        With `row_scale`, `xn` is a norm's input times its weights and the kernel
        would have to apply the rows' factors as well."""
        return False

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache) -> None:
        if cache.owned:
            self.apply(qkv, num_heads + num_kv_heads, head_dim, ctx)
            ops.kv_store(qkv, num_heads, num_kv_heads, head_dim, ctx.slot_map(cache.group),
                         cache.k, cache.v, cache.page_size)
        else:
            self.apply(qkv, num_heads, head_dim, ctx)


class RopeNeox(Position):
    graph_safe = True

    """Half-split rotary encoding (src/ops/rope/op.cpp:13-20, :32-39):
    angle_j = pos / theta^(2j/rotary_dim) in float32; for j < rotary_dim/2 the
    pair (x[j], x[j + rotary_dim/2]) is rotated by angle_j.  The reference
    rotates the whole head (rotary_dim = head_dim)."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.head_dim = int(spec.args["head_dim"])
        self.rotary_dim = int(spec.args.get("rotary_dim", self.head_dim))
        self.theta = float(spec.args["theta"])
        if self.theta <= 0:
            raise ValueError(f"rope: theta must be positive, found {self.theta}")
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rope: rotary_dim must be even and within the head size "
                             f"{self.head_dim}, found {self.rotary_dim}")

    def key(self):
        return ("rope_neox", self.rotary_dim, self.theta)

    def tables(self, ctx):
        def make():
            cos = ctx.ws.buffer(f"rope.cos.{self.rotary_dim}.{self.theta}",
                                (ctx.num_tokens, self.rotary_dim // 2), ops.float32)
            sin = ctx.ws.buffer(f"rope.sin.{self.rotary_dim}.{self.theta}",
                                (ctx.num_tokens, self.rotary_dim // 2), ops.float32)
            ops.rope_table(ctx.positions, self.theta, self.rotary_dim, cos, sin)
            return cos, sin
        return ctx.shared(self.key(), make)

    def apply(self, qkv, n_heads_total, head_dim, ctx):
        cos, sin = self.tables(ctx)
        ops.rope_apply(qkv, n_heads_total, head_dim, self.rotary_dim, cos, sin)

    def project_encode_store(self, proj, xn, qkv, num_heads, num_kv_heads, head_dim, ctx, cache, row_scale=None):
        # few rows (decoding): the rotation and the page write are the projection's epilogue
        if not (cache.owned and xn.dtype is ops.bfloat16 and proj.weight.dtype is ops.bfloat16):
            return False
        if not (ops.few_rows_preferred(xn.shape[0], proj.out_features, proj.in_features)
                and ops.rope_store_takes(xn.shape[0], proj.in_features, proj.weight.dtype, head_dim, self.rotary_dim)):
            # more rows: where the projection is cut along K anyway, the kernel that adds the parts up rotates and stores
            if row_scale is not None or self.rotary_dim != head_dim:
                return False
            cos, sin = self.tables(ctx)
            return ops.linear_rope_store_parts(xn, proj.weight, proj.bias, qkv, num_heads, num_kv_heads, head_dim, cos, sin,
                                               ctx.slot_map(cache.group), cache.k, cache.v, cache.page_size, ctx.ws)
        cos, sin = self.tables(ctx)
        ops.linear_rope_store(xn, proj.weight, proj.bias, qkv, num_heads, num_kv_heads, head_dim, cos, sin,
                              ctx.slot_map(cache.group), cache.k, cache.v, cache.page_size, row_scale=row_scale)
        return True

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache):
        if not cache.owned:
            return self.apply(qkv, num_heads, head_dim, ctx)
        cos, sin = self.tables(ctx)
        ops.rope_kv_store(qkv, num_heads, num_kv_heads, head_dim, self.rotary_dim, cos, sin,
                          ctx.slot_map(cache.group), cache.k, cache.v, cache.page_size)


register_part("position", "rope_neox", RopeNeox)


class RopePairs(Position):
    """Rotary encoding of NEIGHBOURING pairs: on the first `rotary_dim` columns of a head, columns
    (2i, 2i+1) at position p become (u cos a - v sin a, v cos a + u sin a) with a = p * f_i and
    f_i = theta^(-2i / rotary_dim); the other columns pass.  Optional `scaling` (a dict with factor,
    original, fast, slow) is the YaRN rule: with dim(t) = rotary_dim ln(original / (2 pi t)) /
    (2 ln theta), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), rotary_dim - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency is f_i / factor * ramp_i +
    f_i (1 - ramp_i), and cos and sin are multiplied by 0.1 ln(factor) + 1.  A `scaling` with `kind` = "linear"
    divides every frequency by `factor` and changes nothing else.  The frequencies are
    worked out once on the host (float64, rounded to float32); the angle, cos and sin are float32.
    With layout "half" the same angles rotate column i with column i + rotary_dim/2 instead."""
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.head_dim = int(a["head_dim"])
        self.rotary_dim = int(a.get("rotary_dim", self.head_dim))
        self.theta = float(a["theta"])
        self.scaling = dict(a["scaling"]) if a.get("scaling") else None
        # which columns form a pair: "pairs" (2i, 2i + 1) or "half" (i, i + rotary_dim / 2); the angles are the same
        self.layout = str(a.get("layout") or "pairs")
        if self.layout not in ("pairs", "half"):
            raise ValueError(f"rope: layout must be 'pairs' or 'half', found {self.layout!r}")
        if self.theta <= 0:
            raise ValueError(f"rope: theta must be positive, found {self.theta}")
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rope: rotary_dim must be even and within the head size "
                             f"{self.head_dim}, found {self.rotary_dim}")
        freq, self.amplitude = pair_frequencies(self.rotary_dim, self.theta, self.scaling)
        self._freq_host = freq
        self._freq = None

    def key(self):
        sc = tuple(sorted(self.scaling.items())) if self.scaling else None
        return ("rope_pairs", self.rotary_dim, self.theta, sc)

    def tables(self, ctx):
        def make():
            import torch
            if self._freq is None:
                self._freq = torch.tensor(self._freq_host, dtype=torch.float32, device=self.rt.device)
            name = f"rope_pairs.{hash(self.key()) & 0xffffffff:x}"
            cos = ctx.ws.buffer(name + ".cos", (ctx.num_tokens, self.rotary_dim // 2), ops.float32)
            sin = ctx.ws.buffer(name + ".sin", (ctx.num_tokens, self.rotary_dim // 2), ops.float32)
            ops.rope_freq_table(ctx.positions, self._freq, self.amplitude, cos, sin)
            return cos, sin
        return ctx.shared(self.key(), make)

    def apply(self, qkv, n_heads_total, head_dim, ctx):
        cos, sin = self.tables(ctx)
        if self.layout == "half":
            ops.rope_apply(qkv, n_heads_total, head_dim, self.rotary_dim, cos, sin)
        else:
            ops.rope_pairs_apply(qkv, n_heads_total, head_dim, self.rotary_dim, cos, sin)


def pair_frequencies(rotary_dim: int, theta: float, scaling=None):
    """([f_0 .. f_{rotary_dim/2 - 1}], amplitude of cos and sin) as `RopePairs` describes them."""
    import math
    half = rotary_dim // 2
    freq = [theta ** (-2.0 * i / rotary_dim) for i in range(half)]
    if not scaling:
        return freq, 1.0
    if scaling.get("kind") == "linear":
        factor = float(scaling["factor"])
        if factor <= 0:
            raise ValueError(f"rope scaling: factor must be positive, found {factor}")
        return [f / factor for f in freq], 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])
    if factor <= 0 or original <= 0:
        raise ValueError(f"rope scaling: factor and original must be positive, found {factor}, {original}")

    def dim_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))
    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), rotary_dim - 1)
    out = []
    for i, f in enumerate(freq):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


register_part("position", "rope_pairs", RopePairs)
