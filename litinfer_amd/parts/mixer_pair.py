"""Two mixers side by side that read the same input; the result is left_scale * left + right_scale * right.

Each of the two is any registered mixer (`left`, `right`: their PartSpecs) with a cache need of its own: the pair keeps
both (one of them may keep pages, both may keep named states), and both see the entry's one cache view.  The two
outputs are not added here: each mixer writes into an output of its own in the branch that the block hands it, with
its factor, and the kernel that norms the branch and adds it to the stream forms the weighted sum in float32 on its
way.  With both factors 1 the pair also runs in arrangements whose sublayers add straight into the stream.
"""
from __future__ import annotations

from .base import Mixer, build_part, needs_of, register_part


class MixerPair(Mixer):

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.left = build_part("mixer", a["left"], rt)
        self.right = build_part("mixer", a["right"], rt)
        self.left_scale = float(a.get("left_scale", 1.0))
        self.right_scale = float(a.get("right_scale", 1.0))
        needs_of(self.cache_need())                   # (two paged needs, or states of one name, are refused here)

    @property
    def graph_safe(self):
        return self.left.graph_safe and self.right.graph_safe

    def cache_need(self):
        out = []
        for m in (self.left, self.right):
            need = m.cache_need()
            if need is not None:
                out.extend(need if isinstance(need, (tuple, list)) else (need,))
        return tuple(out) if out else None

    def batch_needs(self):
        return self.left.batch_needs().merged(self.right.batch_needs())

    def expected_params(self):
        return {**self.left.expected_params(), **self.right.expected_params()}

    def load_params(self, get):
        self.left.load_params(get)
        self.right.load_params(get)

    def forward(self, xn, residual, ctx, cache):
        if hasattr(residual, "fork"):
            residual.factor = self.left_scale
            self.left.forward(xn, residual, ctx, cache)
            second = residual.fork("mixer_pair.second")
            second.factor = self.right_scale
            self.right.forward(xn, second, ctx, cache)
            return
        if self.left_scale != 1.0 or self.right_scale != 1.0:
            raise NotImplementedError("mixer pair: factors other than 1 need an arrangement that hands the mixer a branch "
                                      "(the sandwich block)")
        self.left.forward(xn, residual, ctx, cache)
        self.right.forward(xn, residual, ctx, cache)


register_part("mixer", "mixer_pair", MixerPair)
