"""Two mixers side by side on the same input: ``left_scale * left(h) + right_scale * right(h)``.

Each side keeps what it needs between steps; the pair asks for both (pages for a side that attends over a cache, a
state slot for a side that carries a recurrence), and each side gets the view of the call's cache and takes its own
share of it.  What comes back is the two results with their scales (:class:`ScaledPair`): a block that normalises
the mixer's result adds them up inside that kernel; anybody else calls ``tensor()``.
"""
from __future__ import annotations

from .base import Mixer, PagedAndStateSpec, PagedKVSpec, StateSpec


class ScaledPair:
    """``left_scale * left + right_scale * right``, not added up yet (two tensors ``[T, W]`` of one type)."""

    def __init__(self, left, left_scale: float, right, right_scale: float):
        self.left, self.left_scale, self.right, self.right_scale = left, float(left_scale), right, float(right_scale)

    def tensor(self, ctx):
        out = ctx.empty(self.left.shape, dtype=self.left.dtype)
        ctx.ops.scaled_sum(self.left, self.left_scale, self.right, self.right_scale, out)
        return out


class ParallelMixers(Mixer):
    def __init__(self, left: Mixer, right: Mixer, left_scale: float, right_scale: float, names=("left", "right")):
        self.left, self.right, self.left_scale, self.right_scale = left, right, float(left_scale), float(right_scale)
        self.names = tuple(names)
        specs = [left.cache_spec(), right.cache_spec()]
        paged = [spec for spec in specs if isinstance(spec, PagedKVSpec)]
        states = [spec for spec in specs if isinstance(spec, StateSpec)]
        if len(paged) > 1 or len(states) > 1 or len(paged) + len(states) != sum(spec is not None for spec in specs):
            raise ValueError("of two mixers side by side at most one may keep pages and at most one a state")
        self._spec = PagedAndStateSpec(paged[0], states[0]) if paged and states else (paged or states or [None])[0]

    @property
    def graph_safe(self):
        return self.left.graph_safe and self.right.graph_safe

    def _sides(self):
        return dict(zip(self.names, (self.left, self.right)))

    def cache_spec(self):
        return self._spec

    def param_specs(self):
        return {f"{prefix}.{name}": spec for prefix, part in self._sides().items() for name, spec in part.param_specs().items()}

    def assign(self, name, tensor):
        prefix, rest = name.split(".", 1)
        self._sides()[prefix].assign(rest, tensor)

    def finalize(self):
        self.left.finalize()
        self.right.finalize()

    def prepare(self, ctx):
        self.left.prepare(ctx)
        self.right.prepare(ctx)

    def graph_shape(self, rows, longest_context):
        shapes = (self.left.graph_shape(rows, longest_context), self.right.graph_shape(rows, longest_context))
        return None if shapes == (None, None) else shapes

    def graph_shape_edges(self):
        return tuple(self.left.graph_shape_edges()) + tuple(self.right.graph_shape_edges())

    def mixing_flops(self, new_tokens, context):
        return self.left.mixing_flops(new_tokens, context) + self.right.mixing_flops(new_tokens, context)

    def forward(self, x, ctx, cache):
        return ScaledPair(self.left.forward(x, ctx, cache), self.left_scale, self.right.forward(x, ctx, cache), self.right_scale)
