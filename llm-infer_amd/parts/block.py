from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_block
from .base import Part


class SubLayer:
    """A built sub-layer: its part, what the part is to the engine ("mixer" or "feed_forward"), the norm
    on its input and the norm on its output (either may be None)."""

    def __init__(self, role: str, part, norm=None, post_norm=None):
        self.role, self.part, self.norm, self.post_norm = role, part, norm, post_norm

    def parts(self) -> list:
        return [p for p in (self.norm, self.part, self.post_norm) if p is not None]


class Block(Part):
    """An arrangement of sub-layers.  A block class is built from the list of its ``SubLayer``s and runs
    them on the float32 residual stream ``x`` [T, hidden] in place: ``forward(x, ctx, cache_views,
    owns_cache)``, where ``cache_views`` holds one view for each mixer of the layer, in their order."""

    def __init__(self, sublayers):
        self.sublayers = list(sublayers)

    def children(self):
        return [p for s in self.sublayers for p in s.parts()]

    def first_norm(self):
        """The norm that reads the residual stream first in this layer (None: the first part takes it raw)."""
        return self.sublayers[0].norm

    # the first of each kind, for layers of the common shape
    def _first(self, role):
        for s in self.sublayers:
            if s.role == role:
                return s
        return None

    @property
    def mixer(self):
        s = self._first("mixer")
        return s.part if s else None

    @property
    def mixer_norm(self):
        s = self._first("mixer")
        return s.norm if s else None

    @property
    def feed_forward(self):
        s = self._first("feed_forward")
        return s.part if s else None

    @property
    def feed_forward_norm(self):
        s = self._first("feed_forward")
        return s.norm if s else None


@register_block("pre_norm")
class PreNormBlock(Block):
    """x += part(norm(x)) for each sub-layer in turn; for the Llama layer: x += mixer(norm(x));
    x += feed_forward(norm(x))   (src/model/block.cpp:106-224)."""
    takes_next_norm = True          # forward accepts ``next_norm``

    def __init__(self, sublayers):
        super().__init__(sublayers)
        for s in self.sublayers:
            if s.norm is None or s.post_norm is not None:
                raise ValueError("a pre_norm block has one norm before each part and none after it")

    def forward(self, x, ctx, cache_views, owns_cache=True, next_norm=None):
        """``next_norm``: the norm that reads ``x`` after this layer, if the caller knows it."""
        views = iter(cache_views)
        for i, s in enumerate(self.sublayers):
            # a part that only passes its input on to ops.linear may get a norm whose last step is taken
            # inside that product (ops.LazyNorm)
            if getattr(s.part, "takes_lazy_norm", False) and getattr(s.norm, "can_be_lazy", False):
                h = s.norm.forward(x, lazy=True)
            else:
                h = s.norm.forward(x)
            # and the product that completes the rows of x may prepare the norm that reads them next
            after = self.sublayers[i + 1].norm if i + 1 < len(self.sublayers) else next_norm
            lazy_after = getattr(after, "can_be_lazy", False)
            ops.expect_norm(x, after.weight if lazy_after else None, after.eps if lazy_after else None)
            _run_part(s, h, ctx, next(views) if s.role == "mixer" else None, x, owns_cache)


@register_block("parallel")
class ParallelBlock(Block):
    """x <- x + sum over the sub-layers of part(norm(x)): every sub-layer reads the same x through a norm of its own,
    and their results are added to it together.  All norms are taken before any part adds into the rows.  A part
    that says ``reads_float32`` is handed its normed rows in float32 (a convolution over time ahead of a mixer, say)."""

    def __init__(self, sublayers):
        super().__init__(sublayers)
        for s in self.sublayers:
            if s.norm is None or s.post_norm is not None:
                raise ValueError("a parallel block has one norm before each part and none after it")

    def forward(self, x, ctx, cache_views, owns_cache=True):
        views = iter(cache_views)
        ops.expect_norm(x, None)                 # the rows are complete only after the last part: no norm rides along
        normed = [s.norm.forward(x, out_dtype=torch.float32) if getattr(s.part, "reads_float32", False) else s.norm.forward(x)
                  for s in self.sublayers]
        for s, h in zip(self.sublayers, normed):
            _run_part(s, h, ctx, next(views) if s.role == "mixer" else None, x, owns_cache)


def _run_part(s, h, ctx, view, out, owns_cache):
    """A sub-layer's part on its normed rows ``h``, adding into ``out``; a feed-forward that says ``takes_ctx`` is
    handed the step too (one that chooses its experts by token id, say)."""
    if s.role == "mixer":
        s.part.forward(h, ctx, view, out, owns_cache)
    elif getattr(s.part, "takes_ctx", False):
        s.part.forward(h, out, ctx)
    else:
        s.part.forward(h, out)


@register_block("sandwich")
class SandwichBlock(Block):
    """x <- x + norm_after(part(norm_before(x))) for each sub-layer in turn: every part stands between two norms,
    one on what it reads and one on what it adds to the residual stream.  The part adds into cleared float32 rows
    of its own; the second norm and the residual sum are then one pass over those rows (``ops.rmsnorm_add``), which
    also takes the norm that reads the finished rows next (the next sub-layer's, or the next layer's first).  A
    part that says ``writes_rows`` is handed rows that it overwrites instead (no clearing), and may hand back a
    bias that the pass adds first (``forward_into`` returns it)."""
    takes_next_norm = True          # forward accepts ``next_norm``

    def __init__(self, sublayers):
        super().__init__(sublayers)
        for s in self.sublayers:
            if s.norm is None or s.post_norm is None or not hasattr(s.post_norm, "weight"):
                raise ValueError("a sandwich block has one norm before each part and one with a weight after it")

    @staticmethod
    def _rides(norm):
        """(weight, eps, dtype) of a norm that the pass before it can take along, or None."""
        if norm is None or not getattr(norm, "can_be_lazy", False) or getattr(norm, "weight", None) is None:
            return None
        return norm.weight, norm.eps, norm.dtype

    def forward(self, x, ctx, cache_views, owns_cache=True, next_norm=None):
        """``next_norm``: the norm that reads ``x`` after this layer, if the caller knows it."""
        views = iter(cache_views)
        ops.expect_norm(x, None)                 # no product adds into x itself: no norm rides along
        for i, s in enumerate(self.sublayers):
            h = s.norm.forward(x)                # (found ready where the pass before has taken it)
            after = self._rides(self.sublayers[i + 1].norm if i + 1 < len(self.sublayers) else next_norm)
            view = next(views) if s.role == "mixer" else None
            if getattr(s.part, "writes_rows", False):
                y = torch.empty_like(x)
                bias = s.part.forward_into(h, y, ctx, view, owns_cache)
            else:
                y, bias = torch.zeros_like(x), None
                _run_part(s, h, ctx, view, y, owns_cache)
            ops.rmsnorm_add(x, y, s.post_norm.weight, s.post_norm.eps, bias, after)


@register_block("post_norm")
class PostNormBlock(Block):
    """x <- norm(alpha * x + part(x)) for each sub-layer in turn: the parts read the residual stream itself and
    the norm comes after the sum; ``alpha`` scales the stream's own share.  Every sub-layer has a norm on its
    output (a layer norm with a weight, ``parts.norm.LayerNorm``) and none on its input.

    A part may hand over what it adds as ``addends(h, ...) -> [(y, scale), ...]`` (float32 rows of the
    stream's shape); the scaled sum, the stream's share and the norm are then one kernel.  A part without
    ``addends`` adds into a cleared buffer through its ``forward``.  A part that says ``reads_residual`` takes
    the float32 rows as they are; the others get them in the compute dtype, a copy that the norm kernel of
    the sub-layer before writes along."""

    def __init__(self, sublayers, alpha: float = 1.0):
        super().__init__(sublayers)
        self.alpha = float(alpha)
        for s in self.sublayers:
            if s.norm is not None or s.post_norm is None or not hasattr(s.post_norm, "weight"):
                raise ValueError("a post_norm block has one norm with a weight after each part and none before it")

    @staticmethod
    def _addends(s, h, x, ctx, view, owns_cache):
        if hasattr(s.part, "addends"):
            return s.part.addends(h, ctx, view, owns_cache) if s.role == "mixer" else s.part.addends(h)
        y = torch.zeros_like(x)
        if s.role == "mixer":
            s.part.forward(h, ctx, view, y, owns_cache)
        else:
            s.part.forward(h, y)
        return [(y, 1.0)]

    def forward(self, x, ctx, cache_views, owns_cache=True):
        views = iter(cache_views)
        copy = None                                  # the rows of x in the compute dtype, if the last norm left them
        for i, s in enumerate(self.sublayers):
            dtype = s.post_norm.dtype
            if getattr(s.part, "reads_residual", False):
                h = x
            else:
                h = copy if copy is not None and copy.dtype == dtype else ops.cast(x, dtype)
            adds = self._addends(s, h, x, ctx, next(views) if s.role == "mixer" else None, owns_cache)
            while len(adds) > 2:                     # the norm kernel takes two: sum the rest beforehand
                (y0, s0), rest = adds[0], adds[1:3]
                y0 = y0 * s0 if s0 != 1.0 else y0
                ops.add_scaled(y0, rest)
                adds = [(y0, 1.0)] + adds[3:]
            nxt = self.sublayers[i + 1] if i + 1 < len(self.sublayers) else None
            wants_copy = nxt is not None and not getattr(nxt.part, "reads_residual", False)
            copy = ops.add_layernorm(x, self.alpha, adds, s.post_norm.weight, s.post_norm.eps,
                                     nxt.post_norm.dtype if wants_copy else None)
