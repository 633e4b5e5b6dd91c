from __future__ import annotations

import torch

from ..cache.specs import StateSpec
from ..kernels import ops
from ..registry import lookup, register_mixer
from ..weights.loader import ParamSpec
from .base import Part, cache_specs_of, views_for


@register_mixer("short_conv")
class ConvMixer(Part):
    """A mixer whose input first passes a short causal convolution over time, channel by channel, beside itself:
    h_t <- h_t + sum over j < taps of w[:, j] * h_(t - taps + 1 + j), zeros before a sequence's first token, no bias
    and no activation.  ``inner`` (a ``PartSpec``) is the mixer that reads the result.

    The inputs before the first token that a sequence brings to a step are the sequence's state: its last taps - 1
    inputs, float32 [taps - 1, hidden], kept for every run of the layer (``StateSpec``).  The part takes its normed rows
    in float32 (``reads_float32``), convolves in float32 and hands the inner mixer its input in the compute dtype.
    ``name``: local name of the weights' tensor [hidden, taps]."""

    reads_float32 = True

    def __init__(self, *, hidden_size, taps, inner, name="conv", position=None, prefix, dtype, device):
        if not 1 <= taps <= 16:
            raise ValueError(f"short convolution over {taps} tokens (1 to 16)")
        self.hidden_size, self.taps, self.name = hidden_size, int(taps), name
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.inner = lookup("mixer", inner.kind)(**inner.params, position=position, prefix=inner.prefix, dtype=dtype,
                                                 device=device)
        self.weight = None

    def children(self):
        return [self.inner]

    def params(self):
        return {self.name: ParamSpec((self.hidden_size, self.taps), "vector", "small")}

    def bind(self, tensors):
        self.weight = tensors[self.name]

    def cache_specs(self):
        return [StateSpec((max(self.taps - 1, 1), self.hidden_size), "float32")] + cache_specs_of(self.inner)

    def forward(self, h, ctx, views, residual, owns_cache=True):
        """``h``: the normed rows in float32; the inner mixer's result is added into ``residual``."""
        if not owns_cache:
            raise ValueError("a mixer behind a short convolution keeps a state of its own in every run")
        if h.dtype != torch.float32:
            raise ValueError("the short convolution reads float32 rows")
        u = ops.conv_add(h, self.weight, views[0].state, ctx, self.dtype)
        inner_views, _ = views_for(self.inner, views, 1)
        self.inner.forward(u, ctx, inner_views, residual, owns_cache)
