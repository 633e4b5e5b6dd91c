from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_stream
from ..weights.loader import ParamSpec
from .base import Part


@register_stream("reinject")
class Reinject(Part):
    """x <- W [x; x0]: the residual stream and the embedding's output side by side through one matrix
    [hidden, 2 hidden] (x's columns first).  Used before the first layer of every pass of a stretch of layers that
    runs several times with the same weights.  ``name``: local name of the matrix."""

    def __init__(self, *, hidden_size, name="weight", prefix, dtype, device):
        self.hidden_size, self.name = hidden_size, name
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {self.name: ParamSpec((self.hidden_size, 2 * self.hidden_size))}

    def bind(self, tensors):
        self.weight = ops.prepare_weight(tensors[self.name])

    def forward(self, x, x0, ctx):
        """A new float32 tensor; ``x`` and ``x0`` stay as they are."""
        return ops.linear(ops.concat_cast(x, x0, self.dtype), self.weight, out_dtype=torch.float32)


@register_stream("depth_average")
class DepthAverage(Part):
    """x <- sum over j < n_terms of w[j] X_j: a weighted average over depth of the residual stream's values so far,
    X_0 the embedding's output and X_j the result of the j-th run of a layer that such a part follows.  It runs
    after a layer (``ScheduleEntry.after``); the model keeps the X_j side by side in one tensor and hands them
    over.  ``name``: local name of the weights' tensor [n_terms], kept in float32."""

    def __init__(self, *, n_terms, name="weight", prefix, dtype, device):
        if n_terms < 1:
            raise ValueError("depth average: at least one term")
        self.n_terms, self.name = int(n_terms), name
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {self.name: ParamSpec((self.n_terms,), "vector", "mean")}

    def bind(self, tensors):
        self.weight = tensors[self.name]

    def forward_after(self, history, n, out, ctx):
        """``history`` float32 [runs, T, width] of which the first ``n`` hold X_0 .. X_{n-1}; writes ``out``."""
        if n != self.n_terms:
            raise ValueError(f"depth average over {self.n_terms} terms after {n} values of the stream")
        return ops.depth_average(history, n, self.weight, out)
