from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_norm
from ..tensor import Tensor
from ..weights.loader import ParamSpec
from .base import Part


@register_norm("rmsnorm")
class RMSNorm(Part):
    """out = x / sqrt(mean(x^2) + eps) * weight, in float32; the weight is kept in float32
    (include/kernels_cpu.hpp:43-54, src/model/block.cpp:81-83)."""
    can_be_lazy = True          # forward takes ``lazy``

    def __init__(self, *, size: int, eps: float, name: str = "weight", one_plus: bool = False, scalar: bool = False,
                 prefix: str, dtype, device):
        """``name``: local name of the weight's tensor.  ``one_plus``: the tensor is stored around zero and the
        rows are multiplied by 1 + w (added once, in float32, when the weights are bound).  ``scalar``: the tensor
        is a single number (shape []) that multiplies every coordinate; it is spread over a vector when the
        weights are bound, so the norm kernels run unchanged."""
        self.size, self.eps, self.prefix, self.dtype, self.device = size, float(eps), prefix, dtype, device
        self.name, self.one_plus, self.scalar = name, bool(one_plus), bool(scalar)
        self.weight = None

    def params(self):
        return {self.name: ParamSpec(() if self.scalar else (self.size,), "vector", "small" if self.one_plus else "ones")}

    def bind(self, tensors):
        w = tensors[self.name]
        if self.scalar:
            w = Tensor.wrap(w.as_subclass(torch.Tensor).float().reshape(1).expand(self.size).contiguous())
        self.weight = Tensor.wrap((w.as_subclass(torch.Tensor).float() + 1.0).contiguous()) if self.one_plus else w

    def forward(self, x: torch.Tensor, rows: torch.Tensor | None = None, lazy: bool = False, out_dtype=None):
        """The normed rows in the compute dtype (``out_dtype``: in that type, for a part that goes on in float32).  ``lazy``: the caller hands the result to parts that pass
        it on to ``ops.linear`` untouched (``takes_lazy_norm``); then, where the product before has prepared
        this norm (a decode step), an ``ops.LazyNorm`` is returned and the product that reads it finishes it."""
        if out_dtype is not None and out_dtype != self.dtype:
            return ops.rmsnorm(x, self.weight, self.eps, out_dtype, rows)
        if lazy and rows is None:
            deferred = ops.lazy_rmsnorm(x, self.weight, self.eps, self.dtype)
            if deferred is not None:
                return deferred
        if rows is None:
            ready = ops.prepared_rmsnorm(x, self.weight, self.eps, self.dtype)    # taken by the product before
            if ready is not None:
                return ready
        return ops.rmsnorm(x, self.weight, self.eps, self.dtype, rows)


@register_norm("layernorm")
class LayerNorm(Part):
    """out = (x - mean) / sqrt(var + eps) * weight in float32, var the mean of the squared deviations; a weight
    and no bias.  ``name`` is the local name of the weight's tensor."""

    def __init__(self, *, size: int, eps: float, name: str = "weight", prefix: str, dtype, device):
        self.size, self.eps, self.name = size, float(eps), name
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {self.name: ParamSpec((self.size,), "vector", "ones")}

    def bind(self, tensors):
        self.weight = tensors[self.name]

    def forward(self, x: torch.Tensor, rows: torch.Tensor | None = None):
        return ops.layernorm(x, self.weight, self.eps, self.dtype, rows)
