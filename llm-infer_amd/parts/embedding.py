from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_embedding, register_head
from ..weights.loader import ParamSpec
from .base import Part


@register_embedding("embedding")
class Embedding(Part):
    """x = float32(table[token]) (src/model/model.cpp:101-118), times ``scale``; ``positions`` "sinusoidal" adds
    to every token the vector of its position p: entry 2i is sin(p f_i), entry 2i+1 cos(p f_i), with
    f_i = position_base^(-2i / hidden_size) (float32 angles)."""

    def __init__(self, *, vocab_size, hidden_size, name="weight", scale=1.0, positions=None, position_base=10000.0,
                 prefix, dtype, device):
        if positions not in (None, "sinusoidal"):
            raise ValueError(f"embedding: positions {positions!r} are not built ('sinusoidal' is)")
        self.vocab_size, self.hidden_size, self.name = vocab_size, hidden_size, name
        self.scale, self.positions = float(scale), positions
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = self.freq = None
        if positions is not None:
            two_i = torch.arange(0, hidden_size, 2, dtype=torch.float64)
            self.freq = torch.pow(torch.tensor(float(position_base), dtype=torch.float64), -two_i / hidden_size) \
                .to(torch.float32).to(device or "cpu")

    def params(self):
        return {self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors):
        self.weight = tensors[self.name]

    def forward(self, ctx):
        """The residual stream's first value for the step's tokens, float32 [T, hidden].  ``ctx`` is the
        step (``token_ids``, and ``pos`` for an embedding that adds positions)."""
        if self.positions is None and self.scale == 1.0:
            return ops.embed(self.weight, ctx.token_ids)
        return ops.embed_positions(self.weight, ctx.token_ids, ctx.pos, self.freq, self.scale)


@register_embedding("bigram_embedding")
class BigramEmbedding(Part):
    """x = float32(table[token]) * ``scale`` + bigram[row]: beside the token's own row, a row of a second table chosen
    by the token and the one before it, row = (previous * ``mul_prev`` + token * ``mul_cur``) mod ``buckets``; a
    sequence's first token takes row number ``buckets``, the last of the table's buckets + 1 rows.

    The token before the first one that a sequence brings to a step is state of the sequence: one int32 for every
    slot (``StateSpec``), which the engine's cache keeps as it keeps a mixer's state, so prompts may be cut anywhere
    and recorded decode steps feed it on the device.  ``names``: local names of the two tables."""

    def __init__(self, *, vocab_size, hidden_size, buckets, mul_prev, mul_cur, scale=1.0, names=None, prefix, dtype, device):
        if buckets < 1:
            raise ValueError("bigram embedding: at least one bucket")
        self.vocab_size, self.hidden_size, self.buckets = vocab_size, hidden_size, int(buckets)
        self.mul_prev, self.mul_cur, self.scale = int(mul_prev), int(mul_cur), float(scale)
        self.names = {"table": "weight", "bigram": "bigram", **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = self.bigram = None

    def params(self):
        return {self.names["table"]: ParamSpec((self.vocab_size, self.hidden_size)),
                self.names["bigram"]: ParamSpec((self.buckets + 1, self.hidden_size))}

    def bind(self, tensors):
        self.weight, self.bigram = tensors[self.names["table"]], tensors[self.names["bigram"]]

    def cache_specs(self):
        from ..cache.specs import StateSpec
        return [StateSpec((), "int32")]

    def forward(self, ctx, views):
        """``views``: the cache's views for ``cache_specs()``; float32 [T, hidden]."""
        return ops.embed_bigram(self.weight, self.bigram, ctx, views[0].state, self.scale, self.mul_prev, self.mul_cur)


@register_head("lm_head")
class LMHead(Part):
    """logits = h W^T in float32 (src/model/model.cpp:93-98).  ``tied``: W is the embedding
    table (the reference has no tied models: it requires output.weight, model.cpp:35-38)."""

    def __init__(self, *, vocab_size, hidden_size, tied, name="weight", softcap=None, scale=1.0, prefix, dtype, device):
        """``softcap`` c: the logits become c * tanh(logits / c).  ``scale``: the logits are multiplied by it (float32)."""
        self.scale = float(scale)
        self.vocab_size, self.hidden_size, self.tied, self.name = vocab_size, hidden_size, tied, name
        self.softcap = None if softcap is None else float(softcap)
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError("lm_head: a positive soft cap")
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {} if self.tied else {self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def ignorable(self):
        return [self.prefix + self.name] if self.tied else []

    def bind(self, tensors):
        if not self.tied:
            self.weight = ops.prepare_weight(tensors[self.name])

    def tie(self, table):
        # the embedding gathers rows, the head streams the whole matrix: it keeps a tiled copy
        self.weight = ops.prepare_weight(table)

    def forward(self, h):
        logits = ops.linear(h, self.weight, out_dtype=torch.float32)
        if self.scale != 1.0:
            ops.scale_values(logits, self.scale)
        return logits if self.softcap is None else ops.softcap(logits, self.softcap)
