"""A decoder model assembled from a ``ModelSpec``: embedding, layers in the order of
the schedule, final norm, output head (src/model/model.cpp:60-99 is the reference's
single-token forward)."""
from __future__ import annotations

import torch

from .. import parts as _parts  # noqa: F401  (registers the built-in parts)
from ..config.spec import ModelSpec
from ..kernels import ops
from ..parts.base import Part, cache_specs_of, collect_params
from ..parts.block import SubLayer
from ..registry import lookup


def _make(table: str, spec, dtype, device, **extra):
    return lookup(table, spec.kind)(**spec.params, prefix=spec.prefix, dtype=dtype, device=device, **extra)


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec, dtype=torch.bfloat16, device="cuda", allocate: bool = True):
        spec.validate()
        self.spec, self.dtype = spec, dtype
        self.device = device if allocate else None
        dev = self.device
        self.embedding = _make("embedding", spec.embedding, dtype, dev)
        self.positions = {}            # layers whose position specs are equal share one part
        self.layers = []
        self.layer_mixers = []         # for each layer its mixers, in the order in which they run
        for ls in spec.layers:
            position = self._position(ls.position, dtype, dev)
            subs, mixers = [], []
            for sub in ls.sublayers:
                if sub.role == "mixer":
                    part = _make("mixer", sub.part, dtype, dev, position=position)
                    mixers.append(part)
                else:
                    part = _make("feed_forward", sub.part, dtype, dev)
                subs.append(SubLayer(sub.role, part,
                                     None if sub.norm is None else _make("norm", sub.norm, dtype, dev),
                                     None if sub.post_norm is None else _make("norm", sub.post_norm, dtype, dev)))
            self.layers.append(lookup("block", ls.block)(subs, **ls.block_params))
            self.layer_mixers.append(mixers)
        # parts that rewrite the residual stream before a run of a layer; equal specs share one part
        self.stream_parts, self._before = {}, []
        for e in spec.schedule:
            b = getattr(e, "before", None)
            key = None if b is None else (b.kind, b.prefix, repr(sorted(b.params.items())))
            if key is not None and key not in self.stream_parts:
                self.stream_parts[key] = _make("stream", b, dtype, dev)
            self._before.append(key)
        # parts that form the stream's next value from all its values so far, after a run of a layer
        self._after = []
        for e in spec.schedule:
            a = getattr(e, "after", None)
            key = None if a is None else ("after", a.kind, a.prefix, repr(sorted(a.params.items())))
            if key is not None and key not in self.stream_parts:
                self.stream_parts[key] = _make("stream", a, dtype, dev)
            self._after.append(key)
        self._n_after = sum(k is not None for k in self._after)
        self.final_norm = _make("norm", spec.final_norm, dtype, dev)
        self.head = _make("head", spec.head, dtype, dev)
        self.schedule = list(spec.schedule)
        # what the cache keeps is counted in units: one for each thing that each mixer of each run of a layer
        # asks of it (one for most mixers; a mixer made of several, or one with a state beside its keys and
        # values, asks for several: ``cache_specs``)
        self._unit, n = {}, 0
        self._asks = [[len(cache_specs_of(m)) for m in mixers] for mixers in self.layer_mixers]
        self._multi = [[hasattr(m, "cache_specs") for m in mixers] for mixers in self.layer_mixers]
        # a mixer that reads another run's cache may still keep some of what it asks for to itself (the history of a
        # convolution on its own queries beside keys and values that it shares): ``keeps_when_reading``, indices
        # into its ``cache_specs()``
        self._keeps = [[tuple(getattr(m, "keeps_when_reading", ())) for m in mixers] for mixers in self.layer_mixers]
        for i, e in enumerate(self.schedule):
            if e.cache_from is not None and self._asks[e.layer] != self._asks[self.schedule[e.cache_from].layer]:
                raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_from}, whose layer has "
                                 "other mixers")
            for k, count in enumerate(self._asks[e.layer]):
                self._unit[i, k] = list(range(n, n + count))
                n += count
        # the unit behind each thing that each mixer of each run sees: its own, or the one of the run it reads
        self._seen = {}
        for i, e in enumerate(self.schedule):
            for k, count in enumerate(self._asks[e.layer]):
                self._seen[i, k] = [self._unit[i, k][j] if e.cache_from is None or j in self._keeps[e.layer][k]
                                    else self._unit[e.cache_from, k][j] for j in range(count)]
        # an embedding may keep state of every sequence too (the token before, say): its units come last
        self._embedding_units = list(range(n, n + len(self._embedding_specs())))
        self._table = collect_params(self)

    def _position(self, spec, dtype, dev):
        if spec is None:
            return None
        key = (spec.kind, spec.prefix, repr(sorted(spec.params.items())))
        if key not in self.positions:
            self.positions[key] = _make("position", spec, dtype, dev)
        return self.positions[key]

    # -- weights -----------------------------------------------------------
    def children(self):
        return [self.embedding, *self.positions.values(), *self.stream_parts.values(), *self.layers, self.final_norm,
                self.head]

    def recordable(self) -> bool:
        """True if every part's forward pass can be recorded into a graph."""
        stack = list(self.children())
        while stack:
            part = stack.pop()
            if not getattr(part, "recordable", True):
                return False
            stack += list(part.children()) if hasattr(part, "children") else []
        return True

    def params(self) -> dict:
        """Full tensor name -> ParamSpec of everything the model needs."""
        return {name: spec for name, (_, _, spec) in getattr(self, "_table", {}).items()}

    def ignorable_names(self) -> list:
        out = []
        stack = [self]
        while stack:
            p = stack.pop()
            out.extend(p.ignorable())
            stack.extend(p.children())
        return out

    def bind(self, tensors) -> None:
        """``tensors``: full tensor name -> tensor.  They are asked for part by part, so a mapping that
        makes each tensor when it is asked for (``weights.loader.OnDemand``) never holds more than one
        part's tensors beside what the parts keep."""
        per_part: dict = {}
        for name, (part, local, _) in self._table.items():
            per_part.setdefault(id(part), (part, []))[1].append((local, name))
        for part, names in per_part.values():
            part.bind({local: tensors[name] for local, name in names})
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.weight)
        # parts that arrange something across their children once all have their tensors (a product shared by
        # mixers that read the same rows)
        stack = list(self.children())
        while stack:
            part = stack.pop()
            if hasattr(part, "finish_bind"):
                part.finish_bind()
            stack += list(part.children())

    # -- cache -------------------------------------------------------------
    def _embedding_specs(self) -> list:
        return list(self.embedding.cache_specs()) if hasattr(self.embedding, "cache_specs") else []

    def cache_specs(self) -> list:
        """For each unit (each mixer of each schedule entry, in order, then whatever the embedding keeps of every
        sequence) what it asks of the cache (None: it reads another's)."""
        return [None if e.cache_from is not None and j not in getattr(m, "keeps_when_reading", ()) else spec
                for e in self.schedule for m in self.layer_mixers[e.layer]
                for j, spec in enumerate(cache_specs_of(m))] + self._embedding_specs()

    # -- the forward pass of one step ---------------------------------------
    def forward(self, ctx, cache) -> torch.Tensor:
        """Runs the step's tokens through the schedule; returns float32 logits [n_want, vocab]."""
        if self._embedding_units:
            x = x0 = self.embedding.forward(ctx, [cache.view(u) for u in self._embedding_units])
        else:
            x = x0 = self.embedding.forward(ctx)
        history, n_hist = None, 0
        if self._n_after:
            # the stream's values side by side: the embedding's output, then the result of every run that an
            # ``after`` part follows (the run works in place on the row that the part before it has written)
            history = torch.empty((self._n_after + 2,) + tuple(x0.shape), dtype=torch.float32, device=x0.device)
            history[0].copy_(x0)
            history[1].copy_(x0)
            x, n_hist = history[1], 1
        for i, e in enumerate(self.schedule):
            if self._before[i] is not None:
                x = self.stream_parts[self._before[i]].forward(x, x0, ctx)       # a new tensor: x0 stays as it is
            elif x is x0 and self.stream_parts and history is None:
                x = ops.copy_rows(x0)            # the layers add in place, and a later part reads the embedding's output
            # one view for a mixer, or the list of its views for one that asks several things of the cache
            views = [[cache.view(u) for u in self._seen[i, k]] if multi else cache.view(self._seen[i, k][0])
                     for k, multi in enumerate(self._multi[e.layer])]
            layer = self.layers[e.layer]
            if getattr(layer, "takes_next_norm", False):
                # the norm that reads the residual stream after this layer: the next layer's first
                nxt = self.layers[self.schedule[i + 1].layer] if i + 1 < len(self.schedule) else None
                first = getattr(nxt, "first_norm", None)
                layer.forward(x, ctx, views, e.cache_from is None, next_norm=first() if first else None)
            else:
                layer.forward(x, ctx, views, e.cache_from is None)
            if self._after[i] is not None:
                n_hist += 1                      # x is history[n_hist - 1], now a finished value of the stream
                x = self.stream_parts[self._after[i]].forward_after(history, n_hist, history[n_hist], ctx)
        if ctx.n_want == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        h = self.final_norm.forward(x, ctx.want_rows)
        return self.head.forward(h)
