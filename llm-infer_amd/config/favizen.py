"""Typed configuration of the Favizen decoder, read from its own config.json keys.

A model of this design is a list of layers over a float32 residual stream of ``width``.  Every sub-layer stands
between two RMS norms with a weight (``norm.eps``): x <- x + norm1b(mixer(norm1(x))), then, where the layer has a
feed-forward, x <- x + norm2b(ff(norm2(x))).  ``layers[i].type`` names the mixer, ``layers[i].mixer`` its sizes
(``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size``).  Both mixers are grouped-query softmax
attention with a learned sink in every head's sum and a sigmoid gate on every head's output (one number a head):

* ``attention``: no value projection (a token's values are its keys as projected, before the rotation); q and k are
  turned by position in their first ``rot.dims`` dimensions, i paired with i + dims / 2, frequencies ``rot.base``^(-2i /
  dims), stretched by wavelength as ``rot.scaling`` {``factor``, ``low``, ``high``, ``original``} says; a sliding
  window of ``mask.size`` positions.
* ``attention_2``: q, k and v with biases, each followed by a causal convolution over ``conv`` tokens on every channel;
  no rotation; a score loses 2^(-8 (h + 1) / heads) for every position between query and key; position i sees the keys
  of its own chunk of ``mask.size`` positions.  ``kv_from``: j: the layer has no key or value tensors and reads layer
  j's keys and values.

``layers[i].mlp`` is null, ``{"kind": "dense", "ff", "limit"}`` (gate, up and down with biases) or ``{"kind": "moe",
"expert": {"ff", "limit"}, "router": {"experts", "top"}, "shared": {"ff", "limit"}}`` (experts without biases that a
table assigns to token ids, each of weight 1 / top, and a shared expert for every token times the sigmoid of one more
product).  Every feed-forward is W_down(g sigmoid(1.702 g) (u + 1)) with g = min(W_gate h, limit), u = clamp(W_up h,
-limit, limit).  The embedding is ``embed[token] * embedding.scale``, the logits ``head`` on the final norm times
``logit_scale``.  Tensor names: ``embed``, ``final.norm``, ``head``, and per layer ``l<i>.norm1``, ``norm1b``,
``norm2``, ``norm2b``, ``l<i>.mix.*`` (q, k, v, their ``.b`` and ``.conv``, sink, g, o), ``l<i>.mlp.*``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, SubLayerSpec

_DTYPES = ("float32", "float16", "bfloat16")
_MIXERS = ("attention", "attention_2")
SLOPE_EXPONENT = 8.0          # the distance bias of attention_2: slope_h = 2^(-8 (h + 1) / heads)
SWISH_ALPHA = 1.702           # the feed-forwards' activation: g sigmoid(1.702 g) (u + 1)
UP_SHIFT = 1.0


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class FavizenConfig:
    width: int
    vocab: int
    norm_eps: float
    embedding_scale: float
    layers: tuple                   # the layers as config.json lists them (plain dicts)
    logit_scale: float = 1.0
    max_positions: int = 0          # the design sets no bound; an optional key may
    torch_dtype: str | None = None
    eos_token_ids: tuple = ()
    architecture: str = "Favizen"

    context_key = "max_positions"

    @classmethod
    def from_dict(cls, c: dict) -> "FavizenConfig":
        layers = _need(c, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        eos = c.get("eos_token_id")
        cfg = cls(width=int(_need(c, "width", "the model")), vocab=int(_need(c, "vocab", "the model")),
                  norm_eps=float(_need(_need(c, "norm", "the model"), "eps", "norm")),
                  embedding_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                  layers=tuple(copy.deepcopy(layers)), logit_scale=float(c.get("logit_scale", 1.0)),
                  max_positions=int(c.get("max_positions") or 0), torch_dtype=c.get("torch_dtype"),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=c.get("architecture") or (c.get("architectures") or ["Favizen"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.width <= 0 or self.vocab <= 0:
            raise ConfigError("width and vocab must be positive")
        if not self.norm_eps >= 0:
            raise ConfigError("norm.eps must not be negative")
        if self.torch_dtype is not None and self.torch_dtype not in _DTYPES:
            raise ConfigError(f"Unsupported torch_dtype: {self.torch_dtype}")
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            kind, m = _need(layer, "type", where), _need(layer, "mixer", where)
            if kind not in _MIXERS:
                raise ConfigError(f"{where}: mixer type {kind!r} is not built ({' and '.join(_MIXERS)} are)")
            for k in ("heads", "kv_heads", "dim", "scale"):
                _need(m, k, where + " mixer")
            H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m.get("vdim", m["dim"]))
            if min(H, G, d, dv) < 1 or H % G:
                raise ConfigError(f"{where}: heads a positive multiple of kv_heads, dim and vdim positive")
            if int(_need(_need(m, "mask", where + " mixer"), "size", where + " mask")) < 1:
                raise ConfigError(f"{where}: mask.size must be positive")
            if kind == "attention":
                if dv != d:
                    raise ConfigError(f"{where}: the values are the keys, so vdim equals dim")
                rot = m.get("rot")
                if rot is not None:
                    dims = int(_need(rot, "dims", where + " rot"))
                    _need(rot, "base", where + " rot")
                    if dims % 2 or not 0 <= dims <= d:
                        raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                    if rot.get("scaling") is not None:
                        for k in ("factor", "low", "high", "original"):
                            _need(rot["scaling"], k, where + " rot.scaling")
            elif not 1 <= int(m.get("conv", 1)) <= 16:
                raise ConfigError(f"{where}: conv: 1 to 16 taps")
            src = m.get("kv_from")
            if src is not None:
                src = int(src)
                if not 0 <= src < i:
                    raise ConfigError(f"{where}: kv_from names layer {src}, which does not run before it")
                other = self.layers[src]
                om = other["mixer"]
                if other["type"] != kind or om.get("kv_from") is not None:
                    raise ConfigError(f"{where}: kv_from names a layer of another kind, or one without keys of its own")
                if (int(om["heads"]), int(om["kv_heads"]), int(om["dim"]), int(om.get("vdim", om["dim"]))) != (H, G, d, dv):
                    raise ConfigError(f"{where}: kv_from names a layer with other head counts or sizes")
            mlp = layer.get("mlp")
            if mlp is not None:
                ff_kind = _need(mlp, "kind", where + " mlp")
                if ff_kind == "dense":
                    if int(_need(mlp, "ff", where + " mlp")) <= 0 or not float(_need(mlp, "limit", where + " mlp")) > 0:
                        raise ConfigError(f"{where} mlp: ff and limit must be positive")
                elif ff_kind == "moe":
                    r = _need(mlp, "router", where + " mlp")
                    for k in ("experts", "top"):
                        _need(r, k, where + " router")
                    for part in ("expert",) + (("shared",) if mlp.get("shared") else ()):
                        for k in ("ff", "limit"):
                            if not float(_need(_need(mlp, part, where + " mlp"), k, f"{where} {part}")) > 0:
                                raise ConfigError(f"{where} {part}: {k} must be positive")
                    if not 1 <= int(r["top"]) <= int(r["experts"]):
                        raise ConfigError(f"{where} router: top between 1 and experts")
                else:
                    raise ConfigError(f"{where}: feed-forward kind {ff_kind!r} is not built ('dense' and 'moe' are)")

    def summary(self) -> list:
        """(label, value) lines for the command line's report."""
        kinds = [layer["type"] for layer in self.layers]
        heads = [int(layer["mixer"]["heads"]) for layer in self.layers]
        span = lambda xs: str(xs[0]) if len(set(xs)) == 1 else f"{min(xs)}..{max(xs)}"
        return [("Layers", f"{len(self.layers)} (" + ", ".join(f"{kinds.count(k)} {k}" for k in sorted(set(kinds))) + ")"),
                ("Dimensions", self.width), ("Heads", span(heads)), ("Vocab size", self.vocab)]

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
               "layers": copy.deepcopy(list(self.layers)), "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps},
               "vocab": self.vocab, "width": self.width}
        if self.max_positions:
            out["max_positions"] = self.max_positions
        if self.torch_dtype is not None:
            out["torch_dtype"] = self.torch_dtype
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------------ the model as data
    def _norm(self, prefix: str, name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "name": name}, prefix)

    def _kept(self, i: int):
        """What the cache of layer i may give back: its own mask's reach, unless a layer that reads its keys and values
        looks elsewhere; then everything is kept."""
        m = self.layers[i]["mixer"]
        sizes = {int(m["mask"]["size"])} | {int(o["mixer"]["mask"]["size"]) for o in self.layers
                                            if o["mixer"].get("kv_from") is not None and int(o["mixer"]["kv_from"]) == i}
        return int(m["mask"]["size"]) if len(sizes) == 1 else None

    def _mixer(self, i: int, layer: dict) -> PartSpec:
        m, second = layer["mixer"], layer["type"] == "attention_2"
        reads = m.get("kv_from") is not None
        size = int(m["mask"]["size"])
        kept = self._kept(int(m["kv_from"]) if reads else i)
        params = {"hidden_size": self.width, "n_heads": int(m["heads"]), "n_kv_heads": int(m["kv_heads"]),
                  "head_dim": int(m["dim"]), "v_head_dim": int(m.get("vdim", m["dim"])), "scale": float(m["scale"]),
                  "sink": True, "gate": True, "reads_kv": reads,
                  "names": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "sink": "sink", "q_bias": "q.b", "k_bias": "k.b",
                            "v_bias": "v.b", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv"}}
        if second:
            params.update({"block": size, "keep_block": kept, "values": "own", "bias": True, "conv_taps": int(m.get("conv", 0)),
                           "slope_exponent": SLOPE_EXPONENT})
        else:
            params.update({"window": size, "keep_window": kept, "values": "keys"})
        return PartSpec("gated_attention", params, f"l{i}.mix.")

    def _position(self, layer: dict) -> PartSpec | None:
        rot = layer["mixer"].get("rot")
        if layer["type"] != "attention" or rot is None or int(rot["dims"]) == 0:
            return None
        scaling = rot.get("scaling")
        return PartSpec("rope_half", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]),
                                      "head_dim": int(layer["mixer"]["dim"]),
                                      "wavelength_scaling": None if scaling is None else {k: float(scaling[k]) for k in
                                                                                          ("factor", "low", "high", "original")}}, "")

    def _feed_forward(self, p: str, mlp: dict) -> PartSpec:
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"hidden_size": self.width, "intermediate_size": int(mlp["ff"]),
                                          "activation": "clamped_swish", "limit": float(mlp["limit"]), "alpha": SWISH_ALPHA,
                                          "up_shift": UP_SHIFT, "bias": True,
                                          "names": {"gate": "gate", "up": "up", "down": "down", "gate_bias": "gate.b",
                                                    "up_bias": "up.b", "down_bias": "down.b"}}, p + "mlp.")
        r, shared = mlp["router"], mlp.get("shared") or {}
        return PartSpec("routed_experts", {
            "hidden_size": self.width, "n_experts": int(r["experts"]), "expert_ff": int(mlp["expert"]["ff"]),
            "top": int(r["top"]), "correction": False, "shared_ff": int(shared.get("ff", 0)), "shared_gate": bool(shared),
            "gated": True, "activation": "clamped_swish", "limit": float(mlp["expert"]["limit"]),
            "shared_limit": float(shared["limit"]) if shared else None, "alpha": SWISH_ALPHA, "up_shift": UP_SHIFT,
            "routing": "table", "vocab_size": self.vocab,
            "names": {"expert": "e{}.", "shared": "shared.", "shared_gate": "shared.sg", "table": "table"}}, p + "mlp.")

    def _layer_spec(self, i: int, layer: dict) -> LayerSpec:
        p = f"l{i}."
        subs = [SubLayerSpec("mixer", self._mixer(i, layer), self._norm(p, "norm1"), self._norm(p, "norm1b"))]
        if layer.get("mlp") is not None:
            subs.append(SubLayerSpec("feed_forward", self._feed_forward(p, layer["mlp"]), self._norm(p, "norm2"),
                                     self._norm(p, "norm2b")))
        return LayerSpec("sandwich", tuple(subs), self._position(layer))

    def model_spec(self) -> ModelSpec:
        spec = ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "hidden_size": self.width, "name": "embed",
                                             "scale": self.embedding_scale}, ""),
            layers=tuple(self._layer_spec(i, layer) for i, layer in enumerate(self.layers)),
            schedule=tuple(ScheduleEntry(i, None if layer["mixer"].get("kv_from") is None else int(layer["mixer"]["kv_from"]))
                           for i, layer in enumerate(self.layers)),
            final_norm=self._norm("final.", "norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tied": False, "name": "head",
                                      "scale": self.logit_scale}, ""),
            stop_token_ids=self.eos_token_ids)
        spec.validate()
        return spec
