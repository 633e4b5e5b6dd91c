"""Typed configuration of the Dupolorn decoder, read from its own config.json keys.

A model of this design is a list of parallel layers over a float32 residual stream of ``width``: both the mixer and
the feed-forward read the same x, each through an RMS norm whose weight is a single number (``norm.eps``), and
x + mixer(norm1(x)) + ff(norm2(x)) is the layer's result.  What the mixer reads first passes a short causal
convolution over time beside itself (``canon.taps`` taps, tensor ``l<i>.canon1`` [width, taps]).  What goes on to
the next layer (and after the last one to the output) is a weighted average over depth of the embedding's output
and all layers' results so far (``l<i>.dwa``, i + 2 weights after layer i).

``layers[i].type`` names the mixer, ``layers[i].mixer`` its sizes:

* ``latent_attention``: softmax attention over one latent per token (``heads``, ``dim`` unrotated and ``rot_dim``
  rotated query/key dimensions a head, ``vdim``, ``kv_rank``, ``scale``, ``rot`` {``base``, ``dims``}: rotation of
  adjacent pairs of the first ``dims`` rotated dimensions);
* ``latent_attention_2``: the same with a learned sink in every head's softmax sum and a sigmoid gate on the heads'
  outputs;
* ``mlstm``: the matrix memory (``heads``, ``dim``, ``vdim``, ``gate_cap``).

``layers[i].mlp`` is null, ``{"kind": "dense", "ff"}`` (down(gelu_tanh(gate) * up)) or ``{"kind": "moe", "expert":
{"ff"}, "router": {"experts", "top"}, "shared": {"ff"}}``: experts down(relu(up)^2) without biases, sigmoid scores, the
``top`` largest chosen, their scores as weights (not renormalised) on the experts' inputs, a shared expert of the
same form for every token.  The embedding is ``embed[token] * embedding.scale`` plus a row of the hashed ``bigram``
table (``embedding.bigram`` {``buckets``, ``mul_prev``, ``mul_cur``}).  The logits pass ``logit_softcap * tanh(. /
logit_softcap)``.  Tensor names: ``embed``, ``bigram``, ``final.norm``, ``head``, and per layer ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.canon1``, ``l<i>.dwa``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, SubLayerSpec

_DTYPES = ("float32", "float16", "bfloat16")
_ATTENTION = ("latent_attention", "latent_attention_2")


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json: {where} lacks '{key}'")
    return d[key]


@dataclass(frozen=True)
class DupolornConfig:
    width: int
    vocab: int
    norm_eps: float
    embedding_scale: float
    bigram: dict                    # {"buckets", "mul_prev", "mul_cur"}
    canon_taps: int
    layers: tuple                   # the layers as config.json lists them (plain dicts)
    logit_softcap: float | None = None
    max_positions: int = 0          # the design sets no bound; an optional key may
    torch_dtype: str | None = None
    eos_token_ids: tuple = ()
    architecture: str = "Dupolorn"

    context_key = "max_positions"

    @classmethod
    def from_dict(cls, c: dict) -> "DupolornConfig":
        layers = _need(c, "layers", "the model")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        eos = c.get("eos_token_id")
        emb = _need(c, "embedding", "the model")
        cap = c.get("logit_softcap")
        cfg = cls(width=int(_need(c, "width", "the model")), vocab=int(_need(c, "vocab", "the model")),
                  norm_eps=float(_need(_need(c, "norm", "the model"), "eps", "norm")),
                  embedding_scale=float(emb.get("scale", 1.0)), bigram=copy.deepcopy(_need(emb, "bigram", "embedding")),
                  canon_taps=int(_need(_need(c, "canon", "the model"), "taps", "canon")),
                  layers=tuple(copy.deepcopy(layers)), logit_softcap=None if cap is None else float(cap),
                  max_positions=int(c.get("max_positions") or 0), torch_dtype=c.get("torch_dtype"),
                  eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=c.get("architecture") or (c.get("architectures") or ["Dupolorn"])[0])
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.width <= 0 or self.vocab <= 0:
            raise ConfigError("width and vocab must be positive")
        if not self.norm_eps >= 0:
            raise ConfigError("norm.eps must not be negative")
        if self.torch_dtype is not None and self.torch_dtype not in _DTYPES:
            raise ConfigError(f"Unsupported torch_dtype: {self.torch_dtype}")
        for k in ("buckets", "mul_prev", "mul_cur"):
            _need(self.bigram, k, "embedding.bigram")
        if int(self.bigram["buckets"]) < 1:
            raise ConfigError("embedding.bigram.buckets must be positive")
        if not 1 <= self.canon_taps <= 16:
            raise ConfigError("canon.taps: 1 to 16")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError("logit_softcap must be positive")
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            kind, m = _need(layer, "type", where), _need(layer, "mixer", where)
            if kind in _ATTENTION:
                for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale"):
                    _need(m, k, where + " mixer")
                if int(m["rot_dim"]) > 0:
                    rot = _need(m, "rot", where + " mixer")
                    dims = int(_need(rot, "dims", where + " rot"))
                    _need(rot, "base", where + " rot")
                    if dims % 2 or not 0 <= dims <= int(m["rot_dim"]):
                        raise ConfigError(f"{where}: rot.dims must be even and at most rot_dim")
                if min(int(m["heads"]), int(m["vdim"]), int(m["kv_rank"])) < 1 or int(m["dim"]) + int(m["rot_dim"]) < 1:
                    raise ConfigError(f"{where}: heads, vdim, kv_rank and dim + rot_dim must be positive")
            elif kind == "mlstm":
                for k in ("heads", "dim", "vdim", "gate_cap"):
                    _need(m, k, where + " mixer")
                if min(int(m["heads"]), int(m["dim"]), int(m["vdim"])) < 1 or not float(m["gate_cap"]) > 0:
                    raise ConfigError(f"{where}: heads, dim, vdim and gate_cap must be positive")
            else:
                raise ConfigError(f"{where}: mixer type {kind!r} is not built ({', '.join(_ATTENTION)} and 'mlstm' are)")
            mlp = layer.get("mlp")
            if mlp is not None:
                ff_kind = _need(mlp, "kind", where + " mlp")
                if ff_kind == "dense":
                    if int(_need(mlp, "ff", where + " mlp")) <= 0:
                        raise ConfigError(f"{where} mlp: ff must be positive")
                elif ff_kind == "moe":
                    r = _need(mlp, "router", where + " mlp")
                    for k in ("experts", "top"):
                        _need(r, k, where + " router")
                    _need(_need(mlp, "expert", where + " mlp"), "ff", where + " expert")
                    if not 1 <= int(r["top"]) <= int(r["experts"]):
                        raise ConfigError(f"{where} router: top between 1 and experts")
                    if mlp.get("shared"):
                        _need(mlp["shared"], "ff", where + " shared")
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
        out = {"architecture": self.architecture, "canon": {"taps": self.canon_taps},
               "embedding": {"bigram": copy.deepcopy(self.bigram), "scale": self.embedding_scale},
               "layers": copy.deepcopy(list(self.layers)), "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
               "width": self.width}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.max_positions:
            out["max_positions"] = self.max_positions
        if self.torch_dtype is not None:
            out["torch_dtype"] = self.torch_dtype
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------------ the model as data
    def _norm(self, prefix: str, name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "name": name, "scalar": True}, prefix)

    def _mixer(self, p: str, layer: dict) -> PartSpec:
        m, w, eps = layer["mixer"], self.width, self.norm_eps
        if layer["type"] == "mlstm":
            inner = PartSpec("mlstm", {
                "hidden_size": w, "n_heads": int(m["heads"]), "head_dim": int(m["dim"]), "v_head_dim": int(m["vdim"]),
                "gate_cap": float(m["gate_cap"]), "norm_eps": eps,
                "names": {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "i_bias": "i.b",
                          "f": "f", "f_bias": "f.b"}}, p + "mix.")
        else:
            second = layer["type"] == "latent_attention_2"
            inner = PartSpec("latent_attention", {
                "hidden_size": w, "n_heads": int(m["heads"]), "head_dim": int(m["dim"]), "rot_dim": int(m["rot_dim"]),
                "v_head_dim": int(m["vdim"]), "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "norm_eps": eps,
                "sink": second, "gate": second,
                "names": {"q": "q", "dkv": "dkv", "kv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "sink": "sink",
                          "g": "g"}}, p + "mix.")
        return PartSpec("short_conv", {"hidden_size": w, "taps": self.canon_taps, "inner": inner, "name": "canon1"}, p)

    def _position(self, layer: dict) -> PartSpec | None:
        m = layer["mixer"]
        if layer["type"] not in _ATTENTION or int(m["rot_dim"]) == 0 or int(m["rot"]["dims"]) == 0:
            return None
        return PartSpec("rope", {"theta": float(m["rot"]["base"]), "rotary_dim": int(m["rot"]["dims"]),
                                 "head_dim": int(m["rot_dim"]), "pairing": "adjacent"}, "")

    def _feed_forward(self, p: str, mlp: dict) -> PartSpec:
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"hidden_size": self.width, "intermediate_size": int(mlp["ff"]), "activation": "gelu",
                                          "names": {"gate": "gate", "up": "up", "down": "down"}}, p + "mlp.")
        r, shared = mlp["router"], mlp.get("shared") or {}
        return PartSpec("routed_experts", {
            "hidden_size": self.width, "n_experts": int(r["experts"]), "expert_ff": int(mlp["expert"]["ff"]),
            "top": int(r["top"]), "correction": False, "shared_ff": int(shared.get("ff", 0)), "shared_gate": False,
            "gated": False, "activation": "relu2", "scores": "sigmoid", "renormalize": False, "weight_on": "input",
            "names": {"router": "router", "expert": "e{}.", "shared": "shared."}}, p + "mlp.")

    def _layer_spec(self, i: int, layer: dict) -> LayerSpec:
        p = f"l{i}."
        subs = [SubLayerSpec("mixer", self._mixer(p, layer), self._norm(p, "norm1"))]
        if layer.get("mlp") is not None:
            subs.append(SubLayerSpec("feed_forward", self._feed_forward(p, layer["mlp"]), self._norm(p, "norm2")))
        return LayerSpec("parallel", tuple(subs), self._position(layer))

    def model_spec(self) -> ModelSpec:
        b = self.bigram
        spec = ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            embedding=PartSpec("bigram_embedding", {"vocab_size": self.vocab, "hidden_size": self.width,
                                                    "buckets": int(b["buckets"]), "mul_prev": int(b["mul_prev"]),
                                                    "mul_cur": int(b["mul_cur"]), "scale": self.embedding_scale,
                                                    "names": {"table": "embed", "bigram": "bigram"}}, ""),
            layers=tuple(self._layer_spec(i, layer) for i, layer in enumerate(self.layers)),
            schedule=tuple(ScheduleEntry(i, None, None, PartSpec("depth_average", {"n_terms": i + 2, "name": "dwa"}, f"l{i}."))
                           for i in range(len(self.layers))),
            final_norm=self._norm("final.", "norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "hidden_size": self.width, "tied": False, "name": "head",
                                      "softcap": self.logit_softcap}, ""),
            stop_token_ids=self.eos_token_ids)
        spec.validate()
        return spec
