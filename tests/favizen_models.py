"""Small Favizen configurations, random weights for them, and model folders: for the tests only, written without
the library (the safetensors package writes the files)."""
import json
import os

import torch


def rotary(heads, kv_heads, dim, window, dims=None, base=10000.0, scaling=None, scale=None, kv_from=None):
    """The mixer with a rotation, a sliding window and values that are the keys."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window},
         "scale": dim ** -0.5 if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    dims = dim if dims is None else dims
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if scaling is not None:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return "attention", m


def convolved(heads, kv_heads, dim, vdim, chunk, taps=3, kv_from=None, scale=None):
    """The mixer with biases, short convolutions, a bias by distance and chunks of positions."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk}, "conv": taps,
         "scale": dim ** -0.5 if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention_2", m


def dense(ff, limit=1.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, limit=2.0, shared=None, shared_limit=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared, "limit": limit if shared_limit is None else shared_limit}
    return out


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, scale=1.0, logit_scale=1.0):
    return {"architecture": "Favizen", "embedding": {"scale": scale}, "layers": layers, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


# three query heads on one key head with 20 dimensions of which 12 are turned, a window of 9; a layer without
# feed-forward; two of five experts beside a shared one with another limit; a chunk of 50 read by a later layer with two
# taps; values wider than keys
TINY_A = config(96, 131, [
    layer(rotary(3, 1, 20, 9, dims=12, base=500.0), dense(72, limit=0.7)),
    layer(convolved(4, 2, 16, 24, 50, taps=2), moe(5, 2, 40, limit=1.5, shared=24, shared_limit=0.5)),
    layer(rotary(2, 2, 32, 70, scaling=(4.0, 1.0, 3.0, 64)), None),
    layer(convolved(4, 2, 16, 24, 50, taps=2, kv_from=1), moe(3, 1, 56)),
], eps=1e-6, scale=2.5, logit_scale=0.25)

# a width that the matrix kernels cannot tile; one head; no rotation at all in one layer; five taps and one tap; a layer
# that reads keys through another mask than their owner's (of either kind); every expert chosen; no shared expert
TINY_B = config(72, 97, [
    layer(convolved(1, 1, 8, 40, 7, taps=5), dense(40, limit=3.0)),
    layer(rotary(4, 4, 16, 1000, dims=0), moe(4, 4, 8)),
    layer(convolved(1, 1, 8, 40, 33, taps=1, kv_from=0), moe(9, 3, 16, shared=16)),
    layer(rotary(6, 2, 48, 33, dims=16, base=77.0, scaling=(6.0, 1.0, 3.0, 32)), dense(24)),
    layer(rotary(6, 2, 48, 90, dims=16, base=77.0, scaling=(6.0, 1.0, 3.0, 32), kv_from=3), None),
], eps=1e-4, scale=1.0, logit_scale=3.0)

# sizes of real layers, few of them: eight heads of 64 on two key heads, sixteen heads of 128 on one; windows and chunks
# beyond a page
TINY_C = config(256, 211, [
    layer(convolved(16, 1, 128, 64, 130, taps=4), moe(4, 2, 96, shared=64)),
    layer(rotary(8, 2, 64, 100, base=2e5, scaling=(16.0, 1.0, 2.0, 128)), dense(320)),
    layer(convolved(16, 1, 128, 64, 130, taps=4, kv_from=0), dense(128, limit=7.0)),
], eps=1e-5, scale=3.0, logit_scale=0.5)

ALL = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def mixer_weights(kind, m, w, g, dtype, sharp=1.0):
    """local name -> tensor of one mixer."""
    mat = lambda n, k, s=None: (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)
    vec = lambda n, mean, s: (mean + s * torch.randn(n, generator=g)).to(dtype)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    out = {"q": mat(H * d, w, sharp * w ** -0.5), "sink": vec(H, 0.5, 1.0), "g": mat(H, w, 2.0 * w ** -0.5), "o": mat(w, H * dv)}
    own = m.get("kv_from") is None
    if own:
        out["k"] = mat(G * d, w, sharp * w ** -0.5)
    if kind == "attention_2":
        taps = m["conv"]
        rows = {"q": H * d}
        if own:
            out["v"] = mat(G * dv, w)
            rows.update({"k": G * d, "v": G * dv})
        for name, n in rows.items():
            out[name + ".b"] = vec(n, 0.0, 0.3)
            out[name + ".conv"] = (torch.randn(n, taps, generator=g) * 0.6).to(dtype)
    return out


def mlp_weights(mlp, w, vocab, g, dtype):
    mat = lambda n, k, s=None: (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)
    vec = lambda n, s: (s * torch.randn(n, generator=g)).to(dtype)
    if mlp["kind"] == "dense":
        f = mlp["ff"]
        return {"gate": mat(f, w, 2.0 * w ** -0.5), "up": mat(f, w, 2.0 * w ** -0.5), "down": mat(w, f), "gate.b": vec(f, 0.3),
                "up.b": vec(f, 0.3), "down.b": vec(w, 0.3)}
    ff, E, top = mlp["expert"]["ff"], mlp["router"]["experts"], mlp["router"]["top"]
    out = {"table": torch.rand(vocab, E, generator=g).argsort(-1)[:, :top].to(torch.int32).contiguous()}
    for e in range(E):
        out.update({f"e{e}.gate": mat(ff, w, 2.0 * w ** -0.5), f"e{e}.up": mat(ff, w, 2.0 * w ** -0.5), f"e{e}.down": mat(w, ff)})
    if mlp.get("shared"):
        f = mlp["shared"]["ff"]
        out.update({"shared.gate": mat(f, w, 2.0 * w ** -0.5), "shared.up": mat(f, w, 2.0 * w ** -0.5), "shared.down": mat(w, f),
                    "shared.sg": mat(1, w, 2.0 * w ** -0.5)})
    return out


def random_weights(cfg, seed, dtype=torch.bfloat16, sharp=1.0):
    """name -> tensor as a file of the design holds it.  ``sharp`` scales the query and key matrices."""
    g = torch.Generator().manual_seed(seed)
    w, V = cfg["width"], cfg["vocab"]
    vec = lambda mean, s: (mean + s * torch.randn(w, generator=g)).to(dtype)
    out = {"embed": torch.randn(V, w, generator=g).to(dtype), "final.norm": vec(1.0, 0.1),
           "head": (torch.randn(V, w, generator=g) * w ** -0.5).to(dtype)}
    for i, layer_ in enumerate(cfg["layers"]):
        p = f"l{i}."
        out[p + "norm1"], out[p + "norm1b"] = vec(1.0, 0.2), vec(0.7, 0.2)
        out.update({p + "mix." + k: v for k, v in mixer_weights(layer_["type"], layer_["mixer"], w, g, dtype, sharp).items()})
        if layer_["mlp"] is not None:
            out[p + "norm2"], out[p + "norm2b"] = vec(1.0, 0.2), vec(0.7, 0.2)
            out.update({p + "mlp." + k: v for k, v in mlp_weights(layer_["mlp"], w, V, g, dtype).items()})
    return out


def stand_out(weights, cfg, i, token, strength=6.0):
    """Makes the key of ``token`` stand out for every query of layer i, in place: every embedding row gets a common
    component along axis 0, the last dimension of every query head reads that axis, and the last dimension of every key
    head reads the direction of the token's own embedding row (as the layer's first norm leaves it)."""
    m, w = cfg["layers"][i]["mixer"], cfg["width"]
    d = m["dim"]
    assert m.get("rot") is None or m["rot"]["dims"] < d, "the last dimension must not be turned"
    dt = weights["embed"].dtype
    e = weights["embed"].double()
    e[:, 0] = 3.0
    weights["embed"] = e.to(dt)
    n1 = weights[f"l{i}.norm1"].double()
    e = weights["embed"].double()                          # as rounded
    own = e[token] / e[token].norm()
    q, k = weights[f"l{i}.mix.q"].double(), weights[f"l{i}.mix.k"].double()
    for h in range(m["heads"]):
        q[h * d + d - 1] = 0.0
        q[h * d + d - 1, 0] = strength / n1[0]
    others = e.mean(0) / e.mean(0).norm()
    direction = own - (own @ others) * others              # what the token has and the average row has not
    for g_ in range(m["kv_heads"]):
        k[g_ * d + d - 1] = strength * direction / n1
    weights[f"l{i}.mix.q"], weights[f"l{i}.mix.k"] = q.to(dt), k.to(dt)
    return weights


def write_model(folder, cfg, weights):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))


def widen(weights, dtype=torch.float64):
    return {k: (v if not v.dtype.is_floating_point else v.to(dtype)) for k, v in weights.items()}


def with_mask(cfg, i, size):
    """The configuration with another mask size in layer i."""
    out = json.loads(json.dumps(cfg))
    out["layers"][i]["mixer"]["mask"]["size"] = size
    return out


def row_error(got, ref):
    """For each row the root mean square of the difference (its mean taken off), relative to the reference's own
    spread: the measure by which logits are compared.  The largest over the rows."""
    d = got.double() - ref.double()
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.double().std()).max().item()


def tolerance(dtype, ref, ref_rounded=None, measure=row_error):
    """What a run in ``dtype`` may differ from the plain implementation's ``ref``: 1e-4 of its spread in float32; in
    bfloat16 3e-2, or three times what rounding the activations where a 16-bit engine stores them does to the plain
    implementation itself (``ref_rounded``), if that is more."""
    if dtype == "float32":
        return 1e-4
    return max(3e-2, 3.0 * measure(ref_rounded, ref)) if ref_rounded is not None else 3e-2
