"""Small Dupolorn configurations, random weights for them, and model folders: for the tests only, written without
the library (the safetensors package writes the files)."""
import json
import os

import torch


def latent(heads, dim, rot_dim, vdim, kv_rank, second=False, base=10000.0, dims=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}
    if rot_dim:
        m["rot"] = {"base": base, "dims": rot_dim if dims is None else dims}
    return "latent_attention_2" if second else "latent_attention", m


def mlstm(heads, dim, vdim, cap=15.0):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(width, vocab, layers, taps=3, eps=1e-5, scale=1.0, bigram=(97, 31, 7), softcap=20.0):
    out = {"architecture": "Dupolorn", "canon": {"taps": taps},
           "embedding": {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}, "scale": scale},
           "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if softcap is not None:
        out["logit_softcap"] = softcap
    return out


# a matrix memory first, a layer without feed-forward, three heads with 20 + 6 query dimensions of which 4 are rotated,
# values 36 wide over a latent of 40; two of five experts chosen beside a shared one; two taps
TINY_A = config(96, 131, [
    layer(mlstm(3, 20, 24, cap=9.0), dense(72)),
    layer(latent(3, 20, 6, 36, 40, second=True, base=500.0, dims=4), moe(5, 2, 40, shared=24)),
    layer(latent(2, 8, 16, 16, 24), None),
    layer(mlstm(1, 33, 70), moe(3, 1, 56)),
], taps=2, eps=1e-6, scale=2.5, bigram=(53, 11, 29))

# a width that the matrix kernels cannot tile; one head; no rotated part at all in one layer and no unrotated part in
# another; five taps; no soft cap; a latent wider than a head's keys
TINY_B = config(72, 97, [
    layer(latent(1, 16, 0, 8, 72, second=True), dense(40)),
    layer(latent(4, 0, 32, 24, 16, base=77.0), moe(9, 4, 8, shared=16)),
    layer(mlstm(4, 16, 16, cap=30.0), moe(2, 2, 24)),
], taps=5, eps=1e-4, scale=1.0, bigram=(1, 3, 5), softcap=None)

# sizes of real layers, few of them: a latent of 192 with a rotated part of 64, eight heads of 64 + 64; a matrix memory of
# 128 x 128 a head; one tap (the convolution is a weight on the input itself)
TINY_C = config(256, 211, [
    layer(latent(8, 64, 64, 64, 192, second=True, base=10000.0), moe(4, 2, 96, shared=64)),
    layer(mlstm(2, 128, 128, cap=11.0), dense(320)),
    layer(latent(4, 32, 16, 48, 320), dense(128)),
], taps=1, eps=1e-5, scale=3.0, bigram=(509, 101, 13), softcap=25.0)

ALL = {"A": TINY_A, "B": TINY_B, "C": TINY_C}


def mixer_weights(kind, m, w, g, dtype, sharp=1.0):
    """local name -> tensor of one mixer."""
    mat = lambda n, k, s=None: (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)
    vec = lambda n, mean, s: (mean + s * torch.randn(n, generator=g)).to(dtype)
    H = m["heads"]
    if kind == "mlstm":
        d, dv = m["dim"], m["vdim"]
        return {"q": mat(H * d, w, sharp * w ** -0.5), "k": mat(H * d, w, sharp * w ** -0.5), "v": mat(H * dv, w), "g": mat(H * dv, w),
                "o": mat(w, H * dv), "norm": vec(H * dv, 1.0, 0.2), "i": mat(H, w, 2.0 * w ** -0.5), "i.b": vec(H, 0.0, 0.5),
                "f": mat(H, w, 2.0 * w ** -0.5), "f.b": vec(H, 2.0, 1.0)}
    d, rd, dv, r = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    out = {"q": mat(H * (d + rd), w, sharp * w ** -0.5), "dkv": mat(r + rd, w, sharp * w ** -0.5), "dkv.norm": vec(r, 1.0, 0.2),
           "uk": mat(H * d, r), "uv": mat(H * dv, r), "o": mat(w, H * dv)}
    if kind == "latent_attention_2":
        out.update({"sink": vec(H, 0.5, 1.0), "g": mat(H * dv, w)})
    return out


def mlp_weights(mlp, w, g, dtype):
    mat = lambda n, k, s=None: (torch.randn(n, k, generator=g) * (s if s is not None else k ** -0.5)).to(dtype)
    if mlp["kind"] == "dense":
        return {"gate": mat(mlp["ff"], w), "up": mat(mlp["ff"], w), "down": mat(w, mlp["ff"])}
    ff = mlp["expert"]["ff"]
    out = {"router": mat(mlp["router"]["experts"], w, 2.0 * w ** -0.5)}
    for e in range(mlp["router"]["experts"]):
        out.update({f"e{e}.up": mat(ff, w), f"e{e}.down": mat(w, ff)})
    if mlp.get("shared"):
        out.update({"shared.up": mat(mlp["shared"]["ff"], w), "shared.down": mat(w, mlp["shared"]["ff"])})
    return out


def random_weights(cfg, seed, dtype=torch.bfloat16, sharp=1.0):
    """name -> tensor as a file of the design holds it.  ``sharp`` scales the query and key matrices."""
    g = torch.Generator().manual_seed(seed)
    w, V, L = cfg["width"], cfg["vocab"], len(cfg["layers"])
    one = lambda mean, s: (mean + s * torch.randn((), generator=g)).to(dtype)
    out = {"embed": torch.randn(V, w, generator=g).to(dtype),
           "bigram": (0.7 * torch.randn(cfg["embedding"]["bigram"]["buckets"] + 1, w, generator=g)).to(dtype),
           "final.norm": one(1.0, 0.1), "head": (torch.randn(V, w, generator=g) * w ** -0.5).to(dtype)}
    for i, layer_ in enumerate(cfg["layers"]):
        p = f"l{i}."
        out[p + "norm1"] = one(1.0, 0.2)
        out[p + "canon1"] = (0.4 * torch.randn(w, cfg["canon"]["taps"], generator=g)).to(dtype)
        out[p + "dwa"] = ((1.0 + 0.3 * torch.randn(i + 2, generator=g)) / (i + 2) * 1.5).to(dtype)
        out.update({p + "mix." + k: v for k, v in mixer_weights(layer_["type"], layer_["mixer"], w, g, dtype, sharp).items()})
        if layer_["mlp"] is not None:
            out[p + "norm2"] = one(1.0, 0.2)
            out.update({p + "mlp." + k: v for k, v in mlp_weights(layer_["mlp"], w, g, dtype).items()})
    return out


def write_model(folder, cfg, weights):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))


def widen(weights, dtype=torch.float64):
    return {k: v.to(dtype) for k, v in weights.items()}


def row_error(got, ref):
    """For each row the root mean square of the difference (its mean taken off), relative to the reference's own
    spread: the measure by which logits are compared."""
    d = got.double() - ref.double()
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.double().std()).max().item()
