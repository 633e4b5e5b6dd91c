"""A plain, slow implementation of the Dupolorn decoder: whole sequences, no cache, one function per mechanism,
in whatever float type the tensors have (float64 for references).  It shares no code with the library; keys and
values of the latent attention are formed head by head from the latent, as the design states them."""
import math

import torch


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_scalar(x, g, eps):
    """RMS norm whose weight is one number."""
    return rms_div(x, eps) * g


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def relu2(z):
    return torch.relu(z) ** 2


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token of one sequence: the first takes row ``buckets``."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * mul_prev + cur * mul_cur) % buckets)
    return rows


def embedding(W, cfg, tokens):
    b = cfg["embedding"]["bigram"]
    rows = bigram_rows(list(tokens), b["buckets"], b["mul_prev"], b["mul_cur"])
    return W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"] + W["bigram"][torch.tensor(rows)]


def rotate(x, positions, base, dims):
    """Adjacent pairs (2i, 2i + 1) of the first ``dims`` of the last axis turned by positions[t] * base^(-2i/dims);
    x [T, ..., n]."""
    out = x.clone()
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        a = torch.tensor([p * f for p in positions], dtype=x.dtype)
        while a.dim() < x.dim() - 1:
            a = a.unsqueeze(-1)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., 2 * i + 1] = v * torch.cos(a) + u * torch.sin(a)
    return out


def canon(h, w):
    """h + causal convolution over time per channel; w [width, taps], the last column the current token's."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] = out[t] + w[:, j] * h[s]
    return out


def latent_attention(h, W, m, eps, second, positions=None, store=None):
    """W: local name -> tensor (q, dkv, dkv.norm, uk, uv, o, and for the second kind sink, g).  ``store``: a 16-bit type
    whose values the latent, the rotated key part and the queries take (what a 16-bit cache holds)."""
    T = h.shape[0]
    H, d, rd, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = list(range(T)) if positions is None else positions
    rnd = (lambda x: x.to(store).to(h.dtype)) if store is not None else (lambda x: x)
    q = (h @ W["q"].T).view(T, H, d + rd)
    dkv = h @ W["dkv"].T
    c = rnd(rms_div(dkv[:, :r], eps) * W["dkv.norm"])
    base, dims = (m["rot"]["base"], m["rot"]["dims"]) if rd else (1.0, 0)
    k_rot = rnd(rotate(dkv[:, r:], positions, base, dims))
    q_rot = rnd(rotate(q[..., d:], positions, base, dims))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        k = c @ W["uk"][hd * d:(hd + 1) * d].T                       # [T, d]
        v = c @ W["uv"][hd * dv:(hd + 1) * dv].T                     # [T, dv]
        for t in range(T):
            s = (k[:t + 1] @ q[t, hd, :d] + k_rot[:t + 1] @ q_rot[t, hd]) * m["scale"]
            if second:
                s = torch.cat([s, W["sink"][hd].reshape(1)])
            p = torch.softmax(s, 0)
            out[t, hd] = p[:t + 1] @ v[:t + 1]
    o = out.reshape(T, H * dv)
    if second:
        o = o * torch.sigmoid(h @ W["g"].T)
    return o @ W["o"].T


def mlstm(h, W, m, eps, state=None):
    """W: q, k, v, g, o, norm, i, i.b, f, f.b.  Returns the mixer's output (and leaves the state in ``state``)."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W["k"].T).view(T, H, d)
    v = (h @ W["v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ W["i"].T + W["i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W["f"].T + W["f.b"]) / cap))
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    n = torch.zeros(H, d, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    ys = []
    for t in range(T):
        new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - new), torch.exp(ig[t] - new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        ys.append(torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None])
    if state is not None:
        state.update(S=S, n=n, m=mx)
    y = rms_div(torch.stack(ys), eps).reshape(T, H * dv) * W["norm"] * torch.sigmoid(h @ W["g"].T)
    return y @ W["o"].T


def dense_ff(h, W):
    return (gelu_tanh(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def router_scores(h, W):
    return torch.sigmoid(h @ W["router"].T)


def moe_ff(h, W, mlp, chosen=None):
    """``chosen``: a list that receives every token's chosen experts."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = router_scores(h, W)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        picked = torch.topk(s[t], top).indices.tolist()
        if chosen is not None:
            chosen.append(picked)
        for e in picked:
            x = s[t, e] * h[t]                                       # the weight on the expert's input
            out[t] = out[t] + relu2(x @ W[f"e{e}.up"].T) @ W[f"e{e}.down"].T
    if mlp.get("shared"):
        out = out + relu2(h @ W["shared.up"].T) @ W["shared.down"].T
    return out


def local(W, prefix):
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def layers(W, cfg, tokens):
    """The stream's values X_0 .. X_L and the stream after every layer's depth average."""
    eps = cfg["norm"]["eps"]
    x = embedding(W, cfg, tokens)
    X, after = [x], []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h1 = canon(norm_scalar(x, W[p + "norm1"], eps), W[p + "canon1"])
        if L["type"] == "mlstm":
            y = x + mlstm(h1, local(W, p + "mix."), L["mixer"], eps)
        else:
            y = x + latent_attention(h1, local(W, p + "mix."), L["mixer"], eps, L["type"] == "latent_attention_2")
        if L["mlp"] is not None:
            h2 = norm_scalar(x, W[p + "norm2"], eps)
            y = y + (dense_ff(h2, local(W, p + "mlp.")) if L["mlp"]["kind"] == "dense" else moe_ff(h2, local(W, p + "mlp."), L["mlp"]))
        X.append(y)
        x = sum(W[p + "dwa"][j] * X[j] for j in range(i + 2))
        after.append(x)
    return X, after


def forward(W, cfg, tokens):
    """Logits [T, vocab] of one sequence."""
    x = layers(W, cfg, tokens)[1][-1]
    logits = norm_scalar(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return logits if cap is None else cap * torch.tanh(logits / cap)
