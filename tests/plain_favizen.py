"""A plain implementation of the Favizen decoder: whole sequences, no cache, one function per mechanism, torch on
the CPU in the precision of the tensors it is given (float32 or float64).  It shares no code with the engine.
``round_to`` (a 16-bit type) rounds the activations where a 16-bit engine stores them (the normed rows that enter a
product, q, k and v as they go to the attention, the heads' outputs, a feed-forward's hidden row) and nothing else: the
difference to the unrounded run says how much of a 16-bit engine's error is that rounding alone.

Notation: x is the residual stream [T, width]; N(v) = v / sqrt(mean(v^2) + eps).

    embedding:   x = table[token] * scale
    layer:       x <- x + N(mixer(N(x) w1)) w1b;   x <- x + N(ff(N(x) w2)) w2b      (the second only with a feed-forward)
    attention:   q = W_q h, k = W_k h, v = k (before the rotation); q and k turned by position in pairs (i, i + dims/2)
                 of their first `dims` dimensions; position i sees j with 0 <= i - j < window
    attention_2: q, k, v = W h + b, then a causal convolution over time on every channel; score - slope_h (i - j);
                 position i sees j <= i of its own chunk of positions; a layer may read another layer's k and v
    both:        p = exp(s_j) / (exp(sink_h) + sum_j' exp(s_j'));  o_h = sigmoid(W_g h)_h sum_j p_j v_j;  out = W_o o
    feed-forward: y = g sigmoid(1.702 g) (u + 1), g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down y
    experts:     table[token] names `top` experts of weight 1 / top; a shared expert times sigmoid(W_sg h)
    logits:      W_head (N(x) w) * logit_scale
"""
from __future__ import annotations

import math

import torch


def rounded(t, round_to):
    return t if round_to is None else t.to(round_to).to(t.dtype)


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rope_frequencies(dims: int, base: float, scaling: dict | None, dtype=torch.float64):
    """One frequency for each of the dims / 2 pairs; with ``scaling`` long wavelengths are stretched by ``factor``,
    short ones kept, and those between blended."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    if scaling:
        factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f.tolist():
            wavelength = 2.0 * math.pi / fi
            if wavelength < original / high:
                out.append(fi)
            elif wavelength > original / low:
                out.append(fi / factor)
            else:
                s = (original / wavelength - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=torch.float64)
    return f.to(dtype)


def rotate(x, positions, freqs, dims: int):
    """x [T, heads, d]: dimension i of the first ``dims`` is paired with i + dims / 2."""
    if dims == 0:
        return x
    half = dims // 2
    angle = positions.to(freqs.dtype)[:, None] * freqs[None, :]           # [T, half]
    cos, sin = torch.cos(angle).to(x.dtype)[:, None, :], torch.sin(angle).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def window_mask(n: int, size: int):
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (i - j >= 0) & (i - j < size)


def chunk_mask(n: int, size: int):
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def slopes(heads: int, dtype):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=dtype)


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token."""
    taps = w.shape[1]
    padded = torch.cat([torch.zeros((taps - 1, u.shape[1]), dtype=u.dtype), u], 0)
    return sum(padded[j:j + u.shape[0]] * w[:, j] for j in range(taps))


def sink_attention(q, k, v, scale, visible, sink, distance_slopes=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv], visible [T, T] (row: query).  Returns [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=q.dtype)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if distance_slopes is not None:
            s = s - distance_slopes[h] * (i - j).to(q.dtype)
        s = s.masked_fill(~visible, -math.inf)
        m = torch.maximum(s.max(-1).values, sink[h].expand(T))
        e = torch.exp(s - m[:, None])
        out[:, h] = (e / (e.sum(-1) + torch.exp(sink[h] - m))[:, None]) @ v[:, g]
    return out


def gate_heads(o, h, w_g):
    """o [T, H, dv] times sigmoid(W_g h) [T, H], one number a head."""
    return o * torch.sigmoid(h @ w_g.T)[:, :, None]


def attention_keys_values(h, W, m, round_to=None):
    """The rotary mixer's keys (turned) and values (the keys as projected)."""
    T = h.shape[0]
    k = (h @ W["k"].T).view(T, int(m["kv_heads"]), int(m["dim"]))
    v = k
    rot = m.get("rot")
    if rot and int(rot["dims"]) > 0:
        k = rotate(k, torch.arange(T), rope_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling")), int(rot["dims"]))
    return rounded(k, round_to), rounded(v, round_to)


def attention_mixer(h, W, m, round_to=None, kv=None):
    """The rotary mixer with a sliding window; the values are the keys before their rotation; ``kv``: another layer's."""
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    q = (h @ W["q"].T).view(T, H, d)
    rot = m.get("rot")
    if rot and int(rot["dims"]) > 0:
        q = rotate(q, torch.arange(T), rope_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling")), int(rot["dims"]))
    k, v = kv if kv is not None else attention_keys_values(h, W, m, round_to)
    q = rounded(q, round_to)
    o = sink_attention(q, k, v, float(m["scale"]), window_mask(T, int(m["mask"]["size"])), W["sink"])
    return rounded(gate_heads(o, h, W["g"]), round_to).reshape(T, -1) @ W["o"].T


def attention2_keys_values(h, W, m, round_to=None):
    T = h.shape[0]
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = causal_conv(h @ W["k"].T + W["k.b"], W["k.conv"]).view(T, G, d)
    v = causal_conv(h @ W["v"].T + W["v.b"], W["v.conv"]).view(T, G, dv)
    return rounded(k, round_to), rounded(v, round_to)


def attention2_mixer(h, W, m, kv=None, round_to=None):
    """The convolved mixer with a distance bias over chunks of positions; ``kv``: another layer's keys and values."""
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    q = rounded(causal_conv(h @ W["q"].T + W["q.b"], W["q.conv"]).view(T, H, d), round_to)
    k, v = kv if kv is not None else attention2_keys_values(h, W, m, round_to)
    o = sink_attention(q, k, v, float(m["scale"]), chunk_mask(T, int(m["mask"]["size"])), W["sink"], slopes(H, h.dtype))
    return rounded(gate_heads(o, h, W["g"]), round_to).reshape(T, -1) @ W["o"].T


def clamped_glu(g, u, limit: float):
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def gated_ff(h, W, prefix: str, limit: float, biases: bool, round_to=None):
    b = (lambda n: W[prefix + n + ".b"]) if biases else (lambda n: 0.0)
    y = clamped_glu(h @ W[prefix + "gate"].T + b("gate"), h @ W[prefix + "up"].T + b("up"), limit)
    return rounded(y, round_to) @ W[prefix + "down"].T + b("down")


def table_experts(h, tokens, W, mlp, round_to=None):
    top = int(mlp["router"]["top"])
    chosen = W["table"][tokens].long()                      # [T, top]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += gated_ff(h[t:t + 1], W, f"e{e}.", float(mlp["expert"]["limit"]), False, round_to)[0] / top
    if mlp.get("shared"):
        out = out + gated_ff(h, W, "shared.", float(mlp["shared"]["limit"]), False, round_to) * torch.sigmoid(h @ W["shared.sg"].T)
    return out


def sub(W, prefix):
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def forward(config: dict, W: dict, tokens, layers_out: list | None = None, round_to=None):
    """Logits [T, vocab] of one sequence.  ``W``: tensor name -> tensor (matrices in the dtype to compute in, the
    experts' table as integers).  ``layers_out``: receives the residual stream after every layer."""
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = W["embed"][tokens] * float(config["embedding"]["scale"])
    kept = {}
    for i, layer in enumerate(config["layers"]):
        L, m = sub(W, f"l{i}."), layer["mixer"]
        h = rounded(rms_norm(x, L["norm1"], eps), round_to)
        mix = sub(L, "mix.")
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(h, mix, m, round_to)
            y = attention_mixer(h, mix, m, round_to, kept[i if m.get("kv_from") is None else int(m["kv_from"])])
        elif layer["type"] == "attention_2":
            if m.get("kv_from") is not None:
                y = attention2_mixer(h, mix, m, kept[int(m["kv_from"])], round_to)
            else:
                kept[i] = attention2_keys_values(h, mix, m, round_to)
                y = attention2_mixer(h, mix, m, kept[i], round_to)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, L["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rounded(rms_norm(x, L["norm2"], eps), round_to)
            f = sub(L, "mlp.")
            y = gated_ff(h, f, "", float(mlp["limit"]), True, round_to) if mlp["kind"] == "dense" else \
                table_experts(h, tokens, f, mlp, round_to)
            x = x + rms_norm(y, L["norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rounded(rms_norm(x, W["final.norm"], eps), round_to) @ W["head"].T) * float(config.get("logit_scale", 1.0))
