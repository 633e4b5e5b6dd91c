"""Dupolorn without a GPU: the plain implementation pinned by library routines, closed forms and invariants; the
configuration's reading, the tensor table, and what the model asks of the cache."""
import math

import pytest
import torch

import dupolorn_models as M
import plain_dupolorn as P


def test_scalar_norm_and_activations():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 40, generator=g, dtype=torch.float64) * 3
    ref = torch.nn.functional.rms_norm(x, (40,), eps=1e-3) * 1.7
    assert (P.norm_scalar(x, torch.tensor(1.7, dtype=torch.float64), 1e-3) - ref).abs().max() < 1e-12
    assert (P.gelu_tanh(x) - torch.nn.functional.gelu(x, approximate="tanh")).abs().max() < 1e-12
    assert (P.relu2(x) - torch.relu(x) ** 2).abs().max() == 0 and P.relu2(torch.tensor(-2.0)) == 0


def test_bigram_rows():
    assert P.bigram_rows([5, 9, 2], 7, 3, 10) == [7, (5 * 3 + 9 * 10) % 7, (9 * 3 + 2 * 10) % 7]
    assert P.bigram_rows([4], 11, 1, 1) == [11]


def test_rotation_is_a_rotation_of_adjacent_pairs():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 3, 10, generator=g, dtype=torch.float64)
    y = P.rotate(x, [0, 1, 2, 50, 700, 7000], 100.0, 6)
    assert (y[0] - x[0]).abs().max() == 0                                      # position 0 turns nothing
    assert (y[..., 6:] - x[..., 6:]).abs().max() == 0                          # the rest passes
    pairs = lambda z: z[..., :6].reshape(6, 3, 3, 2).pow(2).sum(-1)
    assert (pairs(y) - pairs(x)).abs().max() < 1e-12                           # a pair keeps its length
    a = 700 * 100.0 ** (-2 / 6)
    assert abs(y[4, 1, 2] - (x[4, 1, 2] * math.cos(a) - x[4, 1, 3] * math.sin(a))) < 1e-12
    # a score depends on the distance only
    q, k = torch.randn(1, 6, generator=g, dtype=torch.float64), torch.randn(1, 6, generator=g, dtype=torch.float64)
    s = lambda pq, pk: (P.rotate(q, [pq], 50.0, 6) * P.rotate(k, [pk], 50.0, 6)).sum()
    assert abs(s(17, 5) - s(112, 100)) < 1e-10


def test_canon_against_conv1d():
    g = torch.Generator().manual_seed(2)
    h, w = torch.randn(9, 5, generator=g, dtype=torch.float64), torch.randn(5, 4, generator=g, dtype=torch.float64)
    conv = torch.nn.functional.conv1d(torch.nn.functional.pad(h.T[None], (3, 0)), w[:, None, :], groups=5)[0].T
    assert (P.canon(h, w) - (h + conv)).abs().max() < 1e-12


def test_latent_attention_against_scaled_dot_product():
    g = torch.Generator().manual_seed(3)
    m = M.latent(2, 8, 0, 6, 12)[1]
    W = M.widen(M.mixer_weights("latent_attention", m, 16, g, torch.float32))
    h = torch.randn(7, 16, generator=g, dtype=torch.float64)
    c = P.rms_div(h @ W["dkv"].T, 1e-5) * W["dkv.norm"]
    q = (h @ W["q"].T).view(7, 2, 8).transpose(0, 1)
    k = (c @ W["uk"].T).view(7, 2, 8).transpose(0, 1)
    v = (c @ W["uv"].T).view(7, 2, 6).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=m["scale"]).transpose(0, 1).reshape(7, 12)
    assert (P.latent_attention(h, W, m, 1e-5, False) - ref @ W["o"].T).abs().max() < 1e-10


def test_sink_takes_its_share_and_gate_scales():
    g = torch.Generator().manual_seed(4)
    m = M.latent(2, 8, 4, 6, 12, second=True)[1]
    W = M.widen(M.mixer_weights("latent_attention_2", m, 16, g, torch.float32))
    h = torch.randn(5, 16, generator=g, dtype=torch.float64)
    W["g"] = torch.zeros_like(W["g"])                                          # gate = 1/2 everywhere
    W["sink"] = torch.full((2,), -1e9, dtype=torch.float64)                    # no sink to speak of
    plain = P.latent_attention(h, W, m, 1e-5, False)
    assert (P.latent_attention(h, W, m, 1e-5, True) - 0.5 * plain).abs().max() < 1e-10
    # the first token sees one key: its weight is exp(s) / (exp(s) + exp(sink)); with sink = s it is one half
    c = P.rms_div((h @ W["dkv"].T)[:, :12], 1e-5) * W["dkv.norm"]
    for hd in range(2):
        s0 = ((c[0] @ W["uk"][hd * 8:(hd + 1) * 8].T) @ (h @ W["q"].T)[0, hd * 12:hd * 12 + 8]
              + (h @ W["dkv"].T)[0, 12:] @ (h @ W["q"].T)[0, hd * 12 + 8:(hd + 1) * 12]) * m["scale"]
        W["sink"][hd] = s0
    assert (P.latent_attention(h, W, m, 1e-5, True)[0] - 0.25 * plain[0]).abs().max() < 1e-10


def test_mlstm_against_its_unstabilised_form():
    g = torch.Generator().manual_seed(5)
    m = M.mlstm(2, 6, 5, cap=4.0)[1]
    W = M.widen(M.mixer_weights("mlstm", m, 12, g, torch.float32))
    h = torch.randn(8, 12, generator=g, dtype=torch.float64)
    state = {}
    got = P.mlstm(h, W, m, 1e-6, state)
    # without the running maximum: C_t = sigmoid(f') C + exp(i) k v^T, and S = C exp(-m) with m as the recurrence says
    q = (h @ W["q"].T).view(8, 2, 6) / math.sqrt(6)
    k, v = (h @ W["k"].T).view(8, 2, 6), (h @ W["v"].T).view(8, 2, 5)
    ig = 4 * torch.tanh((h @ W["i"].T + W["i.b"]) / 4)
    fs = torch.sigmoid(4 * torch.tanh((h @ W["f"].T + W["f.b"]) / 4))
    C, n, mx = torch.zeros(2, 6, 5, dtype=torch.float64), torch.zeros(2, 6, dtype=torch.float64), torch.zeros(2, dtype=torch.float64)
    ys = []
    for t in range(8):
        C = fs[t][:, None, None] * C + torch.exp(ig[t])[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = fs[t][:, None] * n + torch.exp(ig[t])[:, None] * k[t]
        mx = torch.maximum(torch.log(fs[t]) + mx, ig[t])
        den = torch.maximum((n * q[t]).sum(-1).abs() * torch.exp(-mx), torch.exp(-mx)) + 1e-6
        ys.append(torch.einsum("hdv,hd->hv", C, q[t]) * torch.exp(-mx)[:, None] / den[:, None])
    ref = (P.rms_div(torch.stack(ys), 1e-6).reshape(8, 10) * W["norm"] * torch.sigmoid(h @ W["g"].T)) @ W["o"].T
    assert (got - ref).abs().max() < 1e-9
    assert (state["S"] - C * torch.exp(-mx)[:, None, None]).abs().max() < 1e-10 and mx.abs().max() <= 4.0


def test_experts_weight_on_the_input():
    g = torch.Generator().manual_seed(6)
    mlp = M.moe(4, 2, 10, shared=6)
    W = M.widen(M.mlp_weights(mlp, 12, g, torch.float32))
    h = torch.randn(5, 12, generator=g, dtype=torch.float64)
    chosen = []
    got = P.moe_ff(h, W, mlp, chosen)
    s = torch.sigmoid(h @ W["router"].T)
    for t in range(5):
        assert sorted(chosen[t]) == sorted(torch.argsort(s[t], descending=True)[:2].tolist())
        # relu^2 is homogeneous of degree two: the weight on the input is its square on the output
        ref = sum(s[t, e] ** 2 * (torch.relu(h[t] @ W[f"e{e}.up"].T) ** 2) @ W[f"e{e}.down"].T for e in chosen[t])
        ref = ref + (torch.relu(h[t] @ W["shared.up"].T) ** 2) @ W["shared.down"].T
        assert (got[t] - ref).abs().max() < 1e-10


def test_layer_reads_one_x_and_the_stream_is_averaged_over_depth():
    cfg = M.TINY_A
    W = M.widen(M.random_weights(cfg, 7))
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    X, after = P.layers(W, cfg, toks)
    assert len(X) == len(cfg["layers"]) + 1 and (X[0] - P.embedding(W, cfg, toks)).abs().max() == 0
    assert (after[1] - (W["l1.dwa"][0] * X[0] + W["l1.dwa"][1] * X[1] + W["l1.dwa"][2] * X[2])).abs().max() < 1e-12
    # layer 2 has no feed-forward: its result is its input plus the mixer alone
    h1 = P.canon(P.norm_scalar(after[1], W["l2.norm1"], 1e-6), W["l2.canon1"])
    mix = P.latent_attention(h1, P.local(W, "l2.mix."), cfg["layers"][2]["mixer"], 1e-6, False)
    assert (X[3] - (after[1] + mix)).abs().max() < 1e-12
    # causal: a later token changes nothing before it
    other = P.forward(W, cfg, toks[:5] + [100, 101, 102])
    assert (other[:5] - P.forward(W, cfg, toks)[:5]).abs().max() < 1e-12
    assert P.forward(W, cfg, toks).abs().max() <= cfg["logit_softcap"]


def test_configuration_and_tensor_table():
    import llm_infer_amd
    from llm_infer_amd.cache.specs import KVSpec, StateSpec
    from llm_infer_amd.config import ConfigError
    from llm_infer_amd.engine.model import DecoderModel
    for name, raw in M.ALL.items():
        cfg = llm_infer_amd.config_from_dict(raw)
        assert cfg.to_dict() == raw
        model = DecoderModel(cfg.model_spec(), torch.float32, "cpu", allocate=False)
        W = M.random_weights(raw, 0)
        assert {k: tuple(v.shape) for k, v in model.params().items()} == {k: tuple(v.shape) for k, v in W.items()}, name
        specs = model.cache_specs()
        # per layer the convolution's inputs, then the mixer's own; at the end the embedding's token before
        assert specs[-1] == StateSpec((), "int32")
        assert specs[0] == StateSpec((max(raw["canon"]["taps"] - 1, 1), raw["width"]), "float32")
        n_kv = sum(isinstance(s, KVSpec) for s in specs)
        assert n_kv == sum(layer["type"] != "mlstm" for layer in raw["layers"])
    cfg = llm_infer_amd.config_from_dict(M.TINY_A)
    kv = [s for s in DecoderModel(cfg.model_spec(), torch.float32, "cpu", allocate=False).cache_specs() if isinstance(s, KVSpec)]
    assert kv[0] == KVSpec(1, 48, None, 40, None, "maps") and kv[1] == KVSpec(1, 48, None, 24, None, "maps")
    bad = dict(M.TINY_A, layers=[M.layer(("sliding", {"heads": 1}), None)])
    with pytest.raises(ConfigError):
        llm_infer_amd.config_from_dict(bad)
    with pytest.raises(ConfigError):
        llm_infer_amd.config_from_dict({k: v for k, v in M.TINY_A.items() if k != "canon"})
    odd = M.config(32, 20, [M.layer(M.latent(1, 8, 8, 8, 8, dims=3), None)])
    with pytest.raises(ConfigError):
        llm_infer_amd.config_from_dict(odd)


def test_random_weights_mode_writes_a_folder_of_the_design(tmp_path):
    import llm_infer_amd
    from llm_infer_amd.weights.safetensors_io import SafetensorsFile
    cfg = llm_infer_amd.config_from_dict(M.TINY_B)
    llm_infer_amd.write_random_model(str(tmp_path), cfg, seed=3)
    f = SafetensorsFile(str(tmp_path / "model.safetensors"))
    assert set(f.names()) == set(M.random_weights(M.TINY_B, 0))
    assert tuple(f.info("l0.norm1")[1]) == () and tuple(f.info("l2.dwa")[1]) == (4,)
    assert abs(float(f.tensor("l2.dwa").float().sum()) - 1.0) < 0.5
