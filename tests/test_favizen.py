"""Favizen without a GPU: the plain implementation pinned by library routines, closed forms and invariants; the
configuration's reading and refusals; the tensor table; what the model asks of the cache (a layer that reads another's
keys keeps its own convolution history); the frequencies stretched by wavelength; the random-weights folder."""
import json
import math

import pytest
import torch
import torch.nn.functional as F

import favizen_models as M
import plain_favizen as P

D = torch.float64


def rnd(*shape, seed=0, s=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D) * s


# ---------------------------------------------------------------------------- the plain implementation, pinned
def test_norm_against_torch():
    x, w = rnd(5, 24), rnd(24, seed=1)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)


def test_masks_at_their_edges():
    w = P.window_mask(20, 5)
    assert w[10, 10] and w[10, 6] and not w[10, 5] and not w[10, 11] and w[0, 0] and w[3, 0]
    c = P.chunk_mask(20, 5)
    assert c[9, 5] and not c[10, 9] and c[10, 10] and not c[9, 10] and c[4, 0] and not c[5, 4]
    assert P.window_mask(6, 1).equal(torch.eye(6, dtype=torch.bool))
    assert P.chunk_mask(6, 1).equal(torch.eye(6, dtype=torch.bool))


def test_rotation_is_a_rotation_of_half_pairs_and_scores_depend_on_distance():
    f = P.rope_frequencies(8, 100.0, None)
    assert torch.allclose(f, torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=D))
    x = rnd(1, 1, 12)
    y = P.rotate(x.expand(7, 1, 12), torch.arange(7), f, 8)
    assert torch.allclose(y[0], x[0])                                   # position 0: nothing turns
    assert torch.allclose(y[..., 8:], x.expand(7, 1, 12)[..., 8:])      # beyond dims: unchanged
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1).expand(7, 1))
    a = f[1] * 3                                                         # pair (1, 5) at position 3
    assert torch.allclose(y[3, 0, 1], x[0, 0, 1] * torch.cos(a) - x[0, 0, 5] * torch.sin(a))
    assert torch.allclose(y[3, 0, 5], x[0, 0, 5] * torch.cos(a) + x[0, 0, 1] * torch.sin(a))
    q, k = rnd(1, 1, 8, seed=3), rnd(1, 1, 8, seed=4)
    s = lambda i, j: (P.rotate(q, torch.tensor([i]), f, 8) * P.rotate(k, torch.tensor([j]), f, 8)).sum()
    assert torch.allclose(s(9, 4), s(25, 20))


def test_frequencies_stretched_by_wavelength():
    sc = {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 64}
    f0, f = P.rope_frequencies(32, 10000.0, None), P.rope_frequencies(32, 10000.0, sc)
    wl = 2 * math.pi / f0
    short, long_ = wl < 64 / 3.0, wl > 64 / 1.0
    assert short.any() and long_.any() and (~short & ~long_).any()
    assert torch.equal(f[short], f0[short]) and torch.allclose(f[long_], f0[long_] / 5.0)
    mid = ~short & ~long_
    assert ((f[mid] < f0[mid]) & (f[mid] > f0[mid] / 5.0)).all()
    # the library's own table
    from llm_infer_amd.parts.position import scaled_by_wavelength
    assert torch.allclose(scaled_by_wavelength(10000.0, 32, sc).double(), f, rtol=1e-6)


def test_convolution_against_conv1d():
    u, w = rnd(11, 6), rnd(6, 4, seed=2)
    ref = F.conv1d(F.pad(u.T[None], (3, 0)), w[:, None, :], groups=6)[0].T
    assert torch.allclose(P.causal_conv(u, w), ref, atol=1e-12)
    assert torch.allclose(P.causal_conv(u, w)[0], u[0] * w[:, 3])       # the last tap is the current token's


def test_attention_against_scaled_dot_product_with_a_sink_that_weighs_nothing():
    T, H, G, d, dv = 13, 4, 2, 8, 5
    q, k, v = rnd(T, H, d), rnd(T, G, d, seed=1), rnd(T, G, dv, seed=2)
    vis = P.window_mask(T, 6)
    got = P.sink_attention(q, k, v, 0.3, vis, torch.full((H,), -1e9, dtype=D))
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), attn_mask=vis, scale=0.3)
    assert torch.allclose(got, ref.transpose(0, 1), atol=1e-10)


def test_a_sink_equal_to_the_only_score_halves_the_output_and_is_neither_scaled_nor_biased():
    q, k, v = torch.ones(1, 1, 4, dtype=D), torch.ones(1, 1, 4, dtype=D), rnd(1, 1, 3)
    out = P.sink_attention(q, k, v, 0.5, torch.ones(1, 1, dtype=torch.bool), torch.tensor([2.0], dtype=D), torch.tensor([0.7], dtype=D))
    assert torch.allclose(out, 0.5 * v)                                  # score 4 * 0.5 = 2 = sink, distance 0


def test_distance_bias_and_slopes():
    s = P.slopes(4, D)
    assert torch.allclose(s, torch.tensor([2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8], dtype=D))
    T = 6
    q, k, v = torch.zeros(T, 1, 2, dtype=D), torch.zeros(T, 1, 2, dtype=D), torch.eye(T, dtype=D)[:, None, :]
    out = P.sink_attention(q, k, v, 1.0, P.chunk_mask(T, T), torch.tensor([-1e9], dtype=D), torch.tensor([0.5], dtype=D))
    w = torch.exp(-0.5 * torch.arange(5, -1, -1, dtype=D))              # the last row: distances 5 .. 0
    assert torch.allclose(out[5, 0], w / w.sum())


def test_gate_is_one_number_a_head():
    o, h, wg = rnd(3, 2, 4), rnd(3, 5, seed=1), torch.zeros(2, 5, dtype=D)
    assert torch.allclose(P.gate_heads(o, h, wg), 0.5 * o)


def test_clamped_activation():
    g, u = torch.tensor([-3.0, 0.5, 9.0], dtype=D), torch.tensor([-9.0, 0.25, 9.0], dtype=D)
    y = P.clamped_glu(g, u, 2.0)
    sw = lambda z: z * torch.sigmoid(1.702 * z)
    assert torch.allclose(y, torch.stack([sw(g[0]) * (-2.0 + 1.0), sw(g[1]) * 1.25, sw(torch.tensor(2.0, dtype=D)) * 3.0]))


def test_experts_by_table_and_the_shared_experts_gate():
    w, V = 12, 9
    mlp = M.moe(4, 2, 6, limit=1.5, shared=5, shared_limit=0.5)
    W = M.widen(M.mlp_weights(mlp, w, V, torch.Generator().manual_seed(5), torch.float32))
    h, toks = rnd(3, w), torch.tensor([2, 7, 2])
    out = P.table_experts(h, toks, W, mlp)
    e0, e1 = W["table"][2].tolist()
    assert e0 != e1
    one = lambda t, e: P.gated_ff(h[t:t + 1], W, f"e{e}.", 1.5, False)[0]
    shared = P.gated_ff(h[:1], W, "shared.", 0.5, False)[0] * torch.sigmoid(h[0] @ W["shared.sg"][0])
    assert torch.allclose(out[0], 0.5 * (one(0, e0) + one(0, e1)) + shared)


def test_a_layer_that_reads_anothers_keys_and_causality():
    cfg = M.TINY_A
    W = M.widen(M.random_weights(cfg, 3))
    toks = torch.randint(0, cfg["vocab"], (70,), generator=torch.Generator().manual_seed(1)).tolist()
    full = P.forward(cfg, W, toks)
    assert torch.allclose(P.forward(cfg, W, toks[:40]), full[:40], atol=1e-9)
    # layer 3 by hand: its own queries, mask and feed-forward on the keys and values that layer 1 made of ITS input
    layers, eps = [], cfg["norm"]["eps"]
    P.forward(cfg, W, toks, layers)
    L1, L3 = P.sub(W, "l1."), P.sub(W, "l3.")
    kv = P.attention2_keys_values(P.rms_norm(layers[0], L1["norm1"], eps), P.sub(L1, "mix."), cfg["layers"][1]["mixer"])
    x = layers[2]
    y = P.attention2_mixer(P.rms_norm(x, L3["norm1"], eps), P.sub(L3, "mix."), cfg["layers"][3]["mixer"], kv)
    x = x + P.rms_norm(y, L3["norm1b"], eps)
    y = P.table_experts(P.rms_norm(x, L3["norm2"], eps), torch.tensor(toks), P.sub(L3, "mlp."), cfg["layers"][3]["mlp"])
    assert torch.allclose(x + P.rms_norm(y, L3["norm2b"], eps), layers[3], atol=1e-9)
    assert "l3.mix.k" not in W and "l3.mix.v.conv" not in W and "l3.mix.q.conv" in W


# ---------------------------------------------------------------------------- configuration, tensors, cache
def test_configuration_reading_and_refusals():
    from llm_infer_amd import ConfigError, config_from_dict
    cfg = config_from_dict(M.TINY_A)
    assert cfg.to_dict()["layers"] == M.TINY_A["layers"] and cfg.logit_scale == 0.25
    assert config_from_dict(cfg.to_dict()) == cfg
    bad = json.loads(json.dumps(M.TINY_A))
    bad["layers"][3]["mixer"]["kv_from"] = 0                               # another kind of layer
    with pytest.raises(ConfigError):
        config_from_dict(bad)
    bad = json.loads(json.dumps(M.TINY_A))
    bad["layers"][0]["mixer"]["vdim"] = 8                                  # values that are the keys have their size
    with pytest.raises(ConfigError):
        config_from_dict(bad)
    bad = json.loads(json.dumps(M.TINY_A))
    bad["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ConfigError):
        config_from_dict(bad)
    bad = json.loads(json.dumps(M.TINY_A))
    bad["layers"][0]["type"] = "attention_3"
    with pytest.raises(ConfigError):
        config_from_dict(bad)


@pytest.mark.parametrize("name", sorted(M.ALL))
def test_tensor_table_is_the_designs(name):
    from llm_infer_amd import config_from_dict
    from llm_infer_amd.engine.model import DecoderModel
    cfg = M.ALL[name]
    model = DecoderModel(config_from_dict(cfg).model_spec(), torch.float32, "cpu", allocate=False)
    W = M.random_weights(cfg, 1)
    assert {k: tuple(v.shape) for k, v in model.params().items()} == {k: tuple(v.shape) for k, v in W.items()}


def test_what_the_model_asks_of_the_cache():
    from llm_infer_amd import config_from_dict
    from llm_infer_amd.cache.specs import KVSpec, StateSpec
    from llm_infer_amd.engine.model import DecoderModel
    model = DecoderModel(config_from_dict(M.TINY_A).model_spec(), torch.float32, "cpu", allocate=False)
    specs = model.cache_specs()
    assert specs[0] == KVSpec(1, 32, 9, 20, None, "maps")                   # a window; keys padded to 32
    assert specs[1] == StateSpec((1, 4 * 16 + 2 * 16 + 2 * 24), "float32")  # two taps: one row of q | k | v
    assert specs[2] == KVSpec(2, 16, None, 24, 50, "maps")                  # chunks of 50; its reader looks the same way
    assert specs[4] == StateSpec((1, 4 * 16), "float32") and specs[5] is None   # the reader: its own history, no keys
    assert model._seen[3, 0] == [4, 2]
    # a reader with another mask: the owner keeps everything
    model = DecoderModel(config_from_dict(M.TINY_B).model_spec(), torch.float32, "cpu", allocate=False)
    assert model.cache_specs()[1] == KVSpec(1, 16, None, 40, None, "maps")


def test_random_weights_folder(tmp_path):
    import llm_infer_amd
    from safetensors import safe_open
    cfg = llm_infer_amd.config_from_dict(M.TINY_B)
    llm_infer_amd.write_random_model(str(tmp_path), cfg, seed=4)
    assert llm_infer_amd.config_from_folder(str(tmp_path)).to_dict()["layers"] == M.TINY_B["layers"]
    with safe_open(str(tmp_path / "model.safetensors"), "pt") as f:
        table = f.get_tensor("l2.mlp.table")
        assert table.dtype == torch.int32 and table.shape == (97, 3) and int(table.max()) < 9 and int(table.min()) >= 0
        assert all(len(set(row)) == 3 for row in table.tolist())
        W = {k: f.get_tensor(k) for k in f.keys()}
    out = P.forward(M.TINY_B, M.widen(W), [1, 2, 3, 4, 5, 6, 7, 8, 9])
    assert torch.isfinite(out).all()
