"""Dupolorn on the GPU against the plain implementation: every mechanism alone, whole prompts, prompts cut into
portions, decoding token by token, batches of unequal requests against each alone, slots and pages used again, keys
far away and at page borders, the first tokens, long decoding, other sizes, and greedy generation through the
library's entry point.

Routing: a float32 run follows the plain implementation's choices to rounding.  A bfloat16 run rounds the router's
input, so a token whose scores nearly tie could go either way, and what it then leaves in caches and states reaches
every later token; the whole-model runs in bfloat16 therefore use the same configurations with every expert chosen
(the weights still follow the token), and the choice itself is tested in float32 and, alone, on the same rounded
input in both types."""
import json
import os
import subprocess
import sys

import pytest
import torch

import dupolorn_models as M
import plain_dupolorn as P
import trace_util as TU

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {"float32": 1e-4, "bfloat16": 3e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def lib():
    import llm_infer_amd
    return llm_infer_amd


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in M.ALL.items():
        W = M.random_weights(cfg, 40 + ord(name), sharp=2.0)
        folder = str(tmp_path_factory.mktemp(f"dupolorn_{name}"))
        M.write_model(folder, cfg, W)
        out[name, "float32"] = (folder, cfg, M.widen(W))
        every = json.loads(json.dumps(cfg))
        for layer in every["layers"]:
            if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
                layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
        folder = str(tmp_path_factory.mktemp(f"dupolorn_{name}_every"))
        M.write_model(folder, every, W)
        out[name, "bfloat16"] = (folder, every, M.widen(W))
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def step_context(slots, lens_before, toks):
    from llm_infer_amd.engine.step import StepContext
    return StepContext(DEV, list(slots), [list(t) for t in toks], list(lens_before), [[] for _ in toks])


def error(got, ref):
    """Largest difference relative to the reference's spread."""
    return ((got.double() - ref.double()).abs().max() / ref.double().std()).item()


def build_mixer(spec, weights, dtype, position=None):
    """A mixer as the configuration describes it (``spec`` of the inner mixer), with the given tensors bound."""
    import llm_infer_amd.parts  # noqa: F401  (registers the parts)
    from llm_infer_amd.registry import lookup
    from llm_infer_amd.weights.loader import place_tensor
    pos = None
    if position is not None:
        pos = lookup("position", position.kind)(**position.params, prefix="", dtype=DT[dtype], device=DEV)
    part = lookup("mixer", spec.kind)(**spec.params, position=pos, prefix="", dtype=DT[dtype], device=DEV)
    wanted = part.params()
    assert set(wanted) == set(weights), set(wanted) ^ set(weights)
    part.bind({n: place_tensor(weights[n], wanted[n].kind, DT[dtype], DEV) for n in wanted})
    return part


def one_layer(mixer, mlp=None, width=96, eps=1e-5, taps=3):
    from llm_infer_amd.registry import config_from_dict
    return config_from_dict(M.config(width, 50, [M.layer(mixer, mlp)], eps=eps, taps=taps))


def inner_spec(cfg):
    return cfg._mixer("", cfg.layers[0]).params["inner"].with_prefix("")


def run_mixer(part, h_of, schedule, dtype, f32_in=False, cache=None):
    """Runs a mixer over ``schedule``: a list of steps, each {request: tokens it brings}.  ``h_of[r]`` float32
    [n, width] is request r's input.  Returns {r: what the mixer added, [n, width]} and the cache."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.parts.base import cache_specs_of
    specs = cache_specs_of(part)
    if cache is None:
        cache = Cache(specs, 8192, 8192, DT[dtype], DEV)
    views = [cache.view(i) for i in range(len(specs))]
    views = views if hasattr(part, "cache_specs") else views[0]
    slot, at, out = {}, {r: 0 for r in h_of}, {r: [] for r in h_of}
    for step in schedule:
        for r in step:
            if r not in slot:
                slot[r] = cache.alloc_slot()
        rs = list(step)
        cache.grow([slot[r] for r in rs], [at[r] + step[r] for r in rs], filled=True)
        ctx = step_context([slot[r] for r in rs], [at[r] for r in rs], [[0] * step[r] for r in rs])
        h = torch.cat([h_of[r][at[r]:at[r] + step[r]] for r in rs]).to(DEV).to(torch.float32 if f32_in else DT[dtype])
        res = torch.zeros((h.shape[0], h_of[rs[0]].shape[1]), dtype=torch.float32, device=DEV)
        part.forward(h, ctx, views, res)
        for r, rows in zip(rs, res.cpu().split([step[r] for r in rs])):
            out[r].append(rows)
            at[r] += step[r]
        for r in rs:
            if at[r] == h_of[r].shape[0]:
                cache.free_slot(slot.pop(r))
    return {r: torch.cat(v) for r, v in out.items()}, cache


SCHEDULES = {
    "whole": lambda n: [{"a": n["a"]}, {"b": n["b"]}, {"c": n["c"]}],
    # portions down to two tokens and one, across the edges of pages
    "portions": lambda n: [{"a": 61}, {"a": 2}, {"a": 1}, {"a": 3}, {"a": n["a"] - 67}] + [{"b": 2}] * (n["b"] // 2)
                          + [{"b": n["b"] % 2}] * (n["b"] % 2) + [{"c": n["c"]}],
    # unequal requests together, then decoded together; the shortest ends first, and c comes into a slot used before
    "together": lambda n: [{"a": n["a"] - 9, "b": n["b"] - 4}] + [{"a": 1, "b": 1}] * 4 + [{"a": 1}] * 5 + [{"c": n["c"] - 3}]
                          + [{"c": 1}] * 3,
}


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_bigram_embedding_keeps_the_token_before(lib, dtype):
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.parts.embedding import BigramEmbedding
    g = torch.Generator().manual_seed(0)
    V, w, buckets = 60, 40, 13
    table, bigram = torch.randn(V, w, generator=g).to(DT[dtype]), torch.randn(buckets + 1, w, generator=g).to(DT[dtype])
    emb = BigramEmbedding(vocab_size=V, hidden_size=w, buckets=buckets, mul_prev=1000003, mul_cur=77, scale=1.5, prefix="",
                          dtype=DT[dtype], device=DEV)
    emb.bind({"weight": table.to(DEV), "bigram": bigram.to(DEV)})
    cache = Cache(emb.cache_specs(), 1024, 1024, DT[dtype], DEV)
    seqs = {"a": tokens({"vocab": V}, 11, 1), "b": tokens({"vocab": V}, 5, 2)}
    ref = {r: table[torch.tensor(t)].double() * 1.5 + bigram[torch.tensor(P.bigram_rows(t, buckets, 1000003, 77))].double()
           for r, t in seqs.items()}
    slot = {r: cache.alloc_slot() for r in seqs}
    got, at = {r: [] for r in seqs}, {r: 0 for r in seqs}
    # a portion, both together (b begins in the middle of the step), one token each, the rest
    for step in ([("a", 4)], [("a", 2), ("b", 3)], [("a", 1), ("b", 1)], [("b", 1), ("a", 4)]):
        ctx = step_context([slot[r] for r, _ in step], [at[r] for r, _ in step], [seqs[r][at[r]:at[r] + n] for r, n in step])
        x = emb.forward(ctx, [cache.view(0)]).cpu()
        for (r, n), rows in zip(step, x.split([n for _, n in step])):
            got[r].append(rows)
            at[r] += n
    for r in seqs:
        assert (torch.cat(got[r]).double() - ref[r]).abs().max() < 1e-5, r
    # a slot that is used again begins with the first token's row, whatever the sequence before left
    cache.free_slot(slot["a"])
    s = cache.alloc_slot()
    x = emb.forward(step_context([s], [0], [seqs["b"][:2]]), [cache.view(0)]).cpu()
    assert (x.double() - ref["b"][:2]).abs().max() < 1e-5


def test_scalar_norm_softcap_and_depth_average(lib):
    from llm_infer_amd.kernels import ops
    from llm_infer_amd.parts.norm import RMSNorm
    g = torch.Generator().manual_seed(1)
    x = torch.randn(7, 200, generator=g) * 3
    norm = RMSNorm(size=200, eps=1e-3, name="n", scalar=True, prefix="", dtype=torch.float32, device=DEV)
    norm.bind({"n": torch.tensor(1.7).to(DEV)})
    assert (norm.forward(x.to(DEV)).cpu().double() - P.norm_scalar(x.double(), 1.7, 1e-3)).abs().max() < 1e-5
    z = (torch.randn(5, 77, generator=g) * 40).to(DEV)
    ref = 30 * torch.tanh(z.cpu().double() / 30)
    assert (ops.softcap(z, 30.0).cpu().double() - ref).abs().max() < 1e-4
    for width in (64, 75):
        hist = torch.randn(6, 9, width, generator=g)
        w = torch.randn(5, generator=g)
        dev = hist.to(DEV)
        got = ops.depth_average(dev, 5, w.to(DEV), dev[5]).cpu()
        assert (got.double() - torch.einsum("j,jtc->tc", w.double(), hist[:5].double())).abs().max() < 1e-5
        assert (dev[:5].cpu() - hist[:5]).abs().max() == 0


@pytest.mark.parametrize("taps", [1, 2, 3, 6])
def test_convolution_ahead_of_a_mixer(lib, taps):
    """The convolution alone: whole, in portions shorter than its reach, and one token at a time."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.specs import StateSpec
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(70, taps, generator=g)
    h_of = {"a": torch.randn(40, 70, generator=g), "b": torch.randn(7, 70, generator=g)}
    cache = Cache([StateSpec((max(taps - 1, 1), 70), "float32")], 1024, 1024, torch.float32, DEV)
    for schedule in ([{"a": 40}, {"b": 7}], [{"a": 1}, {"a": 2, "b": 1}, {"a": 1, "b": 1}, {"b": 5, "a": 30}, {"a": 6}],
                     [{"a": 1, "b": 1}] * 7 + [{"a": 1}] * 33):
        slot, at, out = {}, {r: 0 for r in h_of}, {r: [] for r in h_of}
        for step in schedule:
            for r in step:
                if r not in slot:
                    slot[r] = cache.alloc_slot()
            rs = list(step)
            ctx = step_context([slot[r] for r in rs], [at[r] for r in rs], [[0] * step[r] for r in rs])
            rows = torch.cat([h_of[r][at[r]:at[r] + step[r]] for r in rs]).to(DEV)
            got = ops.conv_add(rows, w.to(DEV), cache.view(0).state, ctx, torch.float32).cpu()
            for r, part in zip(rs, got.split([step[r] for r in rs])):
                out[r].append(part)
                at[r] += step[r]
        for r in h_of:
            assert (torch.cat(out[r]).double() - P.canon(h_of[r].double(), w.double())).abs().max() < 1e-5, (r, len(schedule))
            cache.free_slot(slot[r])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_product_per_head_and_gate(lib, dtype):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    for T, H, n_in, n_out in ((1, 3, 20, 40), (37, 2, 130, 7), (16, 5, 64, 64), (70, 3, 192, 200)):
        w = (torch.randn(H, n_out, n_in, generator=g) * n_in ** -0.5).to(DT[dtype])
        c0, hs = (16, n_in + 8) if n_in % 8 == 0 else (11, n_in + 5)         # heads at multiples of 16 bytes, and not
        x = torch.randn(T, c0 + H * hs, generator=g)
        gate = torch.randn(T, 9 + H * n_out, generator=g)
        out = torch.zeros(T, H, n_out + 3, dtype=DT[dtype], device=DEV)
        ops.head_linear(x.to(DEV), c0, hs, w.to(DEV), out, 3, n_out + 3, gate=gate.to(DEV), gate_col=9)
        xin = torch.stack([x[:, c0 + h * hs:c0 + h * hs + n_in] for h in range(H)], 1).double()
        ref = torch.einsum("thi,hji->thj", xin, w.double()) * torch.sigmoid(gate[:, 9:].double().view(T, H, n_out))
        assert error(out[:, :, 3:].cpu(), ref) < (1e-5 if dtype == "float32" else 3e-2)      # the output is rounded to 16 bits
        assert out[:, :, :3].abs().max() == 0                                 # nothing beside a head's own columns


def test_router_scores_and_expert_activation(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    T, E, top, w = 9, 6, 3, 40
    logits = torch.randn(T, E, generator=g) * 2
    h = torch.randn(T, w, generator=g)
    res = torch.zeros(T, w, device=DEV)
    weights = ops.moe_route(logits.to(DEV), None, h.to(DEV), res, E, E, top, 2, 1.0, sigmoid_scores=True, renorm=False).cpu()
    s = torch.sigmoid(logits.double())
    for t in range(T):
        picked = torch.topk(s[t], top).indices.tolist()
        for e in range(E):
            assert abs(weights[t, e].item() - (s[t, e].item() if e in picked else 0.0)) < 1e-6
    assert (weights[:, E] == 1).all() and res.abs().max() == 0
    z = torch.randn(T, E * 5 + 4, generator=g) * 2
    got = ops.expert_act(z.to(DEV), weights.to(DEV), E, 5, 4, "relu2", True, torch.float32).cpu().double()
    wide = torch.cat([weights[:, :E].double().repeat_interleave(5, 1), weights[:, E:].double().expand(T, 4)], 1)
    assert (got - P.relu2(wide * z.double())).abs().max() < 1e-5
    got = ops.expert_act(z.to(DEV), weights.to(DEV), E, 5, 4, "silu", False, torch.float32).cpu().double()
    assert (got - wide * torch.nn.functional.silu(z.double())).abs().max() < 1e-5
    idx = torch.tensor([4, 0, 7], dtype=torch.int32)
    got = ops.expert_act(z[:3, :5].contiguous().to(DEV), weights.to(DEV), 1, 5, 0, "relu2", True, torch.float32, idx.to(DEV), 2).cpu()
    assert (got.double() - P.relu2(weights[idx.long(), 2:3].double() * z[:3, :5].double())).abs().max() < 1e-5


LATENT_SIZES = [(3, 20, 6, 36, 40, True, 4), (2, 8, 16, 16, 24, False, 16), (1, 16, 0, 8, 72, True, 0), (4, 0, 32, 24, 16, False, 32),
                (8, 64, 64, 64, 192, True, 64), (2, 32, 16, 48, 320, False, 16)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, d, rd, dv, r, second, dims", LATENT_SIZES)
@pytest.mark.parametrize("schedule", list(SCHEDULES))
def test_latent_attention_part(lib, dtype, H, d, rd, dv, r, second, dims, schedule):
    width, eps = 96, 1e-5
    mixer = M.latent(H, d, rd, dv, r, second=second, base=300.0, dims=dims)
    cfg = one_layer(mixer, width=width, eps=eps)
    g = torch.Generator().manual_seed(H * 100 + r)
    W = M.mixer_weights(mixer[0], mixer[1], width, g, torch.bfloat16, sharp=2.0)
    part = build_mixer(inner_spec(cfg), W, dtype, cfg._position(cfg.layers[0]))
    n = {"a": 140, "b": 9, "c": 70}
    h_of = {k: torch.randn(v, width, generator=g).to(DT[dtype]).float() for k, v in n.items()}
    got, cache = run_mixer(part, h_of, SCHEDULES[schedule](n), dtype)
    for k in n:
        ref = P.latent_attention(h_of[k].double(), M.widen(W), mixer[1], eps, second)
        tol = TOL[dtype]
        if dtype == "bfloat16":      # not below three times what the rounding of the latent and the queries alone does
            tol = max(tol, 3 * error(P.latent_attention(h_of[k].double(), M.widen(W), mixer[1], eps, second, store=torch.bfloat16), ref))
        assert error(got[k], ref) < tol, k
    assert all(g_.pool.n_free == g_.n_pages - 1 for g_ in cache.groups if hasattr(g_, "pool"))        # every page came back


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_attention_finds_a_far_key_and_feels_its_sink(lib, dtype):
    """Keys made to stand out.  The latent of one early token is what the queries of all later tokens look for (through
    the up-projection of the keys), so every later output is that token's value, however far back it lies: in a
    prompt across pages, in a portion, and in decoded tokens.  Then a large sink takes nearly all the weight."""
    width, H, d, rd, dv, r = 64, 2, 16, 8, 16, 32
    mixer = M.latent(H, d, rd, dv, r, second=True, scale=1.0)
    cfg = one_layer(mixer, width=width)
    g = torch.Generator().manual_seed(9)
    W = M.mixer_weights(mixer[0], mixer[1], width, g, torch.float32)
    W["q"][:, :] = 0
    W["dkv"][r:] = 0                                   # no rotated part: positions do not matter
    W["g"][:, :] = 0
    W["sink"] = torch.tensor([-30.0, -30.0])
    # input channel 0 marks the far token: its latent gets a large component along e_0 ... which the norm would
    # flatten, so the mark goes through the norm's weight: latent coordinate 0 is large only for the marked token
    W["dkv"][:r] = 0
    W["dkv"][0, 0] = 1.0                               # c_raw[0] = h[0]; the others come from channels 1..
    for i in range(1, r):
        W["dkv"][i, i] = 1.0
    W["dkv.norm"] = torch.ones(r)
    W["uk"][:, :] = 0
    W["uk"][0, 0] = 1.0                                # head 0's key dimension 0 reads latent coordinate 0
    W["uk"][d, 0] = 1.0                                # head 1's likewise
    W["q"][0, 1] = 60.0                                # every query looks along key dimension 0, as strongly as h[1] says
    W["q"][d + rd, 1] = 60.0
    n, far = 200, 3
    h = 0.1 * torch.randn(n, width, generator=g)
    h[:, 0] = 0.0
    h[far, 0] = 3.0                                    # the marked token
    h[:, 1] = 1.0
    h = h.to(DT[dtype]).float()
    ref = P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, True)
    alone = P.latent_attention(h[far:far + 1].double(), M.widen(W), mixer[1], 1e-5, True, positions=[far])
    assert error(ref[far + 1:], alone.expand(n - far - 1, -1)) < 1e-3          # the far key decides
    part = build_mixer(inner_spec(cfg), W, dtype, cfg._position(cfg.layers[0]))
    for schedule in ([{"a": n}], [{"a": 130}, {"a": 2}, {"a": 68}], [{"a": 150}] + [{"a": 1}] * 50):
        got, _ = run_mixer(part, {"a": h}, schedule, dtype)
        assert error(got["a"], ref) < TOL[dtype], len(schedule)
    W["sink"] = torch.tensor([40.0, -30.0])            # head 0's sink outweighs even the marked key
    part = build_mixer(inner_spec(cfg), W, dtype, cfg._position(cfg.layers[0]))
    ref2 = P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, True)
    assert error(ref2, ref) > 0.1
    got, _ = run_mixer(part, {"a": h}, [{"a": 150}] + [{"a": 1}] * 50, dtype)
    assert error(got["a"], ref2) < TOL[dtype]


@pytest.mark.parametrize("H, na, nb", [(8, 660, 200), (40, 330, 90)])
def test_decoding_far_into_a_context_with_many_heads(lib, H, na, nb):
    """Many heads on the one latent and a context of several pages: a 16-bit decode step then takes the heads as the
    columns of a tile (forty heads: two tiles) and lets several workgroups share a token's keys; two requests of unequal
    length together."""
    width = 64
    mixer = M.latent(H, 16, 16, 24, 48, second=True, base=1000.0)
    cfg = one_layer(mixer, width=width)
    g = torch.Generator().manual_seed(17)
    W = M.mixer_weights(mixer[0], mixer[1], width, g, torch.bfloat16, sharp=2.0)
    part = build_mixer(inner_spec(cfg), W, "bfloat16", cfg._position(cfg.layers[0]))
    h_of = {"a": torch.randn(na, width, generator=g).bfloat16().float(), "b": torch.randn(nb, width, generator=g).bfloat16().float()}
    got, _ = run_mixer(part, h_of, [{"a": na - 40, "b": nb - 40}] + [{"a": 1, "b": 1}] * 40, "bfloat16")
    for r, h in h_of.items():
        ref = P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, True)
        tol = max(TOL["bfloat16"], 3 * error(P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, True, store=torch.bfloat16), ref))
        assert error(got[r], ref) < tol and error(got[r][-40:], ref[-40:]) < tol, r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_tells_positions_apart_across_steps(lib, dtype):
    """With only rotated dimensions a score depends on the distance alone; a cut prompt must give the same as a whole."""
    width = 64
    mixer = M.latent(2, 0, 32, 16, 16, base=40.0)
    cfg = one_layer(mixer, width=width)
    g = torch.Generator().manual_seed(11)
    W = M.mixer_weights(mixer[0], mixer[1], width, g, torch.bfloat16, sharp=3.0)
    part = build_mixer(inner_spec(cfg), W, dtype, cfg._position(cfg.layers[0]))
    h = torch.randn(150, width, generator=g).to(DT[dtype]).float()
    ref = P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, False)
    wrong = P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, False, positions=[0] * 150)
    assert error(wrong, ref) > 0.1
    for schedule in ([{"a": 150}], [{"a": 63}, {"a": 1}, {"a": 1}, {"a": 85}], [{"a": 100}] + [{"a": 1}] * 50):
        got, _ = run_mixer(part, {"a": h}, schedule, dtype)
        tol = max(TOL[dtype], 3 * error(P.latent_attention(h.double(), M.widen(W), mixer[1], 1e-5, False, store=torch.bfloat16), ref)
                  if dtype == "bfloat16" else 0)
        assert error(got["a"], ref) < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, d, dv, cap", [(3, 20, 24, 9.0), (1, 33, 70, 15.0), (4, 16, 16, 30.0), (2, 128, 128, 11.0), (2, 64, 130, 2.0), (1, 200, 40, 10.0)])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
def test_matrix_memory_part(lib, dtype, H, d, dv, cap, schedule):
    width, eps = 96, 1e-5
    mixer = M.mlstm(H, d, dv, cap)
    cfg = one_layer(mixer, width=width, eps=eps)
    g = torch.Generator().manual_seed(H * 10 + d)
    W = M.mixer_weights("mlstm", mixer[1], width, g, torch.bfloat16, sharp=2.0)
    part = build_mixer(inner_spec(cfg), W, dtype)
    n = {"a": 140, "b": 9, "c": 70}
    h_of = {k: torch.randn(v, width, generator=g).to(DT[dtype]).float() for k, v in n.items()}
    got, _ = run_mixer(part, h_of, SCHEDULES[schedule](n), dtype)
    for k in n:
        assert error(got[k], P.mlstm(h_of[k].double(), M.widen(W), mixer[1], eps)) < TOL[dtype], k


def test_matrix_memory_carries_a_first_token_far(lib):
    """A forget gate near one and an input gate that opens for the first token only: 600 tokens later the output is
    still that token's value, through prompts, portions and decoded tokens; the state starts at zero in a slot used again."""
    width, H, d, dv = 32, 1, 8, 8
    mixer = M.mlstm(H, d, dv, cap=20.0)
    cfg = one_layer(mixer, width=width)
    g = torch.Generator().manual_seed(13)
    W = M.mixer_weights("mlstm", mixer[1], width, g, torch.float32)
    W["f"][:] = 0
    W["f.b"] = torch.tensor([18.0])                     # forget gate: sigmoid(18), nothing is forgotten
    W["i"][:] = 0
    W["i"][0, 0] = 1.0
    W["i.b"] = torch.tensor([-15.0])                    # the input gate opens where channel 0 says so
    n = 600
    h = 0.3 * torch.randn(n, width, generator=g)
    h[:, 0] = 0.0
    h[0, 0] = 30.0
    ref = P.mlstm(h.double(), M.widen(W), mixer[1], 1e-5)
    only = P.mlstm(h[:1].double(), M.widen(W), mixer[1], 1e-5)
    state = {}
    P.mlstm(h.double(), M.widen(W), mixer[1], 1e-5, state)
    k0, v0 = (h[0].double() @ M.widen(W)["k"].T), (h[0].double() @ M.widen(W)["v"].T)
    assert error(state["S"][0], torch.outer(k0, v0) * state["S"][0].norm() / torch.outer(k0, v0).norm()) < 1e-3
    part = build_mixer(inner_spec(cfg), W, "float32")
    cache = None
    for schedule in ([{"a": n}], [{"a": 2}, {"a": 300}, {"a": 298}], [{"a": 500}] + [{"a": 1}] * 100):
        got, cache = run_mixer(part, {"a": h}, schedule, "float32", cache=cache)
        assert error(got["a"], ref) < 3e-4, len(schedule)            # 600 steps of float32 rounding
    assert only.abs().max() > 0


# ---------------------------------------------------------------------------
# the whole model
# ---------------------------------------------------------------------------
def compare(got, ref, dtype):
    assert M.row_error(got, ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.ALL))
def test_model_whole_portions_and_token_by_token(lib, models, dtype, name):
    folder, cfg, W = models[name, dtype]
    eng = lib.load(folder, dtype=dtype, max_tokens=4096)
    toks = tokens(cfg, 150, 3)
    ref = P.forward(W, cfg, toks)
    s = eng.alloc_slot()
    whole = eng.step([s], [toks], [list(range(len(toks)))]).cpu()
    compare(whole, ref, dtype)
    # the first tokens by themselves: one token, two
    for n in (1, 2):
        s2 = eng.alloc_slot()
        compare(eng.step([s2], [toks[:n]], [list(range(n))]).cpu(), ref[:n], dtype)
        eng.free_slot(s2)
    eng.free_slot(s)
    # portions of several sizes, down to two tokens and one, across a page's edge; in a slot used before
    s = eng.alloc_slot()
    parts, at = [], 0
    for n in (61, 2, 1, 3, 40, 2, 41):
        parts.append(eng.step([s], [toks[at:at + n]], [list(range(n))]).cpu())
        at += n
    cut = torch.cat(parts)
    compare(cut, ref, dtype)
    eng.free_slot(s)
    # token by token
    s = eng.alloc_slot()
    single = torch.cat([eng.step([s], [[t]], [[0]]).cpu() for t in toks[:80]])
    compare(single, ref[:80], dtype)
    eng.free_slot(s)
    if dtype == "float32":
        # however the prompt is cut, the same numbers to rounding
        assert M.row_error(cut, whole) < 2e-5 and M.row_error(single, whole[:80]) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(M.ALL))
def test_unequal_requests_together_against_each_alone(lib, models, dtype, name):
    folder, cfg, W = models[name, dtype]
    eng = lib.load(folder, dtype=dtype, max_tokens=4096)
    reqs = {"a": tokens(cfg, 90, 5), "b": tokens(cfg, 1, 6), "c": tokens(cfg, 130, 7), "d": tokens(cfg, 17, 8)}
    decoded = {"a": 12, "b": 0, "c": 40, "d": 16}
    alone = {}
    for r, t in reqs.items():
        s = eng.alloc_slot()
        alone[r] = eng.step([s], [t], [list(range(len(t)))]).cpu()
        eng.free_slot(s)
        compare(alone[r], P.forward(W, cfg, t), dtype)
    # the slots and pages of the runs above are used again
    slot = {r: eng.alloc_slot() for r in reqs}
    head = {r: len(t) - decoded[r] for r, t in reqs.items()}
    got = {r: [] for r in reqs}
    live = list(reqs)
    first = eng.step([slot[r] for r in live], [reqs[r][:head[r]] for r in live], [list(range(head[r])) for r in live]).cpu()
    for r, rows in zip(live, first.split([head[r] for r in live])):
        got[r].append(rows)
    at = dict(head)
    while True:
        for r in [r for r in live if at[r] == len(reqs[r])]:
            eng.free_slot(slot[r])
        live = [r for r in live if at[r] < len(reqs[r])]
        if not live:
            break
        out = eng.step([slot[r] for r in live], [[reqs[r][at[r]]] for r in live]).cpu()
        for r, row in zip(live, out):
            got[r].append(row[None])
            at[r] += 1
    for r in reqs:
        assert M.row_error(torch.cat(got[r]), alone[r]) < (2e-5 if dtype == "float32" else TOL[dtype]), r


def test_long_decoding_and_generation(lib, models):
    """Greedy generation through the library's entry point (recorded and eager decode steps) against the plain
    implementation's choice, as long as that choice has a margin."""
    for dtype, graph in (("float32", True), ("float32", False), ("bfloat16", True)):
        folder, cfg, W = models["A", dtype]
        eng = lib.load(folder, dtype=dtype, max_tokens=4096)
        prompts = [tokens(cfg, 70, 21), tokens(cfg, 3, 22), tokens(cfg, 1, 23)]
        new = eng.generate(prompts, max_new_tokens=90, temperature=0.0, use_graph=graph)
        assert all(len(t) == 90 for t in new)
        if graph:
            assert eng.decode_counts["replayed"] > 50
        margin = 1e-3 if dtype == "float32" else 0.15
        checked = 0
        for p, out in zip(prompts, new):
            logits = P.forward(W, cfg, list(p) + out)
            # causal: row len(p) - 1 + k of the logits over the prompt and what was generated decides token k, so every
            # token is checked by itself wherever the plain logits leave a margin
            for k, t in enumerate(out):
                row = logits[len(p) - 1 + k]
                top2 = torch.topk(row, 2).values
                if (top2[0] - top2[1]).item() < margin:
                    continue
                assert t == int(row.argmax()), (dtype, graph, k)
                checked += 1
        assert checked > (250 if dtype == "float32" else 100), checked


def test_experts_sorted_by_expert_against_every_token_through_every_expert(lib):
    """A prompt long enough that tokens are listed by expert gives what the stacked products give."""
    from llm_infer_amd.parts.feed_forward import RoutedExperts
    from llm_infer_amd.registry import config_from_dict
    from llm_infer_amd.weights.loader import place_tensor
    raw = M.config(64, 50, [M.layer(M.mlstm(1, 8, 8), M.moe(3, 2, 48, shared=32))])
    cfg = config_from_dict(raw)
    spec = cfg._feed_forward("", raw["layers"][0]["mlp"]).with_prefix("")
    g = torch.Generator().manual_seed(31)
    W = M.mlp_weights(raw["layers"][0]["mlp"], 64, g, torch.bfloat16)
    h = torch.randn(600, 64, generator=g)
    ref = P.moe_ff(h.to(torch.bfloat16).double(), M.widen(W), raw["layers"][0]["mlp"])
    for dtype in ("float32", "bfloat16"):
        part = RoutedExperts(**spec.params, prefix="", dtype=DT[dtype], device=DEV)
        wanted = part.params()
        assert set(wanted) == set(W)
        part.bind({n: place_tensor(W[n], wanted[n].kind, DT[dtype], DEV) for n in wanted})
        outs = []
        for limit in (1, 10 ** 9):                     # sorted by expert from the first row on; never
            part.GROUPED_FROM = limit
            res = torch.zeros(600, 64, device=DEV)
            part.forward(h.to(DEV).to(torch.bfloat16).to(DT[dtype]), res)
            outs.append(res.cpu())
        # rows whose choice has a margin (the router reads the same rounded input in both runs, so they agree anyway)
        assert error(outs[1], ref) < TOL[dtype]
        assert error(outs[0], outs[1]) < (1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_in_three_schedules(lib, models, dtype, tmp_path):
    folder, cfg, W = models["B", dtype]
    reqs = {"r1": tokens(cfg, 75, 41), "r2": tokens(cfg, 1, 42), "r3": tokens(cfg, 140, 43)}
    ref = {r: P.forward(W, cfg, t) for r, t in reqs.items()}
    for k, (steps, where) in enumerate((TU.steps_whole(reqs), TU.steps_tail(reqs, 33), TU.steps_batches(reqs, 3, {"r1": 10, "r3": 70}))):
        out_dir = str(tmp_path / f"out{k}")
        got = TU.run_trace(folder, dtype, steps, where, cfg["vocab"], 300, out_dir)
        assert set(got) == {(r, p) for r, t in reqs.items() for p in range(len(t))}
        for r, t in reqs.items():
            g = torch.stack([torch.from_numpy(got[r, p].copy()) for p in range(len(t))])
            compare(g, ref[r], dtype)


def test_command_line_reports_and_generates(lib, models):
    folder, cfg, W = models["A", "float32"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompts = [tokens(cfg, 9, 51), tokens(cfg, 2, 52)]
    cmd = [sys.executable, os.path.join(root, "bin", "infer"), folder, "-n", "6", "-t", "0", "--dtype", "float32", "-T", "64"]
    for p in prompts:
        cmd += ["--tokens", ",".join(map(str, p))]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = [json.loads(line.split("tokens: ", 1)[1]) for line in res.stdout.splitlines() if " tokens: [" in line]
    assert len(got) == 2
    for p, new in zip(prompts, got):
        toks = list(p)
        for t in new:
            last = P.forward(W, cfg, toks)[-1]
            top2 = torch.topk(last, 2).values
            if (top2[0] - top2[1]).item() > 1e-3:
                assert t == int(last.argmax())
            toks.append(t)
    for word in ("Dimensions: 96", "Vocab size: 131"):
        assert word in res.stdout, res.stdout
    info = subprocess.run([sys.executable, os.path.join(root, "bin", "model_info"), folder], capture_output=True, text=True,
                          timeout=300)
    assert info.returncode == 0 and "Architecture: Dupolorn" in info.stdout and "The tensors fit the model." in info.stdout
