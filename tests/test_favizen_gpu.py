"""Favizen on the GPU against the plain implementation: every kernel and mixer alone, whole prompts, prompts cut into
portions, decoding token by token, batches of unequal requests against each alone, slots and pages used again, keys
far away, at page borders and just inside and just outside a window or a chunk, the first tokens, long decoding, other
sizes, a layer that reads another layer's keys, and greedy generation through the library's entry point.

Where random weights would hide a fault, a token's key is made to stand out for every query (``favizen_models.stand_out``)
and the test first shows, with the plain implementation alone, that the fault it looks for would move the result far
beyond the tolerance."""
import json
import os
import subprocess
import sys

import pytest
import torch

import favizen_models as M
import plain_favizen as P
import trace_util as TU

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {"float32": 1e-4, "bfloat16": 3e-2}
SHOWS = {"float32": 20.0, "bfloat16": 2.0}      # a fault shows if it moves the result by this many tolerances
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
        folder = str(tmp_path_factory.mktemp(f"favizen_{name}"))
        M.write_model(folder, cfg, W)
        out[name] = (folder, cfg, M.widen(W))
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def step_context(slots, lens_before, toks):
    from llm_infer_amd.engine.step import StepContext
    return StepContext(DEV, list(slots), [list(t) for t in toks], list(lens_before), [[] for _ in toks])


def error(got, ref):
    """Largest difference relative to the reference's spread."""
    return ((got.double() - ref.double()).abs().max() / ref.double().std()).item()


def rows(n):
    return list(range(n))


def load(lib, tmp_path, cfg, W, dtype, name="m", max_tokens=4096):
    folder = str(tmp_path / f"{name}_{dtype}")
    M.write_model(folder, cfg, W)
    return lib.load(folder, dtype=dtype, max_tokens=max_tokens)


def run_schedule(eng, reqs, schedule):
    """``schedule``: a list of steps, each {request: number of tokens it brings}; all rows wanted.  Returns
    {request: logits [n, vocab]}."""
    slot, at, out = {}, {r: 0 for r in reqs}, {r: [] for r in reqs}
    for step in schedule:
        rs = list(step)
        for r in rs:
            if r not in slot:
                slot[r] = eng.alloc_slot()
        res = eng.step([slot[r] for r in rs], [reqs[r][at[r]:at[r] + step[r]] for r in rs], [rows(step[r]) for r in rs]).cpu()
        for r, part in zip(rs, res.split([step[r] for r in rs])):
            out[r].append(part)
            at[r] += step[r]
            if at[r] == len(reqs[r]):
                eng.free_slot(slot.pop(r))
    return {r: torch.cat(v) for r, v in out.items()}


# ---------------------------------------------------------------------------- kernels alone
def test_bias_scale_and_the_norm_with_the_residual_sum(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    for width, n in ((96, 5), (70, 5), (8200, 5), (8192, 5), (96, 100), (1024, 70)):      # (few rows and many: two instantiations)
        x, y = torch.randn(n, width, generator=g), torch.randn(n, width, generator=g) * 3
        w, b = torch.randn(width, generator=g), torch.randn(width, generator=g)
        for bias in (None, b):
            z = y.double() + (0 if bias is None else bias.double())
            ref = x.double() + z / torch.sqrt(z.pow(2).mean(-1, keepdim=True) + 1e-3) * w.double()
            got = ops.rmsnorm_add(x.clone().to(DEV), y.to(DEV), w.to(DEV), 1e-3, None if bias is None else bias.to(DEV)).cpu()
            assert error(got, ref) < 3e-6, width
            # with the norm that reads the finished rows next taken along
            for dt in (torch.float32, torch.bfloat16):
                xd, w2 = x.clone().to(DEV), (w * 0.5 + 1).to(DEV)
                ops.rmsnorm_add(xd, y.to(DEV), w.to(DEV), 1e-3, None if bias is None else bias.to(DEV), (w2, 1e-5, dt))
                assert error(xd.cpu(), ref) < 3e-6
                ready = ops.prepared_rmsnorm(xd, w2, 1e-5, dt)
                assert ready is not None and ops.prepared_rmsnorm(xd, w2, 1e-4, dt) is None
                nref = ref / torch.sqrt(ref.pow(2).mean(-1, keepdim=True) + 1e-5) * w2.double().cpu()
                # (a 16-bit result: every element within that type's rounding of the reference)
                assert torch.allclose(ready.cpu().double(), nref, rtol=1e-5 if dt == torch.float32 else 2.0 ** -8, atol=1e-5)
                ops.add_bias(xd, 0, w2)                                   # anything written into the rows voids what was prepared
                assert ops.prepared_rmsnorm(xd, w2, 1e-5, dt) is None
    rows_ = torch.randn(7, 50, generator=g)
    b = torch.randn(20, generator=g)
    got = ops.add_bias(rows_.clone().to(DEV), 13, b.to(DEV)).cpu()
    ref = rows_.clone()
    ref[:, 13:33] += b
    assert torch.equal(got, ref)
    assert torch.equal(ops.scale_values(rows_.clone().to(DEV), 0.3).cpu(), rows_ * torch.tensor(0.3))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows_", [3, 12, 40, 100, 300, 1100])
def test_products_with_a_bias_and_with_the_clamped_gated_activation(lib, dtype, rows_):
    """The two epilogues in every product kernel that a row count reaches, with and without a bias, with a tail that
    takes another limit, against float64."""
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(2 + rows_)
    for K, F_, tail in ((96, 70, 0), (256, 200, 56), (1024, 1536, 512)):
        x = torch.randn(rows_, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(2 * F_, K, generator=g) * K ** -0.5 * 2).to(torch.bfloat16)
        bias = torch.randn(2 * F_, generator=g)
        xd, wd = x.to(DEV).to(DT[dtype]), ops.prepare_weight(w.to(DEV).to(DT[dtype]))
        z = x.double() @ w.double().T
        got = ops.linear(xd, wd, ops.EPI_BIAS, out_dtype=torch.float32, params=ops.glu_params(bias.to(DEV))).cpu()
        assert error(got, z + bias.double()) < (1e-5 if dtype == "float32" else 2e-2)
        for b in (None, bias):
            zz = z + (0 if b is None else b.double())
            gate, up = zz[:, 0::2], zz[:, 1::2]
            cut = F_ - tail
            ref = torch.cat([P.clamped_glu(gate[:, :cut], up[:, :cut], 1.5), P.clamped_glu(gate[:, cut:], up[:, cut:], 0.5)], 1)
            params = ops.glu_params(None if b is None else b.to(DEV), 1.5, 0.5, 1.702, 1.0, cut)
            got = ops.linear(xd, wd, ops.EPI_CLAMPGLU, out_dtype=DT[dtype], params=params).cpu()
            assert got.shape == (rows_, F_)
            assert error(got, ref) < (1e-5 if dtype == "float32" else 2e-2), (K, F_, tail, b is None)


def test_experts_by_table(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    V, E, top, T = 40, 7, 3, 25
    table = torch.rand(V, E, generator=g).argsort(-1)[:, :top].to(torch.int32).contiguous()
    toks = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    gate = torch.randn(T, generator=g)
    for has_gate in (0, 1, 2):
        got = ops.table_route(toks.to(DEV), table.to(DEV), E, gate.to(DEV) if has_gate == 1 else None, has_gate).cpu()
        ref = torch.zeros(T, E + (1 if has_gate else 0))
        for t in range(T):
            ref[t, table[toks[t]].long()] = 1.0 / top
        if has_gate:
            ref[:, E] = torch.sigmoid(gate) if has_gate == 1 else 1.0
        assert torch.allclose(got, ref, atol=1e-6)


@pytest.mark.parametrize("taps", [1, 2, 5])
def test_convolution_on_the_way_into_the_cache_in_portions(lib, taps):
    """The store kernel's convolution: portions shorter than its reach, two sequences at once, a slot used again; q as it
    comes back is compared (keys and values take the same path and are checked through the mixers)."""
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    H, d, extra = 2, 5, 3
    C = H * d
    w = torch.randn(C, taps, generator=g)
    u = {r: torch.randn(n, C + extra, generator=g) for r, n in (("a", 11), ("b", 6), ("c", 4))}
    hist = torch.full((4, max(taps - 1, 1), C), 7.0, device=DEV)           # what an earlier sequence left
    slot = {"a": 2, "b": 0, "c": 2}
    got, at = {r: [] for r in u}, {r: 0 for r in u}
    for step in ({"a": 1}, {"a": 2, "b": 5}, {"a": 1, "b": 1}, {"a": 7}, {"c": 1}, {"c": 3}):
        rs = list(step)
        for r in rs:
            if at[r] == 0:
                hist[slot[r]] = 0.0                                        # the cache clears a slot's state when it hands it out
        ctx = step_context([slot[r] for r in rs], [at[r] for r in rs], [[0] * step[r] for r in rs])
        x = torch.cat([u[r][at[r]:at[r] + step[r]] for r in rs]).to(DEV)
        q = ops.rot_store(x, 0, 0, 0, None, 0, ctx.pos, ctx.tok_slot, None, H, 0, d, d, torch.float32, (w.to(DEV), hist))
        ops.conv_history(x, 0, C, taps, hist, ctx)
        out = q[:, :, :d].reshape(-1, C).cpu()
        assert float(q[:, :, d:].abs().max()) == 0.0                        # zeros behind a head's own dimensions
        for r, part in zip(rs, out.split([step[r] for r in rs])):
            got[r].append(part)
            at[r] += step[r]
    for r in u:
        ref = P.causal_conv(u[r][:, :C].double(), w.double())
        assert error(torch.cat(got[r]), ref) < 1e-6, r


# ---------------------------------------------------------------------------- the mixers alone
def build_mixer(raw_cfg, i, weights, dtype):
    """Layer i's mixer as the configuration describes it, with the given tensors bound."""
    import llm_infer_amd.parts  # noqa: F401  (registers the parts)
    from llm_infer_amd.registry import config_from_dict, lookup
    from llm_infer_amd.weights.loader import place_tensor
    cfg = config_from_dict(raw_cfg)
    spec, position = cfg._mixer(i, raw_cfg["layers"][i]).with_prefix(""), cfg._position(raw_cfg["layers"][i])
    pos = None
    if position is not None:
        pos = lookup("position", position.kind)(**position.params, prefix="", dtype=DT[dtype], device=DEV)
    part = lookup("mixer", spec.kind)(**spec.params, position=pos, prefix="", dtype=DT[dtype], device=DEV)
    wanted = part.params()
    assert set(wanted) == set(weights), set(wanted) ^ set(weights)
    part.bind({n: place_tensor(weights[n], wanted[n].kind, DT[dtype], DEV) for n in wanted})
    return part


def run_mixer(part, h_of, schedule, dtype):
    """Runs a mixer over ``schedule`` (steps {request: tokens it brings}) on the inputs ``h_of[r]`` [n, width]; returns
    {r: what the mixer added, [n, width]}."""
    from llm_infer_amd.cache import Cache
    specs = part.cache_specs()
    cache = Cache(specs, 8192, 8192, DT[dtype], DEV)
    views = [cache.view(i) for i in range(len(specs))]
    slot, at, out = {}, {r: 0 for r in h_of}, {r: [] for r in h_of}
    for step in schedule:
        rs = list(step)
        for r in rs:
            if r not in slot:
                slot[r] = cache.alloc_slot()
        cache.grow([slot[r] for r in rs], [at[r] + step[r] for r in rs], filled=True)
        ctx = step_context([slot[r] for r in rs], [at[r] for r in rs], [[0] * step[r] for r in rs])
        h = torch.cat([h_of[r][at[r]:at[r] + step[r]] for r in rs]).to(DEV).to(DT[dtype])
        res = torch.zeros((h.shape[0], h.shape[1]), dtype=torch.float32, device=DEV)
        part.forward(h, ctx, views, res)
        cache.trim_windows([slot[r] for r in rs])
        for r, part_rows in zip(rs, res.cpu().split([step[r] for r in rs])):
            out[r].append(part_rows)
            at[r] += step[r]
        for r in rs:
            if at[r] == h_of[r].shape[0]:
                cache.free_slot(slot.pop(r))
    return {r: torch.cat(v) for r, v in out.items()}


SCHEDULES = {
    "whole": lambda n, m: [{"a": n}, {"b": m}],
    # portions down to two tokens and one, across page edges (64) and the masks' edges
    "portions": lambda n, m: [{"a": 61}, {"a": 2}, {"a": 1}, {"a": 2}, {"a": 70}, {"a": n - 136}, {"b": 1}, {"b": m - 1}],
    # unequal requests together, decoded together, the longer one alone, then a slot used again
    "together": lambda n, m: [{"a": n - 20, "b": m - 5}] + [{"a": 1, "b": 1}] * 5 + [{"a": 1}] * 15 + [{"c": 30}],
}


@pytest.mark.parametrize("schedule", sorted(SCHEDULES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mixer", [
    M.rotary(3, 1, 20, 9, dims=12, base=500.0),                                  # a padded head, a window below a page
    M.rotary(8, 2, 64, 100, scaling=(16.0, 1.0, 2.0, 128), base=2e5),             # a window across pages, stretched frequencies
    M.rotary(4, 4, 16, 1000, dims=0),                                            # no rotation, a window never reached
    M.rotary(2, 1, 48, 64, dims=48, scaling=(2.0, 1.0, 2.0, 40)),                # window = page
    M.convolved(4, 2, 16, 24, 50, taps=2),                                       # values wider than keys
    M.convolved(1, 1, 8, 40, 7, taps=5),                                         # chunks shorter than a tile, five taps
    M.convolved(16, 1, 128, 64, 130, taps=4),                                    # sixteen heads on one key head
    M.convolved(5, 5, 32, 16, 64, taps=1),                                       # one tap, chunk = page
    M.convolved(8, 2, 64, 64, 70, taps=3),                                       # keys and values of one size: the prompt kernel
    M.convolved(6, 1, 32, 32, 200, taps=2),                                      # with slopes and chunks, six heads on one key head
    M.rotary(4, 2, 24, 70, dims=8),                                              # a window on the kernel of padded sizes
], ids=lambda m: f"{m[0]}-{m[1]['heads']}x{m[1]['dim']}-{m[1]['mask']['size']}")
def test_mixer_alone(lib, mixer, dtype, schedule):
    width, n, m_ = 96, 200, 40
    raw = M.config(width, 50, [M.layer(mixer, None)])
    g = torch.Generator().manual_seed(11)
    W = M.mixer_weights(mixer[0], mixer[1], width, g, torch.bfloat16, sharp=2.0)
    part = build_mixer(raw, 0, W, dtype)
    h_of = {r: torch.randn(k, width, generator=g).to(torch.bfloat16).float() for r, k in (("a", n), ("b", m_), ("c", 30))}
    sched = SCHEDULES[schedule](n, m_)
    got = run_mixer(part, {r: h_of[r] for r in {k for s in sched for k in s}}, sched, dtype)
    Wd = M.widen(W)
    fn = P.attention_mixer if mixer[0] == "attention" else P.attention2_mixer
    for r, rows_ in got.items():
        ref = fn(h_of[r].double(), Wd, mixer[1])
        tol = M.tolerance(dtype, ref, fn(h_of[r].double(), Wd, mixer[1], round_to=torch.bfloat16), error)
        assert error(rows_, ref) < tol, r


# ---------------------------------------------------------------------------- edges, far keys, sinks
def edge_case(kind, dtype_w=torch.bfloat16):
    """A one-layer model whose token 7 has a key that stands out, the layer's mask size, and the sizes one off."""
    # (keys and values of one size that is a multiple of 16 run prompts on one kernel, other sizes on another)
    if kind == "window":
        mixer, size = M.rotary(4, 2, 32, 70, dims=16, base=300.0, scaling=(4.0, 1.0, 2.0, 30)), 70
    elif kind == "window_padded":
        mixer, size = M.rotary(4, 2, 24, 70, dims=8, base=300.0), 70
    elif kind == "chunk":
        mixer, size = M.convolved(4, 2, 32, 32, 70, taps=1), 70
    else:
        mixer, size = M.convolved(4, 2, 32, 16, 70, taps=1), 70
    cfg = M.config(64, 60, [M.layer(mixer, M.dense(48))], scale=2.0, logit_scale=0.5)
    W = M.stand_out(M.random_weights(cfg, 77, dtype_w), cfg, 0, 7, strength=8.0)
    return cfg, W, size


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["window", "window_padded", "chunk", "chunk_other"])
def test_a_key_just_inside_and_just_outside_the_mask_in_prompts_portions_and_decoding(lib, kind, dtype, tmp_path):
    cfg, W, size = edge_case(kind)
    Wd = M.widen(W)
    n = 160
    base = [t if t != 7 else 8 for t in tokens(cfg, n, 5)]
    # the token that stands out sits so that the probe rows see it just still, and the next row no more:
    # window: the key at 20 is seen up to position 20 + size - 1; chunk: the key at size - 3 is seen up to size - 1
    window = kind.startswith("window")
    at = 20 if window else size - 3
    toks = list(base)
    toks[at] = 7
    last_seen = at + size - 1 if window else size - 1
    ref = P.forward(cfg, Wd, toks)
    tol = M.tolerance(dtype, ref, P.forward(cfg, Wd, toks, round_to=torch.bfloat16))
    # the plain implementation alone: one position more or less of mask moves the rows at the edge far beyond the tolerance
    for wrong in (size - 1, size + 1):
        off = P.forward(M.with_mask(cfg, 0, wrong), Wd, toks)
        edge_rows = [last_seen, last_seen + 1] if window else [last_seen - 1, last_seen, last_seen + 1, last_seen + 2]
        assert M.row_error(off[edge_rows], ref[edge_rows]) > SHOWS[dtype] * tol, (kind, wrong)
    eng = load(lib, tmp_path, cfg, W, dtype)
    reqs = {"a": toks}
    for name, sched in (("prompt", [{"a": n}]),
                        ("portions", [{"a": last_seen - 1}, {"a": 2}, {"a": 2}, {"a": n - last_seen - 3}]),
                        ("decoding", [{"a": last_seen - 3}] + [{"a": 1}] * 8 + [{"a": n - last_seen - 5}])):
        got = run_schedule(eng, reqs, sched)["a"]
        assert M.row_error(got, ref) < tol, (kind, name)


@pytest.mark.parametrize("vdim", [16, 32])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_and_a_sink_that_outweighs_it(lib, dtype, vdim, tmp_path):
    mixer = M.convolved(4, 1, 32, vdim, 1000, taps=2)
    cfg = M.config(64, 60, [M.layer(mixer, None)], scale=2.0)
    # (strong enough to outweigh hundreds of keys and, in the heads with small slopes, the bias over 700 positions; not so
    # strong that no sink could weigh against it)
    W = M.stand_out(M.random_weights(cfg, 78), cfg, 0, 7, strength=5.0 if vdim == 16 else 3.5)
    n = 700
    base = [t if t != 7 else 8 for t in tokens(cfg, n, 6)]
    toks = list(base)
    toks[3] = 7
    Wd = M.widen(W)
    ref, without = P.forward(cfg, Wd, toks), P.forward(cfg, Wd, base)
    tol = M.tolerance(dtype, ref, P.forward(cfg, Wd, toks, round_to=torch.bfloat16))
    far = list(range(600, 700))
    assert M.row_error(without[far], ref[far]) > SHOWS[dtype] * tol        # the rows far away feel the key at position 3
    eng = load(lib, tmp_path, cfg, W, dtype)
    for sched in ([{"a": n}], [{"a": 640}] + [{"a": 1}] * 60, [{"a": 130}, {"a": 500}, {"a": 70}]):
        assert M.row_error(run_schedule(eng, {"a": toks}, sched)["a"], ref) < tol
    # sinks that differ widely between the heads
    W2 = dict(W)
    W2["l0.mix.sink"] = torch.tensor([-4.0, 9.0, 2.0, 30.0]).to(torch.bfloat16)
    ref2 = P.forward(cfg, M.widen(W2), toks)
    tol = M.tolerance(dtype, ref2, P.forward(cfg, M.widen(W2), toks, round_to=torch.bfloat16))
    assert M.row_error(ref2[far], ref[far]) > SHOWS[dtype] * tol
    eng = load(lib, tmp_path, cfg, W2, dtype, name="sink")
    for sched in ([{"a": n}], [{"a": 690}] + [{"a": 1}] * 10):
        assert M.row_error(run_schedule(eng, {"a": toks}, sched)["a"], ref2) < tol


# ---------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("name", sorted(M.ALL))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_model_whole_first_tokens_portions_and_token_by_token(lib, models, dtype, name):
    folder, cfg, W = models[name]
    n = 210
    toks = tokens(cfg, n, 9)
    ref = P.forward(cfg, W, toks)
    tol = M.tolerance(dtype, ref, P.forward(cfg, W, toks, round_to=torch.bfloat16))
    eng = lib.load(folder, dtype=dtype, max_tokens=2048)
    reqs = {"a": toks}
    whole = run_schedule(eng, reqs, [{"a": n}])["a"]
    assert M.row_error(whole, ref) < tol
    for k in (1, 2, 3):                                                     # the first tokens alone
        assert M.row_error(run_schedule(eng, {"a": toks[:k]}, [{"a": k}])["a"], ref[:k]) < tol
    portions = run_schedule(eng, reqs, [{"a": 2}, {"a": 1}, {"a": 62}, {"a": 2}, {"a": 5}, {"a": 129}, {"a": n - 201}])["a"]
    one_by_one = run_schedule(eng, reqs, [{"a": 1}] * n)["a"]
    for got in (portions, one_by_one):
        assert M.row_error(got, ref) < tol
        if dtype == "float32":
            assert M.row_error(got, whole) < 2e-5


@pytest.mark.parametrize("name", sorted(M.ALL))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_together_against_each_alone(lib, models, dtype, name):
    folder, cfg, W = models[name]
    reqs = {"a": tokens(cfg, 150, 12), "b": tokens(cfg, 1, 13), "c": tokens(cfg, 67, 14), "d": tokens(cfg, 230, 15),
            "e": tokens(cfg, 40, 16)}
    ref = {r: P.forward(cfg, W, t) for r, t in reqs.items()}
    tol = {r: M.tolerance(dtype, ref[r], P.forward(cfg, W, t, round_to=torch.bfloat16)) for r, t in reqs.items()}
    eng = lib.load(folder, dtype=dtype, max_tokens=1024, n_slots=4)
    # slots and pages used before, and given back in between
    first = run_schedule(eng, {"a": reqs["a"], "e": reqs["e"]}, [{"a": 150, "e": 40}])
    sched = [{"a": 140, "b": 1, "c": 60, "d": 190}] + [{"a": 1, "c": 1, "d": 1}] * 7 + [{"a": 1, "d": 1}] * 3 + \
        [{"d": 1, "e": 40}] + [{"d": 1}] * 29
    got = run_schedule(eng, reqs, sched)
    for r in reqs:
        assert M.row_error(got[r], ref[r]) < tol[r], r
    for r in first:
        assert M.row_error(first[r], ref[r]) < tol[r], r
    assert eng.cache.tokens_free() == (eng.cache.n_pages - 1) * 64         # every page came back


@pytest.mark.parametrize("dtype,graph", [("float32", True), ("bfloat16", True), ("bfloat16", False)])
def test_long_decoding_and_generation(lib, models, dtype, graph):
    """Greedy generation through the library's own loop (recorded and eager decode steps), across windows, chunks and
    pages, against the plain implementation's choice wherever its logits leave a margin."""
    folder, cfg, W = models["A"]
    eng = lib.load(folder, dtype=dtype, max_tokens=4096)
    prompts = [tokens(cfg, 70, 21), tokens(cfg, 3, 22), tokens(cfg, 1, 23)]
    new = eng.generate(prompts, max_new_tokens=150, temperature=0.0, use_graph=graph)
    assert all(len(t) == 150 for t in new)
    if graph:
        assert eng.decode_counts["replayed"] > 100
    checked = 0
    for p, out in zip(prompts, new):
        logits = P.forward(cfg, W, list(p) + out)
        margin = (1e-3 if dtype == "float32" else 0.15) * logits.std().item()
        for k, t in enumerate(out):
            row = logits[len(p) - 1 + k]
            top2 = torch.topk(row, 2).values
            if (top2[0] - top2[1]).item() < margin:
                continue
            assert t == int(row.argmax()), (dtype, graph, k)
            checked += 1
    assert checked > (400 if dtype == "float32" else 100), checked


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_experts_sorted_by_expert_against_every_token_through_every_expert(lib, dtype):
    """A prompt long enough that tokens are listed by expert gives what the stacked products give."""
    from llm_infer_amd.engine.step import StepContext
    from llm_infer_amd.parts.feed_forward import RoutedExperts
    from llm_infer_amd.registry import config_from_dict
    from llm_infer_amd.weights.loader import place_tensor
    mlp = M.moe(3, 2, 48, limit=1.2, shared=32, shared_limit=0.6)
    raw = M.config(64, 50, [M.layer(M.rotary(1, 1, 16, 8), mlp)])
    spec = config_from_dict(raw)._feed_forward("", mlp).with_prefix("")
    g = torch.Generator().manual_seed(31)
    W = M.mlp_weights(mlp, 64, 50, g, torch.bfloat16)
    h = torch.randn(600, 64, generator=g).to(torch.bfloat16)
    toks = torch.randint(0, 50, (600,), generator=g).tolist()
    ref = P.table_experts(h.double(), torch.tensor(toks), M.widen(W), mlp)
    ctx = StepContext(DEV, [0], [toks], [0], [[]])
    part = RoutedExperts(**spec.params, prefix="", dtype=DT[dtype], device=DEV)
    wanted = part.params()
    assert set(wanted) == set(W)
    part.bind({n: place_tensor(W[n], wanted[n].kind, DT[dtype], DEV) for n in wanted})
    outs = []
    for limit in (1, 10 ** 9):                     # sorted by expert from the first row on; never
        part.GROUPED_FROM = limit
        res = torch.zeros(600, 64, device=DEV)
        part.forward(h.to(DEV).to(DT[dtype]), res, ctx)
        outs.append(res.cpu())
    assert error(outs[1], ref) < TOL[dtype]
    assert error(outs[0], ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_in_three_schedules(lib, models, dtype, tmp_path):
    folder, cfg, W = models["B"]
    reqs = {"r1": tokens(cfg, 75, 41), "r2": tokens(cfg, 1, 42), "r3": tokens(cfg, 140, 43)}
    ref = {r: P.forward(cfg, W, t) for r, t in reqs.items()}
    tol = {r: M.tolerance(dtype, ref[r], P.forward(cfg, W, t, round_to=torch.bfloat16)) for r, t in reqs.items()}
    for k, (steps, where) in enumerate((TU.steps_whole(reqs), TU.steps_tail(reqs, 33), TU.steps_batches(reqs, 3, {"r1": 10, "r3": 70}))):
        out_dir = str(tmp_path / f"out{k}")
        got = TU.run_trace(folder, dtype, steps, where, cfg["vocab"], 300, out_dir)
        assert set(got) == {(r, p) for r, t in reqs.items() for p in range(len(t))}
        for r, t in reqs.items():
            g = torch.stack([torch.from_numpy(got[r, p].copy()) for p in range(len(t))])
            assert M.row_error(g, ref[r]) < tol[r], (k, r)


def test_command_line_reports_and_generates(lib, models):
    folder, cfg, W = models["A"]
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
            last = P.forward(cfg, W, toks)[-1]
            top2 = torch.topk(last, 2).values
            if (top2[0] - top2[1]).item() > 1e-3:
                assert t == int(last.argmax())
            toks.append(t)
    for word in ("Dimensions: 96", "Vocab size: 131"):
        assert word in res.stdout, res.stdout
    info = subprocess.run([sys.executable, os.path.join(root, "bin", "model_info"), folder], capture_output=True, text=True,
                          timeout=300)
    assert info.returncode == 0 and "Architecture: Favizen" in info.stdout and "The tensors fit the model." in info.stdout
