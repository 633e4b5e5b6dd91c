"""Favizen configurations drawn at random (seeded): any order of the two mixers, layers that read an earlier layer's
keys (through the same mask or another), dense, routed or no feed-forward, sizes that are no multiples of anything,
windows and chunks from one position to beyond the prompt, one to six taps.  Each runs a whole prompt, portions,
token-by-token decoding and a ragged batch in float32 and bfloat16 against the plain implementation (in float32 the
schedules also agree with each other to rounding).  Head sizes are drawn within the pairs whose matrix-core kernels
the build entry compiles, so that no test waits for a compiler."""
import random

import pytest
import torch

import favizen_models as M
import plain_favizen as P

pytestmark = pytest.mark.gpu
PAIRS = ((16, 32), (32, 32), (48, 64), (64, 64), (16, 64), (128, 64), (32, 64), (64, 32))     # (key size, value size) as padded


def draw(seed):
    r = random.Random(seed)
    width = r.choice([64, 72, 96, 100, 128, 160])
    layers, owners = [], []
    for i in range(r.randint(1, 6)):
        size = r.choice([1, 2, 5, 31, 32, 33, 64, 65, 100, 128, 200, 1000])
        if r.random() < 0.5:
            kp = r.choice([p for p in PAIRS if (p[0] + 31) // 32 * 32 == p[1]])[0]        # values are keys: one size
            d = r.randint(max(2, kp - 15), kp)
            G = r.choice([1, 2, 3])
            dims = r.choice([0, 2, d // 2 * 2, d // 4 * 2])
            scaling = r.choice([None, (r.choice([2.0, 8.0, 32.0]), 1.0, r.choice([2.0, 4.0]), r.choice([16, 64, 512]))])
            mixer = M.rotary(G * r.choice([1, 2, 4, 5]), G, d, size, dims=dims, base=r.choice([50.0, 10000.0, 1e6]),
                             scaling=scaling if dims else None, scale=r.uniform(0.05, 0.3))
        else:
            kv_from = r.choice(owners) if owners and r.random() < 0.4 else None
            if kv_from is not None:
                o = layers[kv_from]["mixer"]
                mixer = M.convolved(o["heads"], o["kv_heads"], o["dim"], o["vdim"], r.choice([size, o["mask"]["size"]]),
                                    taps=r.randint(1, 6), kv_from=kv_from, scale=r.uniform(0.05, 0.3))
            else:
                kp, vp = r.choice(PAIRS)
                G = r.choice([1, 2, 3])
                d, dv = r.randint(max(1, kp - 15), kp), r.randint(vp - 31, vp)
                if r.random() < 0.3:
                    d = dv = r.choice([16, 32, 48, 64])                           # one size, a multiple of 16: the prompt kernel
                mixer = M.convolved(G * r.choice([1, 2, 4, 8]), G, d, dv, size, taps=r.randint(1, 6), scale=r.uniform(0.05, 0.3))
                owners.append(i)
        kind = r.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.5:
            mlp = M.dense(r.choice([24, 50, 128]), limit=r.choice([0.5, 1.0, 7.0]))
        else:
            experts = r.randint(1, 12)
            mlp = M.moe(experts, r.randint(1, min(4, experts)), r.choice([8, 24, 40]), limit=r.choice([0.5, 2.0]),
                        shared=r.choice([None, 16, 40]), shared_limit=r.choice([None, 0.3, 5.0]))
        layers.append(M.layer(mixer, mlp))
    return M.config(width, r.randint(40, 300), layers, eps=r.choice([1e-6, 1e-5, 1e-3]), scale=r.uniform(0.5, 20.0),
                    logit_scale=r.choice([1.0, 0.5, 0.37]))


@pytest.fixture(scope="module")
def lib():
    import llm_infer_amd
    return llm_infer_amd


def all_rows(n):
    return list(range(n))


@pytest.mark.parametrize("seed", range(14))
def test_a_random_configuration_in_every_schedule(lib, seed, tmp_path):
    cfg = draw(3000 + seed)
    g = torch.Generator().manual_seed(seed)
    n = 150
    toks = torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
    short = torch.randint(0, cfg["vocab"], (37,), generator=g).tolist()
    W = M.random_weights(cfg, 7 + seed, sharp=2.0)
    ref = P.forward(cfg, M.widen(W), toks)
    ref_short = P.forward(cfg, M.widen(W), short)
    rounded = P.forward(cfg, M.widen(W), toks, round_to=torch.bfloat16), P.forward(cfg, M.widen(W), short, round_to=torch.bfloat16)
    folder = str(tmp_path / "m")
    M.write_model(folder, cfg, W)
    for dtype in ("float32", "bfloat16"):
        tol = max(M.tolerance(dtype, ref, rounded[0]), M.tolerance(dtype, ref_short, rounded[1]))
        eng = lib.load(folder, dtype=dtype, max_tokens=1024)
        s = eng.alloc_slot()
        whole = eng.step([s], [toks], [all_rows(n)]).cpu()
        eng.free_slot(s)
        assert M.row_error(whole, ref) < tol, (cfg, dtype)
        # together with a shorter request, in slots used before, then both decoded
        a, b = eng.alloc_slot(), eng.alloc_slot()
        out = eng.step([a, b], [short[:30], toks[:140]], [all_rows(30), all_rows(140)]).cpu()
        rows_a, rows_b = [out[:30]], [out[30:]]
        for j in range(7):
            out = eng.step([a, b], [[short[30 + j]], [toks[140 + j]]], [[0], [0]]).cpu()
            rows_a.append(out[:1])
            rows_b.append(out[1:])
        eng.free_slot(a)
        rows_b += [eng.step([b], [[t]], [[0]]).cpu() for t in toks[147:]]
        eng.free_slot(b)
        got_a, got_b = torch.cat(rows_a), torch.cat(rows_b)
        assert M.row_error(got_a, ref_short) < tol and M.row_error(got_b, ref) < tol, (cfg, dtype)
        s = eng.alloc_slot()
        pieces, at = [], 0
        for k in (63, 2, 1, 34, n - 100):
            pieces.append(eng.step([s], [toks[at:at + k]], [all_rows(k)]).cpu())
            at += k
        eng.free_slot(s)
        assert M.row_error(torch.cat(pieces), ref) < tol, (cfg, dtype)
        if dtype == "float32":
            assert M.row_error(got_b, whole) < 2e-5 and M.row_error(torch.cat(pieces), whole) < 2e-5, cfg
