"""Dupolorn configurations drawn at random (seeded): any order of the three mixers, layers with dense, routed or no
feed-forward, sizes that are no multiples of anything, one to six taps, with and without a soft cap.  Each runs a whole
prompt, portions, token-by-token decoding and a ragged batch in float32 (against the plain implementation, and equal to
rounding among the schedules) and a whole prompt and a batch in bfloat16 (every expert chosen there: a choice that
rounding could turn reaches every later token).  The latent attention's sizes are drawn within the pairs of sizes whose
matrix-core kernels the build entry compiles, so that no test waits for a compiler, and now and then beyond what those
kernels take."""
import json
import random

import pytest
import torch

import dupolorn_models as M
import plain_dupolorn as P

pytestmark = pytest.mark.gpu
PAIRS = ((48, 32), (48, 64), (64, 64), (80, 96), (16, 32), (64, 32), (128, 128))     # (key size, value size) as padded


def draw(seed):
    r = random.Random(seed)
    width = r.choice([64, 72, 96, 100, 128, 160])
    layers = []
    for _ in range(r.randint(1, 5)):
        kind = r.random()
        if kind < 0.6:
            kp, vp = r.choice(PAIRS)
            rank = r.randint(max(1, vp - 31), min(vp, kp))              # the latent: within its value block, not wider than the key
            rot = r.choice([0, 2, 4, 8, 16])
            rot = min(rot, (kp - rank) // 2 * 2)
            if kp - rank - rot >= 16:                                     # keep the key inside its padded size's last 16
                rank = min(vp, kp - rot)
            if r.random() < 0.1:
                rank, rot = 270, 8                                        # beyond the matrix-core kernels' sizes
            dims = r.choice([rot, rot, max(0, rot - 2)]) if rot else 0
            d = r.choice([0, 4, 16, 24, 40]) if rot else r.choice([4, 16, 24])
            mixer = M.latent(r.choice([1, 2, 3, 4, 5, 8]), d, rot, r.choice([4, 10, 16, 33, 64]), rank, second=r.random() < 0.5,
                             base=r.choice([50.0, 10000.0, 500000.0]), dims=dims, scale=r.uniform(0.05, 0.3))
        else:
            mixer = M.mlstm(r.randint(1, 4), r.choice([1, 7, 16, 40, 64, 100]), r.choice([4, 10, 16, 33, 64, 80, 130]),
                            cap=r.choice([1.0, 8.0, 15.0, 50.0]))
        kind = r.random()
        if kind < 0.25:
            mlp = None
        elif kind < 0.5:
            mlp = M.dense(r.choice([24, 50, 128]))
        else:
            experts = r.randint(1, 12)
            mlp = M.moe(experts, r.randint(1, min(4, experts)), r.choice([8, 24, 40]), shared=r.choice([None, 16, 40]))
        layers.append(M.layer(mixer, mlp))
    buckets = r.choice([1, 7, 64, 1021])
    return M.config(width, r.randint(40, 300), layers, taps=r.randint(1, 6), eps=r.choice([1e-6, 1e-5, 1e-3]),
                    scale=r.uniform(0.5, 4.0), bigram=(buckets, r.randint(1, 200000), r.randint(1, 999)),
                    softcap=r.choice([None, 5.0, 30.0]))


@pytest.fixture(scope="module")
def lib():
    import llm_infer_amd
    return llm_infer_amd


def all_rows(n):
    return list(range(n))


@pytest.mark.parametrize("seed", range(12))
def test_a_random_configuration_in_every_schedule(lib, seed, tmp_path):
    drawn = draw(2000 + seed)
    g = torch.Generator().manual_seed(seed)
    n = 150
    toks = torch.randint(0, drawn["vocab"], (n,), generator=g).tolist()
    short = torch.randint(0, drawn["vocab"], (37,), generator=g).tolist()
    W = M.random_weights(drawn, 7 + seed)
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 3e-2)):
        cfg = json.loads(json.dumps(drawn))
        if dtype == "bfloat16":
            for layer in cfg["layers"]:
                if layer["mlp"] is not None and layer["mlp"]["kind"] == "moe":
                    layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
        folder = str(tmp_path / dtype)
        M.write_model(folder, cfg, W)
        ref = P.forward(M.widen(W), cfg, toks)
        ref_short = P.forward(M.widen(W), cfg, short)
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
        if dtype == "float32":
            assert M.row_error(got_b, whole) < 2e-5, cfg
            s = eng.alloc_slot()
            pieces, at = [], 0
            for k in (63, 2, 1, 34, n - 100):
                pieces.append(eng.step([s], [toks[at:at + k]], [all_rows(k)]).cpu())
                at += k
            eng.free_slot(s)
            assert M.row_error(torch.cat(pieces), whole) < 2e-5, cfg
