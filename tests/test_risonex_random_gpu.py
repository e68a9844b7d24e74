"""Risonex configurations drawn at random (seeded): any order of the two mixers, layers with dense, routed or no
feed-forward, loops anywhere or none, sizes that are no multiples of anything.  Each runs a whole prompt, portions,
token-by-token decoding and a ragged batch in float32 (against the plain implementation, and bit-equal among the
schedules) and a whole prompt and a batch in bfloat16.  The attention's sizes are drawn within the pairs of sizes whose
matrix-core kernels the build entry compiles, so that no test waits for a compiler."""
import random

import pytest
import torch

import plain_risonex as P
import risonex_models as M

pytestmark = pytest.mark.gpu
PAIRS = ((16, 32), (16, 160), (32, 64), (64, 32), (64, 128), (128, 128))     # (map size, value size) as padded


def draw(seed):
    r = random.Random(seed)
    width = r.choice([64, 72, 96, 100, 128, 160])
    layers = []
    for _ in range(r.randint(1, 4)):
        if r.random() < 0.5:
            dp, dvp = r.choice(PAIRS)
            G = r.choice([1, 2, 3])
            # (values at least 8 wide: the norm of a head's output over two or three values magnifies every rounding)
            mixer = M.attention(G * r.choice([1, 2, 3, 5]), G, r.randint(max(4, dp - 15), dp), r.randint(max(8, dvp - 31), dvp),
                                r.choice([1, 2, 5, 31, 32, 33, 64, 100, 129, 300]), diff=r.uniform(0.05, 0.8),
                                scale=r.uniform(0.05, 0.4))
        else:
            groups = r.choice([1, 1, 2, 3])
            heads, dv = groups * r.randint(1, 3), r.choice([4, 10, 16, 33, 64, 80])
            parts = r.choice([g for g in (1, 2, 3, 4, 5, 8) if (heads * dv) % g == 0])
            mixer = M.mamba(heads, dv, r.choice([1, 7, 16, 40, 64, 100, 140]), groups, r.randint(1, 6), parts)
        kind = r.random()
        if kind < 0.25:
            mlp = None
        elif kind < 0.5:
            mlp = M.dense(r.choice([24, 50, 128]))
        else:
            experts, identity = r.randint(1, 12), r.choice([0, 0, 1, 3])
            mlp = M.moe(experts, r.randint(1, min(4, experts + identity)), r.choice([8, 24, 40]), identity=identity,
                        scale=r.uniform(0.5, 2.5), shared=r.choice([None, 16, 40]))
        layers.append(M.layer(mixer, mlp))
    loop = None
    if r.random() < 0.6:
        lo = r.randint(0, len(layers) - 1)
        loop = (lo, r.randint(lo + 1, len(layers)), r.randint(1, 3))
    return M.config(width, r.randint(40, 300), layers, loop=loop, eps=r.choice([1e-6, 1e-5, 1e-3]), scale=r.uniform(0.5, 4.0))


@pytest.fixture(scope="module")
def lib():
    import llm_infer_amd
    return llm_infer_amd


def all_rows(n):
    return list(range(n))


@pytest.mark.parametrize("seed", range(10))
def test_a_random_configuration_in_every_schedule(lib, seed, tmp_path):
    cfg = draw(1000 + seed)
    g = torch.Generator().manual_seed(seed)
    n = 150
    toks = torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
    short = torch.randint(0, cfg["vocab"], (37,), generator=g).tolist()
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 3e-2)):
        W = M.random_weights(cfg, 7 + seed, fixed_choice=dtype == "bfloat16")
        folder = str(tmp_path / dtype)
        M.write_model(folder, cfg, W)
        ref = P.forward(cfg, M.widen(W), toks, torch.float64)
        ref_short = P.forward(cfg, M.widen(W), short, torch.float64)
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
            assert torch.equal(got_b, whole), cfg
            s = eng.alloc_slot()
            pieces, at = [], 0
            for k in (63, 2, 1, 34, n - 100):
                pieces.append(eng.step([s], [toks[at:at + k]], [all_rows(k)]).cpu())
                at += k
            eng.free_slot(s)
            assert torch.equal(torch.cat(pieces), whole), cfg
