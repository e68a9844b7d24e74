"""Manirax configurations drawn at random (seeded) from the sizes the design allows, each run whole, in portions and
token by token in float32 and bfloat16 against the plain implementation: widths that are no multiple of 32 (matrices
that cannot be tiled), head sizes that are no multiple of 16, key and value sizes that differ, 1 to 9 query heads on a
key head, rotated parts from nothing to the whole head, layers with and without feed-forward."""
import random

import pytest
import torch

import manirax_models as M
import plain_manirax as P

pytestmark = pytest.mark.gpu
TOL = {"float32": 1e-4, "bfloat16": 3e-2}


def draw(seed):
    r = random.Random(seed)
    width = r.choice([40, 72, 96, 136, 200, 264, 320 + 8 * r.randrange(8)])
    layers = []
    for _ in range(r.randint(1, 4)):
        group = r.choice([1, 1, 2, 3, 4, 9])
        kv = r.randint(1, 3)
        dim = 2 * r.randint(4, 70)
        vdim = r.choice([dim, r.randint(3, 140)])
        rot = None
        if r.random() < 0.8:
            rot = {"base": r.choice([100.0, 1e4, 5e5]), "dims": 2 * r.randint(1, dim // 2)}
            if r.random() < 0.6:
                rot["scaling"] = {"factor": r.choice([1.0, 2.0, 4.0, 7.5])}
        heads_r = r.randint(1, 5)
        layers.append(M.layer(
            M.left(group * kv, kv, dim, vdim, scale=r.choice([None, 0.05, 0.2]), rot=rot),
            M.right(heads_r, r.randint(2, 100), r.randint(2, 100), [r.choice([1.0, 0.999, 0.9, 0.5, 0.1]) for _ in range(heads_r)]),
            r.choice([1.0, 0.3, 1.6]), r.choice([1.0, 0.6, 2.2]), r.choice([None, r.randint(8, 400)])))
    return M.config(width, r.randint(50, 700), layers, eps=r.choice([1e-5, 1e-6, 1e-3]), alpha=r.choice([1.0, 0.5, 2.0, 3.3]))


@pytest.mark.parametrize("seed", range(10))
def test_random_configuration(seed, tmp_path):
    import llm_infer_amd
    cfg = draw(1000 + seed)
    W = M.random_weights(cfg, seed, sharp=1.5)
    folder = str(tmp_path / "m")
    M.write_model(folder, cfg, W)
    W64 = M.widen(W)
    g = torch.Generator().manual_seed(seed)
    lens = [97, 1, 34]
    reqs = [torch.randint(0, cfg["vocab"], (n + 4,), generator=g).tolist() for n in lens]
    refs = [P.forward(W64, cfg, r) for r in reqs]
    for dtype in ("float32", "bfloat16"):
        eng = llm_infer_amd.load(folder, dtype=dtype, max_tokens=1024)
        slots = [eng.alloc_slot() for _ in reqs]
        # the first request in two portions beside the others whole, then four tokens each one by one
        first = eng.step([slots[0]], [reqs[0][:33]], [list(range(33))]).cpu()
        out = eng.step(slots, [reqs[0][33:lens[0]], reqs[1][:lens[1]], reqs[2][:lens[2]]],
                       [list(range(lens[0] - 33)), list(range(lens[1])), list(range(lens[2]))]).cpu()
        got = list(out.split([lens[0] - 33, lens[1], lens[2]]))
        got[0] = torch.cat([first, got[0]])
        for j in range(4):
            out = eng.step(slots, [[r[n + j]] for r, n in zip(reqs, lens)], [[0]] * 3).cpu()
            got = [torch.cat([a, row[None]]) for a, row in zip(got, out)]
        for a, ref in zip(got, refs):
            assert M.row_error(a, ref) < TOL[dtype], (seed, dtype, cfg)
