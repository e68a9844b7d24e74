"""Manirax on the GPU against the plain implementation: every mechanism alone, whole prompts, prompts cut
into portions, decoding token by token, batches of unequal requests, slots and pages used again, keys far
away and at page borders, long decoding, and greedy generation through the library's entry point."""
import copy
import json
import os
import subprocess
import sys

import pytest
import torch

import manirax_models as M
import plain_manirax as P
import trace_util as TU

pytestmark = pytest.mark.gpu
DEV = "cuda"
# the measure is manirax_models.row_error: float32 runs agree with the float64 plain implementation to rounding;
# a bfloat16 run rounds every activation that enters a product (some ten roundings of 2^-9 a layer)
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
        folder = str(tmp_path_factory.mktemp("manirax_" + name))
        M.write_model(folder, cfg, W)
        out[name] = (folder, cfg, M.widen(W))
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def ctx_for(lens_before, toks):
    from llm_infer_amd.engine.step import StepContext
    return StepContext(DEV, list(range(len(toks))), toks, lens_before, [[] for _ in toks])


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
def test_layer_norm_and_the_residual_step(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    for d in (72, 320, 2050):
        x = torch.randn(9, d, generator=g) * 2 + 0.5
        y1, y2, w = torch.randn(9, d, generator=g), torch.randn(9, d, generator=g), 1 + 0.1 * torch.randn(d, generator=g)
        rows = torch.tensor([8, 0, 3], dtype=torch.int32)
        got = ops.layernorm(x.to(DEV), w.to(DEV), 1e-3, torch.float32, rows.to(DEV))
        assert (got.cpu().double() - P.layer_norm(x.double()[rows.long()], w.double(), 1e-3)).abs().max() < 1e-5
        for adds, ref_sum in (([(y1, 0.7)], 0.7 * y1.double()), ([(y1, 0.7), (y2, 1.3)], 0.7 * y1.double() + 1.3 * y2.double())):
            xd = x.to(DEV).clone()
            copy_ = ops.add_layernorm(xd, 1.9, [(y.to(DEV), s) for y, s in adds], w.to(DEV), 1e-3, torch.bfloat16)
            ref = P.layer_norm(1.9 * x.double() + ref_sum, w.double(), 1e-3)
            assert (xd.cpu().double() - ref).abs().max() < 1e-5
            assert torch.equal(copy_.cpu(), xd.cpu().to(torch.bfloat16))


def test_token_shift_carries_the_row_before_across_steps(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    d, slots = 50, 5
    mu = torch.rand(d, generator=g)
    seqs = {3: torch.randn(7, d, generator=g), 1: torch.randn(4, d, generator=g)}
    ref = {s: P.token_shift(x.double(), mu.double()) for s, x in seqs.items()}
    state = torch.full((slots, d), 9.0, device=DEV)        # what an earlier sequence left: not read at position 0
    # step one: 5 tokens of sequence 3 and 1 of sequence 1; step two: a single token each; step three: the rest
    cuts = {3: [(0, 5), (5, 6), (6, 7)], 1: [(0, 1), (1, 2), (2, 4)]}
    for step in range(3):
        rows = torch.cat([seqs[s][a:b] for s in (3, 1) for a, b in [cuts[s][step]]])
        pos = [p for s in (3, 1) for p in range(*cuts[s][step])]
        slot = [s for s in (3, 1) for _ in range(*cuts[s][step])]
        out = ops.token_shift(rows.to(DEV), mu.to(DEV), state, torch.tensor(pos, dtype=torch.int32, device=DEV),
                              torch.tensor(slot, dtype=torch.int32, device=DEV), torch.float32)
        want = torch.cat([ref[s][a:b] for s in (3, 1) for a, b in [cuts[s][step]]])
        assert (out.cpu().double() - want).abs().max() < 1e-6
    assert torch.equal(state[3].cpu(), seqs[3][-1]) and torch.equal(state[1].cpu(), seqs[1][-1])
    assert torch.equal(state[0].cpu(), torch.full((d,), 9.0))


def test_polynorm_and_gated_norm(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    for n in (100, 256, 3000):
        z = torch.randn(6, n, generator=g) * 1.5
        coef = torch.tensor([0.6, 0.3, -0.2, 0.1])
        got = ops.polynorm(z.to(DEV), coef.to(DEV), 1e-5, torch.float32)
        assert (got.cpu().double() - P.poly_norm(z.double(), coef.double(), 1e-5)).abs().max() < 1e-5
        rows = torch.randn(6, n + 37, generator=g)
        w = 1 + 0.1 * torch.randn(n, generator=g)
        got = ops.gated_rmsnorm(z.to(DEV), w.to(DEV), rows.to(DEV), 37, 1e-5, torch.float32)
        ref = P.unit_rms(z.double(), 1e-5) * w.double() * torch.sigmoid(rows.double()[:, 37:])
        assert (got.cpu().double() - ref).abs().max() < 1e-5


def _attention_part(lib, dt, H, G, d, dv, rot, base, factor, scale, eps, window=None):
    from llm_infer_amd.parts import NoPosition, RotaryPosition, SigmoidAttention
    pos = (RotaryPosition(theta=base, rotary_dim=rot, head_dim=d, pairing="half", scaling_factor=factor, dtype=dt, device=DEV)
           if rot else NoPosition(dtype=dt, device=DEV))
    return SigmoidAttention(hidden_size=64, n_heads=H, n_kv_heads=G, head_dim=d, v_head_dim=dv, scale=scale,
                            unit_norm_eps=eps, position=pos, prefix="a.", dtype=dt, device=DEV, window=window)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, d, dv, rot, factor", [(6, 2, 40, 24, 16, 2.0), (4, 4, 32, 48, 32, 1.0), (3, 1, 128, 128, 64, 4.0),
                                                       (2, 1, 16, 80, 0, 1.0)])
def test_sigmoid_attention_part_alone(lib, dtype, H, G, d, dv, rot, factor):
    """Ragged prompts in one step, then three tokens each one by one, against the plain mechanism; lengths that
    end on, before and behind a page's edge."""
    from llm_infer_amd.cache import Cache
    dt = DT[dtype]
    g = torch.Generator().manual_seed(H * 100 + d)
    part = _attention_part(lib, dt, H, G, d, dv, rot, 1000.0, factor, d ** -0.5, 1e-5)
    w = {"q_proj.weight": torch.randn(H * d, 64, generator=g) * 0.3, "k_proj.weight": torch.randn(G * d, 64, generator=g) * 0.3,
         "v_proj.weight": torch.randn(G * dv, 64, generator=g) * 0.2, "o_proj.weight": torch.randn(64, H * dv, generator=g) * 0.1,
         "head_bias": torch.randn(H, generator=g) - 1.0}
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    part.bind({k: v.to(DEV).to(dt if v.dim() == 2 else torch.float32) for k, v in w.items()})
    lens = [64, 131, 1, 63]
    hs = [torch.randn(n + 3, 64, generator=g).to(torch.bfloat16).float() for n in lens]
    cache = Cache([part.cache_spec()], 1024, 512, dt, DEV)
    slots = [cache.alloc_slot() for _ in lens]
    assert slots == list(range(len(lens)))

    def plain(h):
        h = h.double()
        T = h.shape[0]
        q = (h @ w["q_proj.weight"].double().t()).view(T, H, d)
        k = (h @ w["k_proj.weight"].double().t()).view(T, G, d)
        v = (h @ w["v_proj.weight"].double().t()).view(T, G, dv)
        if rot:
            q, k = (P.rotate_half_layout(t, torch.arange(T), 1000.0, rot, factor) for t in (q, k))
        o = P.sigmoid_attention(P.unit_rms(q, 1e-5), P.unit_rms(k, 1e-5), v, d ** -0.5, w["head_bias"].double())
        return o.reshape(T, H * dv) @ w["o_proj.weight"].double().t()

    ref = [plain(h) for h in hs]
    tol = 2e-5 if dtype == "float32" else 2e-2
    scale_of = max(r.abs().max().item() for r in ref)

    def run(lens_before, rows):
        cache.grow(slots, [b + r.shape[0] for b, r in zip(lens_before, rows)], filled=True)
        ctx = ctx_for(lens_before, [[0] * r.shape[0] for r in rows])
        (y, s), = part.addends(torch.cat(rows).to(DEV).to(dt), ctx, cache.view(0))
        assert s == 1.0 and y.dtype == torch.float32
        return y.cpu().double().split([r.shape[0] for r in rows])

    got = run([0] * len(lens), [h[:n] for h, n in zip(hs, lens)])
    for a, r, n in zip(got, ref, lens):
        assert (a - r[:n]).abs().max() < tol * scale_of
    for j in range(3):
        got = run([n + j for n in lens], [h[n + j:n + j + 1] for h, n in zip(hs, lens)])
        for a, r, n in zip(got, ref, lens):
            assert (a - r[n + j:n + j + 1]).abs().max() < tol * scale_of


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sigmoid_attention_finds_one_far_key(lib, dtype):
    """Weights made so that one key far back, on another page, carries the whole result: the bias shuts every
    other key out, the query equals that key."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.specs import KVSpec
    from llm_infer_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(7)
    H, G, d, dv, T = 2, 1, 32, 16, 700
    k = torch.randn(T, G, d, generator=g)
    v = torch.randn(T, G, dv, generator=g)
    q = torch.randn(T, H, d, generator=g)
    far = {699: 3, 500: 63, 641: 64, 130: 127, 65: 0, 64: 64}        # query position -> the key it must find
    for t, j in far.items():
        q[t] = k[j, 0] * 5.0
    bias = torch.full((H,), -0.8 * d)
    cache = Cache([KVSpec(G, d, None, dv)], 1024, 1024, dt, DEV)
    slot = cache.alloc_slot()
    cache.grow([slot], [T], filled=True)
    ctx = ctx_for([0], [[0] * T])
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).to(DEV)
    kv = cache.view(0).as_tuple()
    qd = ops.rope_norm_store(qkv, None, 0, False, 0.0, ctx.pos, ctx.tok_slot, kv, H, G, d, dv, d, d, dv, dt)
    out = ops.sigmoid_attention(qd, kv, ctx.pos, ctx.tok_slot, bias.to(DEV), H, G, d, dv, dv, 1.0)
    ref = P.sigmoid_attention(P.unit_rms(q.double(), 0.0), P.unit_rms(k.double(), 0.0), v.double(), 1.0, bias.double())
    for t, j in far.items():
        assert (ref[t, 0] - v[j, 0].double()).abs().max() < 0.05          # the test's own premise
        assert (out[t].cpu().double() - ref[t]).abs().max() < (1e-4 if dtype == "float32" else 3e-2)
    assert (out.cpu().double() - ref).abs().max() < (1e-4 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, d, dv, decay", [(3, 24, 40, (0.5, 0.9, 0.99)), (1, 16, 16, (1.0,)), (2, 128, 128, (0.999, 0.9)),
                                              (4, 48, 32, (0.55, 0.8, 0.93, 0.995)), (2, 8, 200, (0.3, 0.95))])
def test_decay_attention_part_alone(lib, dtype, H, d, dv, decay):
    """A prompt in one step, in portions (down to two tokens and one), and two sequences side by side, against
    the plain recurrence; the state of a slot that is used again starts at zero."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.parts import DecayLinearAttention
    dt = DT[dtype]
    g = torch.Generator().manual_seed(H * 10 + d)
    part = DecayLinearAttention(hidden_size=48, n_heads=H, head_dim=d, v_head_dim=dv, decay=decay, norm_eps=1e-5,
                                prefix="r.", dtype=dt, device=DEV)
    shapes = {k: s.shape for k, s in part.params().items()}
    w = {k: (torch.randn(*s, generator=g) * (0.3 if len(s) == 2 else 0.1) + (1.0 if len(s) == 1 else 0.0)).to(torch.bfloat16).float()
         for k, s in shapes.items()}
    part.bind({k: v.to(DEV).to(dt if v.dim() == 2 else torch.float32) for k, v in w.items()})
    hs = [torch.randn(n, 48, generator=g).to(torch.bfloat16).float() for n in (150, 37)]

    def plain(h):
        h = h.double()
        T = h.shape[0]
        q, k, v = (P.silu(h @ w[n + "_proj.weight"].double().t()).view(T, H, s) for n, s in (("q", d), ("k", d), ("v", dv)))
        o = P.decayed_linear_attention(q, k, v, torch.tensor(decay, dtype=torch.float64)).reshape(T, H * dv)
        o = P.unit_rms(o, 1e-5) * w["norm.weight"].double() * torch.sigmoid(h @ w["g_proj.weight"].double().t())
        return o @ w["o_proj.weight"].double().t()

    ref = [plain(h) for h in hs]
    tol = (3e-5 if dtype == "float32" else 2e-2) * max(r.abs().max().item() for r in ref)
    cache = Cache([part.cache_spec()], 1024, 512, dt, DEV)

    def run(slots, lens_before, rows):
        ctx = ctx_for(lens_before, [[0] * r.shape[0] for r in rows])
        ctx.seq_slot = torch.tensor(slots, dtype=torch.int32, device=DEV)
        (y, s), = part.addends(torch.cat(rows).to(DEV).to(dt), ctx, cache.view(0))
        return y.cpu().double().split([r.shape[0] for r in rows])

    a, b = cache.alloc_slot(), cache.alloc_slot()
    whole = run([a, b], [0, 0], hs)
    for got, r in zip(whole, ref):
        assert (got - r).abs().max() < tol
    cache.free_slot(a)
    cache.free_slot(b)
    # the same two slots again (their states are cleared when handed out), the long one in portions
    b2, a2 = cache.alloc_slot(), cache.alloc_slot()
    assert {a2, b2} == {a, b}
    at, pieces = 0, []
    for n in (2, 64, 1, 30, 2, 51):
        rows = [hs[0][at:at + n]] + ([hs[1]] if at == 0 else [])
        got = run([a2, b2][:len(rows)], [at, 0][:len(rows)], rows)
        pieces.append(got[0])
        if at == 0:
            assert torch.equal(got[1], whole[1]) if dtype == "float32" else (got[1] - ref[1]).abs().max() < tol
        at += n
    cut = torch.cat(pieces)
    assert (cut - ref[0]).abs().max() < tol
    if dtype == "float32":
        assert torch.equal(cut, whole[0])          # the recurrence does the same arithmetic however it is cut


# ---------------------------------------------------------------------------
# the whole model through the engine
# ---------------------------------------------------------------------------
def engine_for(lib, models, name, dtype, max_tokens=2048):
    folder, cfg, W = models[name]
    return lib.load(folder, dtype=dtype, max_tokens=max_tokens), cfg, W


def all_rows(n):
    return list(range(n))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_whole_prompts_portions_and_decoding(lib, models, name, dtype):
    eng, cfg, W = engine_for(lib, models, name, dtype)
    assert eng.max_positions == 2048           # the design sets no bound: the cache's
    n = 150
    toks = tokens(cfg, n, 3)
    ref = P.forward(W, cfg, toks)
    s = eng.alloc_slot()
    whole = eng.step([s], [toks], [all_rows(n)]).cpu()
    assert M.row_error(whole, ref) < TOL[dtype]
    eng.free_slot(s)
    # the first tokens alone
    for m in (1, 2, 3):
        s = eng.alloc_slot()
        got = eng.step([s], [toks[:m]], [all_rows(m)]).cpu()
        assert M.row_error(got, ref[:m]) < TOL[dtype]
        eng.free_slot(s)
    # portions of several sizes, down to two tokens and one, across a page's edge
    s = eng.alloc_slot()
    at, pieces = 0, []
    for m in (2, 61, 2, 1, 64, 3, 17):
        pieces.append(eng.step([s], [toks[at:at + m]], [all_rows(m)]).cpu())
        at += m
    assert at == n
    cut = torch.cat(pieces)
    assert M.row_error(cut, ref) < TOL[dtype]
    if dtype == "float32":
        assert torch.equal(cut, whole)
    eng.free_slot(s)
    # a prompt, then token by token
    s = eng.alloc_slot()
    head = 70
    pieces = [eng.step([s], [toks[:head]], [all_rows(head)]).cpu()]
    pieces += [eng.step([s], [[t]], [[0]]).cpu() for t in toks[head:]]
    dec = torch.cat(pieces)
    assert M.row_error(dec, ref) < TOL[dtype]
    if dtype == "float32":
        assert torch.equal(dec, whole)
    eng.free_slot(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(lib, models, dtype):
    eng, cfg, W = engine_for(lib, models, "P", dtype)
    lens = [1, 130, 64, 7, 65]
    reqs = [tokens(cfg, n + 6, 10 + i) for i, n in enumerate(lens)]
    refs = [P.forward(W, cfg, r) for r in reqs]
    alone = []
    for r, n in zip(reqs, lens):
        s = eng.alloc_slot()
        rows = [eng.step([s], [r[:n]], [all_rows(n)]).cpu()] + [eng.step([s], [[t]], [[0]]).cpu() for t in r[n:]]
        alone.append(torch.cat(rows))
        eng.free_slot(s)
    for a, ref in zip(alone, refs):
        assert M.row_error(a, ref) < TOL[dtype]
    # together, in slots and pages that the runs before have used; the shorter requests end earlier
    for round_ in range(2):
        slots = [eng.alloc_slot() for _ in reqs]
        out = eng.step(slots, [r[:n] for r, n in zip(reqs, lens)], [all_rows(n) for n in lens]).cpu()
        got = list(out.split(lens))
        live = list(range(len(reqs)))
        for j in range(6):
            if j == 3:
                for i in (0, 2):
                    eng.free_slot(slots[i])
                    live.remove(i)
            out = eng.step([slots[i] for i in live], [[reqs[i][lens[i] + j]] for i in live], [[0] for _ in live]).cpu()
            for row, i in zip(out, live):
                got[i] = torch.cat([got[i], row[None]])
        for i in live:
            eng.free_slot(slots[i])
        for i, (a, g_) in enumerate(zip(alone, got)):
            if dtype == "float32":
                assert torch.equal(g_, a[:g_.shape[0]])
            assert M.row_error(g_, refs[i][:g_.shape[0]]) < TOL[dtype]


def test_a_far_token_decides_and_long_decoding(lib, models):
    """Long decoding in float32 (300 tokens one by one over five pages) against the whole prompt and the plain
    implementation; and the state that only the linear attention carries: with decay 1 in TINY_Q's first layer
    the first token still moves the last logits."""
    eng, cfg, W = engine_for(lib, models, "Q", "float32")
    n = 330
    toks = tokens(cfg, n, 21)
    ref = P.forward(W, cfg, toks)
    s = eng.alloc_slot()
    rows = [eng.step([s], [toks[:30]], [all_rows(30)]).cpu()] + [eng.step([s], [[t]], [[0]]).cpu() for t in toks[30:]]
    eng.free_slot(s)
    dec = torch.cat(rows)
    assert M.row_error(dec, ref) < TOL["float32"]
    other = list(toks)
    other[0] = (toks[0] + 1) % cfg["vocab"]
    moved = (P.forward(W, cfg, other)[-1] - ref[-1]).abs().max().item()
    assert moved > 100 * (dec[-1].double() - ref[-1]).abs().max().item()
    s = eng.alloc_slot()
    got = eng.step([s], [other], [[n - 1]]).cpu()
    eng.free_slot(s)
    assert (got[0].double() - P.forward(W, cfg, other)[-1]).abs().max() < moved / 50


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(lib, models, dtype):
    """engine.generate (planner, batches, recorded decode steps) against the plain implementation's own choice,
    as long as its margin leaves no doubt; recorded and eager steps give the same tokens."""
    eng, cfg, W = engine_for(lib, models, "P", dtype)
    prompts = [tokens(cfg, n, 30 + n) for n in (5, 66, 1, 20)]
    n_new = 24
    got = eng.generate(prompts, max_new_tokens=n_new, temperature=0.0)
    eager = eng.generate(prompts, max_new_tokens=n_new, temperature=0.0, use_graph=False)
    assert eng.decode_counts["replayed"] > 0
    checked = 0
    for p, new, e in zip(prompts, got, eager):
        assert len(new) == n_new
        toks = list(p)
        for t, te in zip(new, e):
            last = P.forward(W, cfg, toks)[-1]
            top2 = torch.topk(last, 2).values
            if (top2[0] - top2[1]).item() <= 4 * TOL[dtype] * last.std().item():
                break
            assert t == te == int(last.argmax())
            toks.append(t)
            checked += 1
    assert checked > n_new * len(prompts) // 2
    # sampling with a temperature runs through the same path
    hot = eng.generate(prompts, max_new_tokens=8, temperature=0.8, seed=3)
    assert hot == eng.generate(prompts, max_new_tokens=8, temperature=0.8, seed=3) and all(len(h) == 8 for h in hot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_in_three_schedules(lib, models, dtype, tmp_path):
    folder, cfg, W = models["P"]
    reqs = {"a": tokens(cfg, 140, 1), "b": tokens(cfg, 3, 2), "c": tokens(cfg, 70, 3), "d": tokens(cfg, 1, 4)}
    refs = {r: P.forward(W, cfg, t) for r, t in reqs.items()}
    for k, (steps, where) in enumerate((TU.steps_whole(reqs), TU.steps_tail(reqs, tail=12),
                                        TU.steps_batches(reqs, 3, {"a": 9, "b": 2, "c": 9}))):
        out = TU.run_trace(folder, dtype, steps, where, cfg["vocab"], 512, str(tmp_path / f"{dtype}{k}"))
        for (r, p), row in out.items():
            assert M.row_error(torch.from_numpy(row)[None], refs[r][p:p + 1]) < TOL[dtype], (k, r, p)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sigmoid_attention_window_edges(lib, dtype):
    """The mixer's optional window (the design itself has none): a key exactly at the window's edge counts, the
    one before it does not, in a prompt, in a portion that continues it and in decoding, with the keys that
    decide made to stand out."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.specs import KVSpec
    from llm_infer_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(9)
    H, G, d, dv, T, W = 2, 1, 32, 32, 200, 70
    k, v, q = torch.randn(T, G, d, generator=g), torch.randn(T, G, dv, generator=g), torch.randn(T, H, d, generator=g)
    for t in (100, 150, 199, 69, 70):            # queries that look at the key just inside and just outside
        q[t, 0] = k[max(0, t - W + 1), 0] * 5.0
        q[t, 1] = k[max(0, t - W), 0] * 5.0
    bias = torch.full((H,), -0.8 * d)
    ref = P.sigmoid_attention(P.unit_rms(q.double(), 0.0), P.unit_rms(k.double(), 0.0), v.double(), 1.0, bias.double(), window=W)
    assert (ref[150, 0] - v[81, 0].double()).abs().max() < 0.05 and ref[150, 1].abs().max() < 0.05
    cache = Cache([KVSpec(G, d, W, dv)], 1024, 1024, dt, DEV)
    slot = cache.alloc_slot()
    got, at = [], 0
    for n in [130, 40] + [1] * 30:               # a prompt, a portion, then token by token
        cache.grow([slot], [at + n], filled=True)
        ctx = ctx_for([at], [[0] * n])
        rows = slice(at, at + n)
        qkv = torch.cat([q[rows].reshape(n, -1), k[rows].reshape(n, -1), v[rows].reshape(n, -1)], 1).to(DEV)
        kv = cache.view(0).as_tuple()
        qd = ops.rope_norm_store(qkv, None, 0, False, 0.0, ctx.pos, ctx.tok_slot, kv, H, G, d, dv, d, d, dv, dt)
        if dtype == "float32":
            out = ops.sigmoid_attention(qd, kv, ctx.pos, ctx.tok_slot, bias.to(DEV), H, G, d, dv, dv, 1.0, W)
        elif ctx.is_decode:
            out = ops.sigmoid_attention_decode(qd, kv, ctx.seq_slot, ctx.seq_ctx, 1, bias.to(DEV), H, G, d, dv, dv, 1.0, W, 2)
        else:
            out = ops.sigmoid_attention_prefill(qd, kv, ops.prefill_meta(ctx), bias.to(DEV), H, G, d, dv, dv, 1.0, W)
        got.append(out.cpu().double())
        at += n
        cache.trim_windows([slot])
    assert at == T
    assert (torch.cat(got) - ref).abs().max() < (1e-4 if dtype == "float32" else 3e-2)


def test_float16_runs_the_same_kernels(lib, models):
    folder, cfg, W = models["Q"]
    eng = lib.load(folder, dtype="float16", max_tokens=1024)
    toks = tokens(cfg, 100, 8)
    ref = P.forward(W, cfg, toks)
    s = eng.alloc_slot()
    rows = [eng.step([s], [toks[:90]], [all_rows(90)]).cpu()] + [eng.step([s], [[t]], [[0]]).cpu() for t in toks[90:]]
    assert M.row_error(torch.cat(rows), ref) < 1e-2


def test_command_line_and_model_info(lib, models):
    folder, cfg, W = models["P"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompts = [tokens(cfg, 9, 51), tokens(cfg, 2, 52)]
    cmd = [sys.executable, os.path.join(root, "bin", "infer"), folder, "-n", "6", "-t", "0", "--dtype", "float32", "-T", "64"]
    for p in prompts:
        cmd += ["--tokens", ",".join(map(str, p))]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = [json.loads(line.split("tokens: ", 1)[1]) for line in res.stdout.splitlines() if " tokens: [" in line]
    for p, new in zip(prompts, got):
        toks = list(p)
        for t in new:
            assert t == int(P.forward(W, cfg, toks)[-1].argmax())
            toks.append(t)
    for word in ("Layers: 2", "Dimensions: 72", "Heads: 2..6 sigmoid + 2..3 linear", "Vocab size: 131", "Max seq len: 64"):
        assert word in res.stdout, res.stdout
    info = subprocess.run([sys.executable, os.path.join(root, "bin", "model_info"), folder], capture_output=True, text=True,
                          timeout=300)
    assert info.returncode == 0 and "Architecture: Manirax" in info.stdout and "The tensors fit the model." in info.stdout
