"""Risonex on the GPU against the plain implementation: every mechanism alone, whole prompts, prompts cut
into portions, decoding token by token, batches of unequal requests, slots and pages used again, keys far
away, at page borders and at the edges of a block, long decoding, and greedy generation through the library's
entry point.

Routing: a float32 run follows the plain implementation's choices to rounding.  A bfloat16 run rounds the router's
input, so a token whose choice scores nearly tie could go either way; the bfloat16 models therefore get corrections
that lie far apart (the same outputs win for every token, with weights that still follow the token), and the choice
itself is tested alone, on scores with clear margins."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_risonex as P
import risonex_models as M
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
        for fixed in (False, True):
            W = M.random_weights(cfg, 60 + ord(name), sharp=2.0, fixed_choice=fixed)
            folder = str(tmp_path_factory.mktemp(f"risonex_{name}_{int(fixed)}"))
            M.write_model(folder, cfg, W)
            out[name, fixed] = (folder, cfg, M.widen(W))
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def step_context(slots, lens_before, counts):
    from llm_infer_amd.engine.step import StepContext
    return StepContext(DEV, list(slots), [[0] * n for n in counts], list(lens_before), [[] for _ in counts])


def error(got, ref):
    """Largest difference relative to the reference's spread."""
    return ((got.double() - ref.double()).abs().max() / ref.double().std()).item()


def build_part(table, spec, weights, dtype):
    """A part as the configuration describes it, with the given tensors (by local name) bound."""
    import llm_infer_amd.parts  # noqa: F401  (registers the parts)
    from llm_infer_amd.registry import lookup
    from llm_infer_amd.weights.loader import place_tensor
    extra = {"position": None} if table == "mixer" else {}
    part = lookup(table, spec.kind)(**spec.params, prefix=spec.prefix, dtype=DT[dtype], device=DEV, **extra)
    wanted = part.params()
    assert set(wanted) == set(weights), set(wanted) ^ set(weights)
    part.bind({n: place_tensor(weights[n], wanted[n].kind, DT[dtype], DEV) for n in wanted})
    return part


def one_layer(mixer, mlp=None, width=96, eps=1e-5):
    from llm_infer_amd.registry import config_from_dict
    return config_from_dict(M.config(width, 50, [M.layer(mixer, mlp)], eps=eps))


def run_mixer(part, h_of, schedule, dtype, cache=None):
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
        ctx = step_context([slot[r] for r in rs], [at[r] for r in rs], [step[r] for r in rs])
        h = torch.cat([h_of[r][at[r]:at[r] + step[r]] for r in rs]).to(DEV).to(DT[dtype])
        res = torch.zeros((h.shape[0], h_of[rs[0]].shape[1]), dtype=torch.float32, device=DEV)
        part.forward(h, ctx, views, res)
        for r, rows in zip(rs, res.cpu().split([step[r] for r in rs])):
            out[r].append(rows)
            at[r] += step[r]
        cache.trim_windows([slot[r] for r in rs])
        for r in rs:
            if at[r] == h_of[r].shape[0]:
                cache.free_slot(slot.pop(r))
    return {r: torch.cat(v) for r, v in out.items()}, cache


SCHEDULES = {
    "whole": lambda n: [{"a": n["a"]}, {"b": n["b"]}, {"c": n["c"]}],
    # portions down to two tokens and one, across the edges of pages and blocks
    "portions": lambda n: [{"a": 61}, {"a": 2}, {"a": 1}, {"a": 3}, {"a": n["a"] - 67}] + [{"b": 2}] * (n["b"] // 2)
                          + [{"b": n["b"] % 2}] * (n["b"] % 2) + [{"c": n["c"]}],
    # unequal requests together, then decoded together; the shortest ends first, and c comes into a slot used before
    "together": lambda n: [{"a": n["a"] - 9, "b": n["b"] - 4}] + [{"a": 1, "b": 1}] * 4 + [{"a": 1}] * 5 + [{"c": n["c"] - 3}]
                          + [{"c": 1}] * 3,
}


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
def test_embedding_scale_and_sinusoidal_positions(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(0)
    for width in (64, 75):
        table = torch.randn(40, width, generator=g)
        toks = torch.randint(0, 40, (6,), generator=g)
        pos = torch.tensor([0, 1, 63, 64, 1000, 7001])
        two_i = torch.arange(0, width, 2, dtype=torch.float64)
        freq = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -two_i / width).float()
        got = ops.embed_positions(table.to(DEV), toks.int().to(DEV), pos.int().to(DEV), freq.to(DEV), 2.5).cpu()
        ref = table[toks].double() * 2.5 + P.sinusoid(pos.tolist(), width, torch.float64)
        # float32 angles: at position 7,001 the angle itself is rounded to 5e-4
        assert (got.double() - ref).abs().max() < 2e-3 and (got[:4].double() - ref[:4]).abs().max() < 1e-5
        plain32 = table[toks] * 2.5 + P.sinusoid(pos.tolist(), width, torch.float32)
        assert (got - plain32).abs().max() < 1e-3


def test_norm_with_a_weight_stored_around_zero(lib):
    from llm_infer_amd.parts.norm import RMSNorm
    g = torch.Generator().manual_seed(1)
    x, w = torch.randn(7, 200, generator=g) * 3, 0.2 * torch.randn(200, generator=g)
    norm = RMSNorm(size=200, eps=1e-3, name="n", one_plus=True, prefix="", dtype=torch.float32, device=DEV)
    norm.bind({"n": w.to(DEV)})
    ref = P.norm_one_plus(x.double(), w.double(), 1e-3)
    assert (norm.forward(x.to(DEV)).cpu().double() - ref).abs().max() < 1e-5
    assert (ref - P.rms_div(x.double(), 1e-3)).abs().max() > 0.1          # the weight is not taken as it is stored


def test_activations_and_the_gated_norm_in_groups(lib):
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    z = torch.randn(5, 300, generator=g) * 3
    assert (ops.activation(z.to(DEV), "gelu", torch.float32).cpu().double() - P.gelu_erf(z.double())).abs().max() < 1e-5
    assert (ops.activation(z.to(DEV), "silu", torch.float32).cpu().double() - P.silu(z.double())).abs().max() < 1e-5
    tanh_form = 0.5 * z.double() * (1 + torch.tanh(0.7978845608028654 * (z.double() + 0.044715 * z.double() ** 3)))
    assert (ops.activation(z.to(DEV), "gelu_tanh", torch.float32).cpu().double() - tanh_form).abs().max() < 1e-5
    assert (P.gelu_erf(z.double()) - tanh_form).abs().max() > 1e-4
    for n, groups in ((96, 1), (96, 4), (520, 5)):
        y, rows, w = torch.randn(6, n, generator=g), torch.randn(6, n + 30, generator=g), 1 + 0.2 * torch.randn(n, generator=g)
        got = ops.gated_group_norm(y.to(DEV), rows.to(DEV), 20, w.to(DEV), groups, 1e-4, torch.float32).cpu().double()
        gated = y.double() * P.silu(rows[:, 20:20 + n].double())
        ref = P.rms_div(gated.view(6, groups, n // groups), 1e-4).reshape(6, n) * w.double()
        assert (got - ref).abs().max() < 1e-5
        if groups > 1:       # the gate comes before the norm, and every part has its own root mean square
            assert (ref - P.rms_div(gated, 1e-4) * w.double()).abs().max() > 1e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, d, dv, block", [(6, 2, 20, 36, 50), (2, 2, 64, 16, 7), (3, 1, 8, 130, 200), (4, 1, 128, 128, 64),
                                                (2, 1, 16, 16, 1)])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
def test_differential_attention_part(lib, dtype, H, G, d, dv, block, schedule):
    width, eps = 96, 1e-5
    mixer = M.attention(H, G, d, dv, block, diff=0.3)
    cfg = one_layer(mixer, width=width, eps=eps)
    g = torch.Generator().manual_seed(H * 100 + d)
    W = M.mixer_weights("attention", mixer[1], width, g, torch.bfloat16, sharp=2.0)
    part = build_part("mixer", cfg._mixer("", cfg.layers[0]), W, dtype)
    n = {"a": 140, "b": 9, "c": 70}
    h_of = {r: torch.randn(k, width, generator=g).to(DT[dtype]).float() for r, k in n.items()}
    got, cache = run_mixer(part, h_of, SCHEDULES[schedule](n), dtype)
    for r in n:
        ref = P.diff_attention(h_of[r].double(), M.widen(W), mixer[1], eps)
        tol = TOL[dtype]
        if dtype == "bfloat16":      # not below three times what the rounding of q, k, v and the output alone does
            tol = max(tol, 3 * error(P.diff_attention(h_of[r].double(), M.widen(W), mixer[1], eps, store=torch.bfloat16), ref))
        assert error(got[r], ref) < tol, r
    assert all(g_.pool.n_free == g_.n_pages - 1 for g_ in cache.groups)         # every page came back


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_sees_its_block_and_nothing_before_it(lib, dtype):
    """Keys made to stand out: the first map of a query looks for the first key of its own block (just inside),
    the second map for the key before it (just outside, which it must not find); and one far key at the block's
    start decides a query at its end.  In a prompt that crosses pages, in a portion and in decoding."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.specs import KVSpec
    from llm_infer_amd.kernels import ops
    dt = DT[dtype]
    g = torch.Generator().manual_seed(9)
    H, G, d, dv, T, B = 2, 1, 32, 48, 420, 150
    q, k, v = torch.randn(T, H, 2, d, generator=g), torch.randn(T, G, 2, d, generator=g), torch.randn(T, G, dv, generator=g)
    probes = (149, 150, 151, 299, 300, 310, 419)
    for t in probes:
        lo = t - t % B
        q[t, :, 0] = k[lo, 0, 0] * 4.0
        q[t, :, 1] = k[max(lo - 1, 0), 0, 1] * 4.0
    if dtype == "bfloat16":                      # what the cache and the kernel's q hold
        q, k, v = q.bfloat16().float(), k.bfloat16().float(), v.bfloat16().float()
    lam, scale = 0.6, 1.0
    ref = P.diff_attention_core(q.double(), k.double(), v.double(), scale, lam, B, 1e-6, 0.7)
    # the same tokens one position later (a token put in front): every block then begins one token earlier, which is
    # what an edge that is one token off looks like, and the probes must tell
    pad = lambda x: torch.cat([torch.zeros_like(x[:1]), x]).double()
    shifted = P.diff_attention_core(pad(q), pad(k), pad(v), scale, lam, B, 1e-6, 0.7)[1:]
    assert all((ref[t] - shifted[t]).abs().max() > 0.3 for t in probes)
    cache = Cache([KVSpec(G, 2 * d, None, dv, B, "maps")], 2048, 2048, dt, DEV)
    slot = cache.alloc_slot()
    got, at = [], 0
    for n in [200, 97, 2] + [1] * 121:
        cache.grow([slot], [at + n], filled=True)
        ctx = step_context([slot], [at], [n])
        rows = slice(at, at + n)
        qkv = torch.cat([q[rows].reshape(n, -1), k[rows].reshape(n, -1), v[rows].reshape(n, -1)], 1).to(DEV)
        kv = cache.view(0).as_tuple()
        qd = ops.qk_norm_store(qkv, 0, None, None, None, ctx.pos, ctx.tok_slot, kv, H, G, 2, d, dv)
        out = ops.diff_attention(qd, kv, ctx.pos, ctx.tok_slot, H, G, 2, d, dv, scale, B, None, lam, 1e-6, 0.7, dt,
                                 ops.diff_tiles(ctx, B) if dtype != "float32" else None)
        got.append(out.cpu().double().view(n, H, dv))
        at += n
        cache.trim_windows([slot])
        # the pages of the blocks behind the newest token have been given back
        assert min(cache.groups[0].pages_of[slot]) == (at - at % B) // 64
    assert at == T
    assert (torch.cat(got) - ref).abs().max() < (1e-4 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("P_, dv, N, G, taps, parts", [(4, 24, 20, 1, 3, 1), (6, 16, 33, 3, 5, 4), (2, 80, 130, 2, 2, 2),
                                                       (8, 64, 128, 1, 4, 8), (1, 8, 4, 1, 1, 1)])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
def test_state_space_part(lib, dtype, P_, dv, N, G, taps, parts, schedule):
    width, eps = 96, 1e-5
    mixer = M.mamba(P_, dv, N, G, taps, parts)
    cfg = one_layer(mixer, width=width, eps=eps)
    g = torch.Generator().manual_seed(P_ * 10 + N)
    W = M.mixer_weights("mamba2", mixer[1], width, g, torch.bfloat16)
    part = build_part("mixer", cfg._mixer("", cfg.layers[0]), W, dtype)
    n = {"a": 140, "b": 9, "c": 70}
    h_of = {r: torch.randn(k, width, generator=g).to(DT[dtype]).float() for r, k in n.items()}
    got, _ = run_mixer(part, h_of, SCHEDULES[schedule](n), dtype)
    for r in n:
        ref = P.mamba2(h_of[r].double(), M.widen(W), mixer[1], eps)
        assert error(got[r], ref) < TOL[dtype], r


def test_state_space_carries_the_first_token_far(lib):
    """A head whose decay is nearly one: the first token still moves what the mixer adds 700 tokens later, by far
    more than the engine differs from the plain implementation; cut into a prompt, portions and decoding."""
    width, eps = 64, 1e-5
    mixer = M.mamba(2, 16, 24, 1, 4, 1)
    cfg = one_layer(mixer, width=width, eps=eps)
    g = torch.Generator().manual_seed(5)
    W = M.mixer_weights("mamba2", mixer[1], width, g, torch.float32)
    W["dt_bias"] = torch.tensor([-7.0, -6.0])
    W["A_log"] = torch.tensor([-1.0, 0.0])
    part = build_part("mixer", cfg._mixer("", cfg.layers[0]), W, "float32")
    n = 700
    h = torch.randn(n, width, generator=g) * 0.3
    h[0] *= 20.0
    got, _ = run_mixer(part, {"a": h}, [{"a": 300}, {"a": 2}, {"a": 333}] + [{"a": 1}] * 65, "float32")
    ref = P.mamba2(h.double(), M.widen(W), mixer[1], eps)
    other = h.clone()
    other[0] = -other[0]
    moved = (P.mamba2(other.double(), M.widen(W), mixer[1], eps)[-1] - ref[-1]).abs().max().item()
    assert error(got["a"], ref) < 1e-4
    assert moved > 300 * (got["a"][-1].double() - ref[-1]).abs().max().item()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_real, n_identity, top", [(5, 1, 3), (3, 0, 1), (66, 4, 4), (2, 2, 4)])
def test_router_choice_weights_and_identity(lib, dtype, n_real, n_identity, top):
    """Scores with clear margins: the choice follows score + correction, the weights the scores alone, divided by
    the chosen scores' sum and multiplied by the scale; identity outputs add weight * h to the residual rows;
    the column behind the router's is the shared expert's gate."""
    from llm_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(n_real)
    T, width, n_out = 40, 48, n_real + n_identity
    # logits on a grid of 0.5 with all values of a row different, corrections on a grid of 0.05 x their rank: no ties
    logits = torch.stack([torch.randperm(n_out, generator=g).float() * (3.0 / n_out) for _ in range(T)])
    correction = torch.randperm(n_out, generator=g).float() * 0.21
    gate = torch.randn(T, 1, generator=g)
    h = torch.randn(T, width, generator=g).to(DT[dtype])
    res0 = torch.randn(T, width, generator=g)
    res = res0.clone().to(DEV)
    w = ops.moe_route(torch.cat([logits, gate], 1).to(DEV), correction.to(DEV), h.to(DEV), res, n_out, n_real, top, 1, 1.7).cpu()
    s = torch.softmax(logits.double(), -1)
    chosen = torch.topk(s + correction.double(), top, dim=-1).indices
    ref = torch.zeros(T, n_out, dtype=torch.float64)
    picked = torch.gather(s, 1, chosen)
    ref.scatter_(1, chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20) * 1.7)
    assert (w[:, :n_real].double() - ref[:, :n_real]).abs().max() < 1e-5
    assert (w[:, n_real].double() - torch.sigmoid(gate[:, 0].double())).abs().max() < 1e-6
    passed = ref[:, n_real:].sum(-1, keepdim=True) * h.double()
    assert (res.cpu().double() - (res0.double() + passed)).abs().max() < 1e-5
    if n_identity and top < n_out:
        without = torch.topk(s, top, dim=-1).indices                      # the correction decides, and only the choice
        assert not torch.equal(chosen.sort(-1).values, without.sort(-1).values)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mlp", [M.moe(5, 3, 40, identity=1, scale=2.0, shared=24), M.moe(3, 1, 56), M.moe(66, 4, 8, identity=4, shared=16),
                                 M.dense(72)])
def test_feed_forward_parts(lib, dtype, mlp):
    width = 96
    cfg = one_layer(M.mamba(2, 8, 8), mlp, width=width)
    g = torch.Generator().manual_seed(11)
    W = M.mlp_weights(mlp, width, g, torch.bfloat16, fixed_choice=dtype == "bfloat16")
    part = build_part("feed_forward", cfg._feed_forward("", mlp), W, dtype)
    for T in (1, 5, 150):
        h = torch.randn(T, width, generator=g).to(DT[dtype])
        res0 = torch.randn(T, width, generator=g)
        res = res0.clone().to(DEV)
        part.forward(h.to(DEV), res)
        ref = P.dense_ff(h.double(), M.widen(W)) if mlp["kind"] == "dense" else P.moe_ff(h.double(), M.widen(W), mlp)
        assert error(res.cpu() - res0, ref) < TOL[dtype]
        alone = torch.zeros(1, width, device=DEV)                          # a token's rows do not depend on the batch
        part.forward(h[-1:].to(DEV), alone)
        assert error(alone.cpu(), ref[-1:]) < TOL[dtype]


def test_routed_experts_sorted_by_expert_in_a_long_prompt(lib):
    """A bfloat16 prompt long enough that the tokens are listed by expert and every expert runs on its own rows,
    with a choice that differs from token to token and margins that no rounding can turn: a token's input has a
    large entry where its first expert's router row has its only weight and a smaller one for its second."""
    width, mlp = 96, M.moe(4, 2, 48, identity=1, scale=1.3, shared=32)
    cfg = one_layer(M.mamba(2, 8, 8), mlp, width=width)
    g = torch.Generator().manual_seed(17)
    W = M.mlp_weights(mlp, width, g, torch.bfloat16)
    W["router"] = torch.zeros(5, width, dtype=torch.bfloat16)
    W["router"][torch.arange(5), torch.arange(5)] = 2.0
    W["correction"] = torch.zeros(5, dtype=torch.bfloat16)
    part = build_part("feed_forward", cfg._feed_forward("", mlp), W, "bfloat16")
    T = 400
    part.GROUPED_FROM = 48                       # rows an expert from which the tokens are sorted: far fewer than in use
    assert T * 2 >= part.GROUPED_FROM * 4 and part.per_expert is not None
    h = 0.3 * torch.randn(T, width, generator=g)
    first = torch.randint(0, 5, (T,), generator=g)
    second = (first + torch.randint(1, 5, (T,), generator=g)) % 5
    h[torch.arange(T), first] += 4.0
    h[torch.arange(T), second] += 2.0
    h = h.bfloat16()
    chosen, _ = P.route(h.double(), M.widen(W), mlp["router"])
    assert torch.equal(chosen.sort(-1).values, torch.stack([first, second], 1).sort(-1).values)
    res = torch.zeros(T, width, device=DEV)
    part.forward(h.to(DEV), res)
    ref = P.moe_ff(h.double(), M.widen(W), mlp)
    assert error(res.cpu(), ref) < TOL["bfloat16"]
    few = torch.zeros(7, width, device=DEV)                      # the same rows among few: every token through every expert
    part.forward(h[:7].to(DEV), few)
    assert error(few.cpu(), ref[:7]) < TOL["bfloat16"]


def test_reinject_multiplies_stream_and_embedding_side_by_side(lib):
    from llm_infer_amd.config.spec import PartSpec
    g = torch.Generator().manual_seed(3)
    w = 64
    weight = (torch.randn(w, 2 * w, generator=g) / 8).bfloat16()
    part = build_part("stream", PartSpec("reinject", {"hidden_size": w, "name": "in"}, "loop."), {"in": weight}, "float32")
    x, x0 = torch.randn(9, w, generator=g), torch.randn(9, w, generator=g)
    xd, x0d = x.to(DEV), x0.to(DEV)
    got = part.forward(xd, x0d, None).cpu()
    assert (got.double() - torch.cat([x, x0], 1).double() @ weight.double().T).abs().max() < 1e-5
    assert torch.equal(xd.cpu(), x) and torch.equal(x0d.cpu(), x0)


# ---------------------------------------------------------------------------
# the whole model
# ---------------------------------------------------------------------------
def engine_for(lib, models, name, dtype, max_tokens=2048):
    folder, cfg, W = models[name, dtype == "bfloat16"]
    return lib.load(folder, dtype=dtype, max_tokens=max_tokens), cfg, W


def all_rows(n):
    return list(range(n))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompts_portions_and_decoding(lib, models, name, dtype, monkeypatch):
    from llm_infer_amd.parts.feed_forward import RoutedExperts
    monkeypatch.setattr(RoutedExperts, "GROUPED_FROM", 8)      # so that these short prompts sort their tokens by expert too
    eng, cfg, W = engine_for(lib, models, name, dtype)
    n = 230
    toks = tokens(cfg, n, 7)
    ref = P.forward(cfg, W, toks, torch.float64)
    s = eng.alloc_slot()
    whole = eng.step([s], [toks], [all_rows(n)]).cpu()
    eng.free_slot(s)
    assert M.row_error(whole, ref) < TOL[dtype]
    assert M.row_error(whole[:3], ref[:3]) < TOL[dtype]                    # the first tokens of a sequence
    # portions of several sizes, down to two tokens and one
    s = eng.alloc_slot()
    pieces, at = [], 0
    for k in [49, 2, 1, 12, 64, 2, 3, n - 133]:
        pieces.append(eng.step([s], [toks[at:at + k]], [all_rows(k)]).cpu())
        at += k
    cut = torch.cat(pieces)
    eng.free_slot(s)
    assert at == n and M.row_error(cut, ref) < TOL[dtype]
    # a prompt, then token by token
    s = eng.alloc_slot()
    head = 70
    pieces = [eng.step([s], [toks[:head]], [all_rows(head)]).cpu()]
    pieces += [eng.step([s], [[t]], [[0]]).cpu() for t in toks[head:]]
    dec = torch.cat(pieces)
    eng.free_slot(s)
    assert M.row_error(dec, ref) < TOL[dtype]
    if dtype == "float32":
        assert torch.equal(cut, whole) and torch.equal(dec, whole)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(lib, models, dtype):
    eng, cfg, W = engine_for(lib, models, "A", dtype)
    lens = [1, 130, 64, 7, 51]
    reqs = [tokens(cfg, n + 6, 10 + i) for i, n in enumerate(lens)]
    refs = [P.forward(cfg, W, r, torch.float64) for r in reqs]
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


def test_long_decoding(lib, models):
    """330 tokens one by one in float32, over seven blocks of the first attention and five pages."""
    eng, cfg, W = engine_for(lib, models, "A", "float32")
    n = 360
    toks = tokens(cfg, n, 21)
    ref = P.forward(cfg, W, toks, torch.float64)
    s = eng.alloc_slot()
    rows = [eng.step([s], [toks[:30]], [all_rows(30)]).cpu()] + [eng.step([s], [[t]], [[0]]).cpu() for t in toks[30:]]
    eng.free_slot(s)
    assert M.row_error(torch.cat(rows), ref) < TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(lib, models, dtype):
    """engine.generate (planner, batches, recorded decode steps) against the plain implementation's own choice,
    as long as its margin leaves no doubt; recorded and eager steps give the same tokens."""
    eng, cfg, W = engine_for(lib, models, "A", dtype)
    prompts = [tokens(cfg, n, 30 + n) for n in (5, 66, 1, 48)]
    n_new = 20
    got = eng.generate(prompts, max_new_tokens=n_new, temperature=0.0)
    eager = eng.generate(prompts, max_new_tokens=n_new, temperature=0.0, use_graph=False)
    assert eng.decode_counts["replayed"] > 0
    checked = 0
    for p, new, e in zip(prompts, got, eager):
        assert len(new) == n_new
        toks = list(p)
        for t, te in zip(new, e):
            last = P.forward(cfg, W, toks, torch.float64)[-1]
            top2 = torch.topk(last, 2).values
            if (top2[0] - top2[1]).item() <= 1.5 * TOL[dtype] * last.std().item():
                break
            assert t == te == int(last.argmax())
            toks.append(t)
            checked += 1
    assert checked > n_new * len(prompts) // 4
    hot = eng.generate(prompts, max_new_tokens=8, temperature=0.8, seed=3)
    assert hot == eng.generate(prompts, max_new_tokens=8, temperature=0.8, seed=3) and all(len(h) == 8 for h in hot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_in_three_schedules(lib, models, dtype, tmp_path):
    folder, cfg, W = models["A", dtype == "bfloat16"]
    reqs = {"a": tokens(cfg, 140, 1), "b": tokens(cfg, 3, 2), "c": tokens(cfg, 70, 3), "d": tokens(cfg, 1, 4)}
    refs = {r: P.forward(cfg, W, t, torch.float64) for r, t in reqs.items()}
    for k, (steps, where) in enumerate((TU.steps_whole(reqs), TU.steps_tail(reqs, tail=12),
                                        TU.steps_batches(reqs, 3, {"a": 9, "b": 2, "c": 9}))):
        out = TU.run_trace(folder, dtype, steps, where, cfg["vocab"], 512, str(tmp_path / f"{dtype}{k}"))
        for (r, p), row in out.items():
            assert M.row_error(torch.from_numpy(row)[None], refs[r][p:p + 1]) < TOL[dtype], (k, r, p)


def test_command_line_and_model_info(lib, models):
    folder, cfg, W = models["A", False]
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
            assert t == int(P.forward(cfg, W, toks, torch.float64)[-1].argmax())
            toks.append(t)
    for word in ("Dimensions: 96", "Vocab size: 131"):
        assert word in res.stdout, res.stdout
    info = subprocess.run([sys.executable, os.path.join(root, "bin", "model_info"), folder], capture_output=True, text=True,
                          timeout=300)
    assert info.returncode == 0 and "Architecture: Risonex" in info.stdout and "The tensors fit the model." in info.stdout
