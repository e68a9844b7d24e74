"""Risonex without a GPU: the plain implementation pinned by library routines, closed forms and invariants; the
configuration read from its keys; the order of runs with a loop; the tensor table; what the cache does with blocks
of positions."""
import math

import pytest
import torch

import plain_risonex as P
import risonex_models as M


def test_norm_gelu_and_sinusoid_against_library_routines():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(5, 48, generator=g, dtype=torch.float64), 0.1 * torch.randn(48, generator=g, dtype=torch.float64)
    ref = torch.nn.functional.rms_norm(x, (48,), 1.0 + w, 1e-5)
    assert (P.norm_one_plus(x, w, 1e-5) - ref).abs().max() < 1e-12
    assert (P.gelu_erf(x) - torch.nn.functional.gelu(x)).abs().max() < 1e-12
    assert (P.silu(x) - torch.nn.functional.silu(x)).abs().max() < 1e-12
    assert (P.softplus(x * 20) - torch.nn.functional.softplus(x * 20, threshold=50)).abs().max() < 1e-12
    s = P.sinusoid([0, 3, 17], 10, torch.float64)
    assert s[0].tolist() == [0.0, 1.0] * 5
    for i in range(5):
        a = 17 * 10000.0 ** (-2 * i / 10)
        assert abs(s[2, 2 * i] - math.sin(a)) < 1e-12 and abs(s[2, 2 * i + 1] - math.cos(a)) < 1e-12


def test_attention_maps_blocks_and_the_difference():
    g = torch.Generator().manual_seed(1)
    n, H, G, d, dv, B = 23, 4, 2, 6, 5, 8
    q, k = torch.randn(n, H, 2, d, generator=g, dtype=torch.float64), torch.randn(n, G, 2, d, generator=g, dtype=torch.float64)
    v = torch.randn(n, G, dv, generator=g, dtype=torch.float64)
    see = P.chunk_mask(n, B)
    assert see[7, 0] and see[8, 8] and not see[8, 7] and not see[7, 8] and see[15, 8] and not see[16, 15]
    raw = P.diff_attention_core(q, k, v, 0.4, 0.0, B, None, 1.0)       # lambda 0: the first map alone
    for head in (0, 3):
        kv = head // 2
        bias = torch.zeros(n, n, dtype=torch.float64).masked_fill(~see, float("-inf"))
        ref = torch.nn.functional.scaled_dot_product_attention(q[None, :, head, 0], k[None, :, kv, 0], v[None, :, kv],
                                                               attn_mask=bias[None], scale=0.4)[0]
        assert (raw[:, head] - ref).abs().max() < 1e-12
    # the second map enters with -lambda, the first token of every block copies its own value
    both = P.diff_attention_core(q, k, v, 0.4, 0.7, B, None, 1.0)
    second = P.diff_attention_core(q.flip(2), k.flip(2), v, 0.4, 0.0, B, None, 1.0)
    assert (both - (raw - 0.7 * second)).abs().max() < 1e-12
    assert (both[8, 1] - (1 - 0.7) * v[8, 0]).abs().max() < 1e-12
    normed = P.diff_attention_core(q, k, v, 0.4, 0.7, B, 0.0, 0.3)
    assert ((normed ** 2).mean(-1) - 0.09).abs().max() < 1e-12
    # what lies before the block changes nothing
    k2, v2 = k.clone(), v.clone()
    k2[:16], v2[:16] = 9.0, -9.0
    assert torch.equal(P.diff_attention_core(q, k2, v2, 0.4, 0.7, B, 1e-5, 1.0)[16:], P.diff_attention_core(q, k, v, 0.4, 0.7, B, 1e-5, 1.0)[16:])
    t = {"lq1": torch.tensor([0.5, 1.0]), "lk1": torch.tensor([2.0, -1.0]), "lq2": torch.tensor([1.0, 1.0]), "lk2": torch.tensor([0.5, 0.5])}
    assert abs(P.diff_lambda(t, 0.2) - (1.0 - math.e + 0.2)) < 1e-6


def test_convolution_and_recurrence_against_closed_forms():
    g = torch.Generator().manual_seed(2)
    u, w, b = torch.randn(9, 3, generator=g, dtype=torch.float64), torch.randn(3, 4, generator=g, dtype=torch.float64), torch.randn(3, dtype=torch.float64, generator=g)
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (3, 0)), w[:, None, :], b, groups=3)[0].T
    assert (P.causal_conv(u, w, b) - ref).abs().max() < 1e-12
    # one head, one value, a state of one: y_t = sum over s <= t of (product of the decays after s) dt_s B_s x_s C_t + D x_t
    m = {"heads": 1, "vdim": 1, "state": 1, "groups": 1, "conv": 1, "norm_groups": 1}
    width, n = 4, 6
    t = {"in": torch.randn(5, width, generator=g, dtype=torch.float64), "conv": torch.ones(3, 1, dtype=torch.float64),
         "conv.b": torch.zeros(3, dtype=torch.float64), "dt_bias": torch.tensor([0.3], dtype=torch.float64),
         "A_log": torch.tensor([-0.2], dtype=torch.float64), "D": torch.tensor([0.7], dtype=torch.float64),
         "norm": torch.ones(1, dtype=torch.float64), "o": torch.ones(1, 1, dtype=torch.float64)}
    h = torch.randn(n, width, generator=g, dtype=torch.float64)
    proj = h @ t["in"].T
    z, x, B, C = proj[:, 0], P.silu(proj[:, 1]), P.silu(proj[:, 2]), P.silu(proj[:, 3])
    dt = torch.nn.functional.softplus(proj[:, 4] + 0.3)
    a = torch.exp(-math.exp(-0.2) * dt)
    y = torch.stack([sum(torch.prod(a[s + 1:i + 1]) * dt[s] * B[s] * x[s] for s in range(i + 1)) * C[i] + 0.7 * x[i] for i in range(n)])
    gated = y * P.silu(z)
    ref = gated / torch.sqrt(gated ** 2 + 1e-5)
    assert (P.mamba2(h, t, m, 1e-5)[:, 0] - ref).abs().max() < 1e-10
    # causal: a later token changes nothing before it
    h2 = h.clone()
    h2[4] += 1.0
    assert torch.equal(P.mamba2(h2, t, m, 1e-5)[:4], P.mamba2(h, t, m, 1e-5)[:4])


def test_routing_choice_weights_identity_and_the_shared_gate():
    g = torch.Generator().manual_seed(3)
    width, mlp = 8, M.moe(3, 2, 4, identity=2, scale=1.5, shared=4)
    t = {k: v.double() for k, v in M.mlp_weights(mlp, width, g, torch.float32).items()}
    h = torch.randn(1, width, generator=g, dtype=torch.float64)
    t["router"] = torch.zeros(5, width, dtype=torch.float64)
    t["router"][:, 0] = torch.tensor([0.0, 1.0, 2.0, 3.0, 0.5], dtype=torch.float64) / h[0, 0]        # logits 0, 1, 2, 3, 0.5
    t["correction"] = torch.tensor([10.0, 0.0, 0.0, 0.0, 0.0], dtype=torch.float64)
    chosen, w = P.route(h, t, mlp["router"])
    s = torch.softmax(torch.tensor([0.0, 1.0, 2.0, 3.0, 0.5], dtype=torch.float64), 0)
    assert sorted(chosen[0].tolist()) == [0, 3]                                  # the correction chose output 0
    assert abs(w.sum().item() - 1.5) < 1e-12
    assert abs(w[0, chosen[0].tolist().index(0)].item() - 1.5 * s[0] / (s[0] + s[3])) < 1e-12   # weighted without it
    out = P.moe_ff(h, t, mlp)
    ref = (1.5 * s[0] / (s[0] + s[3])) * P.gated_expert(h, t, "e0.") + (1.5 * s[3] / (s[0] + s[3])) * h \
        + torch.sigmoid(h @ t["shared.sg"].T) * P.gated_expert(h, t, "shared.")
    assert (out - ref).abs().max() < 1e-12                                       # output 3 is the first identity


def test_the_order_of_runs_and_the_loop_input():
    cfg = M.TINY_A
    assert P.layer_runs(cfg) == [(0, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert P.layer_runs(M.TINY_B) == [(0, False), (1, False)]
    assert P.layer_runs(M.TINY_C) == [(0, True), (0, True), (0, True), (1, False)]
    W = M.widen(M.random_weights(cfg, 5))
    toks = [3, 9, 27, 81, 4]
    logits, streams = P.forward(cfg, W, toks, torch.float64, streams=True)
    assert streams.shape == (6, 5, cfg["width"])
    # the loop's matrix takes the stream first and the embedding's output second
    x0 = P.embed(toks, W["embed"], cfg["embedding"]["scale"], cfg["width"])
    after0 = streams[0]
    entered = after0 @ W["loop.in"][:, :cfg["width"]].T + x0 @ W["loop.in"][:, cfg["width"]:].T
    assert (P.layer(entered, 1, cfg["layers"][1], W, cfg["norm"]["eps"], torch.float64) - streams[1]).abs().max() < 1e-9
    # causal as a whole
    longer = P.forward(cfg, W, toks + [7], torch.float64)
    assert (longer[:5] - logits).abs().max() < 1e-9


def test_configuration_reads_every_key_and_describes_the_model():
    import llm_infer_amd  # noqa: F401
    from llm_infer_amd.config.spec import ConfigError
    from llm_infer_amd.engine.model import DecoderModel
    from llm_infer_amd.registry import config_from_dict
    for name, raw in M.ALL.items():
        cfg = config_from_dict(raw)
        assert config_from_dict(cfg.to_dict()) == cfg
        assert cfg.runs() == P.layer_runs(raw)
        spec = cfg.model_spec()
        assert [(e.layer, e.before is not None) for e in spec.schedule] == P.layer_runs(raw)
        model = DecoderModel(spec, torch.float32, "cpu", allocate=False)
        W = M.random_weights(raw, 1)
        assert {k: tuple(v.shape) for k, v in model.params().items()} == {k: tuple(v.shape) for k, v in W.items()}
        # one cache unit for each attention run, two (state and the convolution's history) for each state-space run
        kinds = [raw["layers"][i]["type"] for i, _ in P.layer_runs(raw)]
        assert len(model.cache_specs()) == sum(1 if k == "attention" else 2 for k in kinds)
    a = config_from_dict(M.TINY_A).model_spec()
    att = a.layers[1].sublayers[0].part.params
    assert (att["block"], att["lambda_init"], att["out_scale"], att["scale"]) == (50, 0.2, 0.8, 20 ** -0.5)
    ffn = a.layers[1].sublayers[1].part.params
    assert (ffn["n_experts"], ffn["n_identity"], ffn["top"], ffn["route_scale"], ffn["shared_ff"]) == (5, 1, 3, 2.0, 24)
    assert len(a.layers[0].sublayers) == 1 and a.embedding.params["scale"] == 2.5
    for broken in ({"type": "conv"}, {"mixer": {"heads": 3}}):
        raw = M.config(32, 10, [dict(M.layer(M.mamba(2, 8, 4), None), **broken)])
        with pytest.raises(ConfigError):
            config_from_dict(raw)
    with pytest.raises(ConfigError):
        config_from_dict(M.config(32, 10, [M.layer(M.mamba(2, 8, 4), None)], loop=(0, 2, 2)))


def test_the_cache_gives_back_the_pages_behind_a_block():
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.specs import KVSpec, StateSpec
    cache = Cache([KVSpec(2, 32, None, 16, 150, "maps"), StateSpec((4,)), KVSpec(2, 32, None, 16, None, "maps")], 4096, 4096,
                  torch.float32, None)
    blocked, plain = cache.groups[0], cache.groups[2]
    s = cache.alloc_slot()
    cache.grow([s], [200])
    assert sorted(blocked.pages_of[s]) == [0, 1, 2, 3] == sorted(plain.pages_of[s])
    cache.trim_windows([s])
    assert sorted(blocked.pages_of[s]) == [2, 3]                   # the block of position 200 begins at 150, in page 2
    cache.grow([s], [299])
    cache.trim_windows([s])
    assert sorted(blocked.pages_of[s]) == [2, 3, 4]
    cache.grow([s], [300])
    cache.trim_windows([s])
    assert sorted(blocked.pages_of[s]) == [4] and sorted(plain.pages_of[s]) == [0, 1, 2, 3, 4]
    cache.grow([s], [301])                                         # page 4 is there already, nothing before it comes back
    assert sorted(blocked.pages_of[s]) == [4]
    cache.free_slot(s)
    assert blocked.pool.n_free == blocked.n_pages - 1


def test_tiles_and_segments_are_planned_from_the_steps_lengths():
    """The host's plans for a step: attention tiles of up to 32 consecutive tokens that never cross a sequence, and
    the recurrence's segments with every sequence's first segment and count."""
    from llm_infer_amd.engine.step import StepContext
    from llm_infer_amd.kernels import ops
    ctx = StepContext("cpu", [0, 1, 2], [[0] * 70, [0], [0] * 32], [5, 0, 100], [[], [], []])
    # tiles as (first row, rows, steps of 32 keys) with blocks of 64 positions: the first sequence, from position 5,
    # has (0, 32, 2), (32, 32, 3) (positions 37 .. 68 straddle a block's edge) and (64, 6, 1); then (70, 1, 1); the third,
    # from position 100, (71, 32, 3); the heaviest with the lightest, an odd one alone
    t0, n, count = ops.diff_tiles(ctx, 64)
    assert count == 3 and t0.tolist() == [32, 70, 71, 64, 0, 0] and n.tolist() == [32, 1, 32, 6, 32, 0]
    assert ops.diff_tiles(ctx, 64) is ops.diff_tiles(ctx, 64)              # made once per step for a block size
    assert ops.diff_tile_pairs([100], [0], 0, 0) == ([96, 0, 64, 32], [4, 32, 32, 32])   # no blocks: later tiles see more
    seg = ops.ssm_segments(ctx, 32)
    assert seg["n"] == 5 and seg["seg_seq"].tolist() == [0, 0, 0, 1, 2] and seg["seg_t0"].tolist() == [0, 32, 64, 0, 0]
    assert seg["seg_n"].tolist() == [32, 32, 6, 1, 32] and seg["seq_seg0"].tolist() == [0, 3, 4] and seg["seq_nseg"].tolist() == [3, 1, 1]
    decode = StepContext("cpu", [0, 1], [[3], [4]], [9, 2], [[0], [0]])
    assert ops.diff_tiles(decode) is None                                  # every token a tile of its own
