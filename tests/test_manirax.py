"""Manirax without a GPU: the configuration and what it turns into, and pins of the plain implementation
(each mechanism by a library routine, a closed form or an invariant)."""
import copy
import math

import pytest
import torch

import manirax_models as M
import plain_manirax as P


# ---------------------------------------------------------------------------
# configuration
# ---------------------------------------------------------------------------
def test_config_reads_every_key_and_round_trips():
    import llm_infer_amd
    cfg = llm_infer_amd.config_from_dict(copy.deepcopy(M.TINY_P))
    assert type(cfg).__name__ == "ManiraxConfig"
    assert (cfg.width, cfg.vocab, cfg.norm_eps, cfg.postln_alpha, len(cfg.layers)) == (72, 131, 1e-6, 1.7, 2)
    again = llm_infer_amd.config_from_dict(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()
    # the plural key that other designs use names the class as well
    raw = dict(copy.deepcopy(M.TINY_Q), architectures=["Manirax"])
    del raw["architecture"]
    assert type(llm_infer_amd.config_from_dict(raw)).__name__ == "ManiraxConfig"


@pytest.mark.parametrize("name", list(M.ALL))
def test_parameter_table_names_and_shapes(name):
    import llm_infer_amd
    from llm_infer_amd.engine.model import DecoderModel
    raw = M.ALL[name]
    model = DecoderModel(llm_infer_amd.config_from_dict(copy.deepcopy(raw)).model_spec(), torch.float32, "cpu", allocate=False)
    table = {k: tuple(v.shape) for k, v in model.params().items()}
    want = {k: tuple(v.shape) for k, v in M.random_weights(raw, 0).items()}
    assert table == want
    # a layer without a feed-forward has neither its matrices nor its norm
    for i, L in enumerate(raw["layers"]):
        assert (f"l{i}.norm2" in table) == (L["mlp"] is not None) == (f"l{i}.mlp.up" in table)


def test_model_spec_carries_the_constants():
    import llm_infer_amd
    spec = llm_infer_amd.config_from_dict(copy.deepcopy(M.TINY_P)).model_spec()
    l0, l1 = spec.layers
    assert l0.block == "post_norm" and l0.block_params == {"alpha": 1.7}
    assert l0.position.kind == "rope" and l0.position.params["scaling_factor"] == 2.0
    assert l0.position.params["pairing"] == "half" and l0.position.params["rotary_dim"] == 16
    assert l1.position.params["scaling_factor"] == 1.0 and l1.position.params["theta"] == 500.0
    shift = l0.sublayers[0].part
    assert shift.kind == "token_shift" and shift.params["inner"].kind == "parallel"
    (attn, ls), (lin, rs) = shift.params["inner"].params["branches"]
    assert (ls, rs) == (0.7, 1.3)
    assert attn.params["unit_norm_eps"] == 1e-6 and attn.params["scale"] == 40 ** -0.5 and attn.params["v_head_dim"] == 24
    assert lin.params["decay"] == (0.5, 0.9, 0.99) and lin.params["norm_eps"] == 1e-6
    assert len(l0.sublayers) == 2 and len(l1.sublayers) == 1
    # no rotation in a layer: no position part that rotates
    q = llm_infer_amd.config_from_dict(copy.deepcopy(M.TINY_Q)).model_spec()
    assert q.layers[1].position.kind == "none"
    assert q.max_positions == 0 and q.head.params["tied"] is True


def test_what_the_mixers_ask_of_the_cache():
    import llm_infer_amd
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.specs import KVSpec, StateSpec
    from llm_infer_amd.engine.model import DecoderModel
    model = DecoderModel(llm_infer_amd.config_from_dict(copy.deepcopy(M.TINY_P)).model_spec(), torch.float32, "cpu",
                         allocate=False)
    specs = model.cache_specs()
    assert specs == [StateSpec((72,)), KVSpec(2, 48, None, 32), StateSpec((3, 24, 40)),
                     StateSpec((72,)), KVSpec(1, 16, None, 32), StateSpec((2, 8, 16))]
    cache = Cache(specs, 256, 256, torch.bfloat16, None)
    kv = [g for g in cache.groups if hasattr(g, "pool")]
    # keys 48 wide, values 32 wide (already a multiple of 32): (2 * 64 * 48 + 2 * 64 * 32) elements a page and layer
    assert sorted(g.layer_elems for g in kv) == sorted([2 * 64 * 48 + 2 * 64 * 32, 64 * 16 + 64 * 32])


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].__setitem__("type", "serial"), "not built"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "not built"),
    (lambda c: c["layers"][0]["mixer"]["right"].__setitem__("decay", [0.5]), "one decay for each"),
    (lambda c: c["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 4), "multiple of kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 42), "dims even and within dim"),
    (lambda c: c.pop("postln_alpha"), "lacks 'postln_alpha'"),
    (lambda c: c["norm"].pop("eps"), "lacks 'eps'"),
])
def test_config_errors(change, message):
    import llm_infer_amd
    raw = copy.deepcopy(M.TINY_P)
    change(raw)
    with pytest.raises(llm_infer_amd.ConfigError, match=message):
        llm_infer_amd.config_from_dict(raw)


def test_random_weights_mode_draws_every_tensor():
    from llm_infer_amd.engine.model import DecoderModel
    from llm_infer_amd.weights import random_tensors
    import llm_infer_amd
    model = DecoderModel(llm_infer_amd.config_from_dict(copy.deepcopy(M.TINY_Q)).model_spec(), torch.float32, "cpu",
                         allocate=False)
    t = random_tensors(model.params(), 3)
    assert 0.0 <= t["l0.shift"].min() and t["l0.shift"].max() <= 1.0 and abs(t["l0.shift"].mean() - 0.5) < 0.1
    assert t["l0.mix.left.pb"].abs().max() < 0.2 and abs(t["l0.norm1"].mean() - 1.0) < 0.05


# ---------------------------------------------------------------------------
# the plain implementation, mechanism by mechanism
# ---------------------------------------------------------------------------
def test_plain_layer_norm():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(5, 33, generator=g, dtype=torch.float64) * 3 + 1, torch.randn(33, generator=g, dtype=torch.float64)
    ref = torch.nn.functional.layer_norm(x, (33,), w, None, 1e-3)
    assert (P.layer_norm(x, w, 1e-3) - ref).abs().max() < 1e-12


def test_plain_token_shift():
    h = torch.tensor([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]], dtype=torch.float64)
    mu = torch.tensor([0.0, 0.25], dtype=torch.float64)
    out = P.token_shift(h, mu)
    # channel 0 keeps the token's own value; channel 1 takes a quarter of the way to the one before (0 at the start)
    assert torch.equal(out, torch.tensor([[1.0, 7.5], [2.0, 17.5], [4.0, 35.0]], dtype=torch.float64))


def test_plain_rotation_is_a_rotation_by_scaled_position():
    g = torch.Generator().manual_seed(1)
    v = torch.randn(7, 2, 12, generator=g, dtype=torch.float64)
    pos = torch.arange(7) * 3
    out = P.rotate_half_layout(v, pos, 50.0, 8, 4.0)
    assert torch.equal(out[..., 8:], v[..., 8:])                        # beyond the rotated dimensions
    for i in range(4):
        z = torch.complex(v[..., i], v[..., i + 4]) * torch.polar(torch.ones(7, dtype=torch.float64),
                                                                  pos.double() * 50.0 ** (-2 * i / 8) / 4.0)[:, None]
        assert (out[..., i] - z.real).abs().max() < 1e-12 and (out[..., i + 4] - z.imag).abs().max() < 1e-12
    # a score between rotated vectors depends on the distance only
    a, b = torch.randn(1, 1, 12, generator=g, dtype=torch.float64), torch.randn(1, 1, 12, generator=g, dtype=torch.float64)
    s = [(P.rotate_half_layout(a, torch.tensor([p + 5]), 50.0, 8, 4.0) * P.rotate_half_layout(b, torch.tensor([p]), 50.0, 8, 4.0)).sum()
         for p in (0, 11)]
    assert abs(s[0] - s[1]) < 1e-12


def test_plain_sigmoid_attention_against_the_matrix_form():
    g = torch.Generator().manual_seed(2)
    T, H, G, d, dv = 9, 4, 2, 6, 5
    q, k, v = (torch.randn(T, n, s, generator=g, dtype=torch.float64) for n, s in ((H, d), (G, d), (G, dv)))
    bias = torch.randn(H, generator=g, dtype=torch.float64)
    out = P.sigmoid_attention(q, k, v, 0.4, bias)
    mask = torch.tril(torch.ones(T, T, dtype=torch.float64))
    for h in range(H):
        w = torch.sigmoid(q[:, h] @ k[:, h // 2].t() * 0.4 + bias[h]) * mask
        assert (out[:, h] - w @ v[:, h // 2]).abs().max() < 1e-12
    assert (out[0, 0] - torch.sigmoid((q[0, 0] * k[0, 0]).sum() * 0.4 + bias[0]) * v[0, 0]).abs().max() < 1e-12


def test_plain_decayed_linear_attention_against_the_closed_form():
    g = torch.Generator().manual_seed(3)
    T, H, d, dv = 8, 2, 3, 4
    q, k, v = (torch.randn(T, H, s, generator=g, dtype=torch.float64) for s in (d, d, dv))
    decay = torch.tensor([0.5, 1.0], dtype=torch.float64)
    out = P.decayed_linear_attention(q, k, v, decay)
    for h in range(H):
        for t in range(T):
            ref = sum(decay[h] ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h] for s in range(t + 1))
            assert (out[t, h] - ref).abs().max() < 1e-12


def test_plain_poly_norm():
    z = torch.tensor([[1.0, -2.0, 2.0]], dtype=torch.float64)
    coef = torch.tensor([2.0, 3.0, 5.0, 7.0], dtype=torch.float64)
    r1, r2, r3 = math.sqrt(9 / 3), math.sqrt(33 / 3), math.sqrt(129 / 3)
    ref = 2 * z / r1 + 3 * z ** 2 / r2 + 5 * z ** 3 / r3 + 7
    assert (P.poly_norm(z, coef, 0.0) - ref).abs().max() < 1e-12
    assert (P.unit_rms(z, 1.0) - z / 2.0).abs().max() < 1e-12            # eps inside the root


@pytest.mark.parametrize("name", ["P", "Q"])
def test_plain_model_is_causal_and_layered(name):
    cfg = M.ALL[name]
    W = M.widen(M.random_weights(cfg, 5))
    toks = torch.randint(0, cfg["vocab"], (19,), generator=torch.Generator().manual_seed(6)).tolist()
    logits, streams = P.forward(W, cfg, toks, return_layers=True)
    assert logits.shape == (19, cfg["vocab"]) and streams.shape == (len(cfg["layers"]), 19, cfg["width"])
    assert (P.forward(W, cfg, toks[:11]) - logits[:11]).abs().max() < 1e-9
    # the last layer's stream, normed, times the table
    assert (P.layer_norm(streams[-1], W["final.norm"], cfg["norm"]["eps"]) @ W["embed"].t() - logits).abs().max() < 1e-12
    # alpha and the branch scales matter
    other = copy.deepcopy(cfg)
    other["postln_alpha"] += 0.5
    assert (P.forward(W, other, toks) - logits).abs().max() > 1e-3
    other = copy.deepcopy(cfg)
    other["layers"][0]["mixer"]["right_scale"] += 0.5
    assert (P.forward(W, other, toks) - logits).abs().max() > 1e-3


def test_chunk_lists_of_the_decay_attention():
    from llm_infer_amd.kernels import ops
    assert ops.DECAY_CHUNK == 32
    seq, t0, first = ops.decay_chunk_lists([70, 1, 32, 33])
    assert seq == [0, 0, 0, 1, 2, 3, 3] and t0 == [0, 32, 64, 0, 0, 0, 32] and first == [0, 3, 4, 5]
    # the width of a head in the kernels: the next of 32, 64, 128, 256 (a head of 79 is held as 128, not as 96)
    assert [ops.decay_padded_dim(d) for d in (1, 32, 33, 64, 65, 79, 96, 128, 129, 256)] == [32, 32, 64, 64, 128, 128, 128, 128, 256, 256]


def test_default_slots_are_capped_by_the_states_memory():
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.cache.cache import STATE_BUDGET
    from llm_infer_amd.cache.specs import KVSpec, StateSpec
    big = StateSpec((16, 128, 128))                         # a megabyte a layer and sequence
    cache = Cache([KVSpec(2, 64), big, big], 1 << 20, 4096, torch.bfloat16, None)
    assert cache.n_slots == STATE_BUDGET // (2 * 16 * 128 * 128 * 4) == 4096
    cache = Cache([KVSpec(2, 64)] + [big] * 64, 1 << 20, 4096, torch.bfloat16, None)
    assert cache.n_slots == STATE_BUDGET // (64 * 16 * 128 * 128 * 4) == 128
    assert Cache([KVSpec(2, 64)] + [big] * 64, 1 << 20, 4096, torch.bfloat16, None, n_slots=300).n_slots == 300
    assert Cache([KVSpec(2, 64)], 640, 4096, torch.bfloat16, None).n_slots == 10
