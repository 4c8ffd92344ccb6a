"""Piditar without a GPU: its configuration keys and their errors, the ModelSpec they become (run order, needs, tensor names),
steps and generation of a model in host memory on the null device, and the plain implementation pinned by closed forms."""
import copy
import math

import pytest
import torch

import piditar_common as C
import plain_piditar as plain
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import PAGE
from tq_kv_amd.config import ConfigError, config_from_dict, known_architectures
from tq_kv_amd.config.registry import spec_from_dict
from tq_kv_amd.parts.spec import ModelSpec


def test_the_architecture_is_known_by_its_name():
    assert "Piditar" in known_architectures()
    name, typed = config_from_dict(C.config_mixed())
    assert name == "Piditar"
    assert config_from_dict(typed.to_dict())[1] == typed                # round trip through config.json
    t = typed.to_typed()
    assert (t["vocab"], t["width"], t["norm_eps"], t["embedding_scale"]) == (331, 96, 3e-6, 7.5)
    assert [l["type"] for l in t["layers"]] == ["rglru", "attention", "mamba2", "rglru", "mamba2", "attention"]
    assert (t["loop_start"], t["loop_stop"], t["loop_times"]) == (1, 4, 3)
    assert typed.run_order() == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4, 5]
    assert [None if l["mlp"] is None else l["mlp"]["ff"] for l in t["layers"]] == [72, 56, None, 40, 88, 64]
    # a configuration without the key runs every layer once
    plain_cfg = C.config_single("rglru")
    assert "loop" not in plain_cfg and config_from_dict(plain_cfg)[1].run_order() == [0]


def test_the_span_of_layers_runs_again_with_the_embedding_added():
    """What the run order says for spans at the start, in the middle, at the end, of one pass, of no layer, and without the key."""
    five = [(C.rglru(8, 1, 2), None)] * 5
    for loop, order in [((0, 5, 2), [0, 1, 2, 3, 4, 0, 1, 2, 3, 4]), ((1, 3, 3), [0, 1, 2, 1, 2, 1, 2, 3, 4]), ((3, 5, 2), [0, 1, 2, 3, 4, 3, 4]),
                        ((2, 4, 1), [0, 1, 2, 3, 4]), ((2, 2, 4), [0, 1, 2, 3, 4]), (None, [0, 1, 2, 3, 4])]:
        cfg = C.config(40, 16, five, loop=loop)
        spec = spec_from_dict(cfg)
        assert [r.layer for r in spec.order] == order == [i for i, _ in plain.run_order(cfg)]
        again = [k for k, r in enumerate(spec.order) if r.add_embedding]
        assert again == [k for k, (_, a) in enumerate(plain.run_order(cfg)) if a]
        if loop and loop[2] > 1 and loop[1] > loop[0]:
            assert len(again) == loop[2] - 1 and all(order[k] == loop[0] for k in again)
        else:
            assert again == []
        assert ModelSpec.from_json(spec.to_json()) == spec                  # the flag survives the round trip through JSON


def test_the_spec_names_tensors_parts_and_needs():
    spec = spec_from_dict(C.config_mixed())
    assert spec.embedding_name == "embed" and spec.head_name is None and spec.final_norm_prefix == "final.norm" and spec.embedding_scale == 7.5
    assert all(l.block.kind == "pre_norm" for l in spec.layers)
    assert [l.block.params["mixer"].kind for l in spec.layers] == ["rglru", "attention", "mamba2", "rglru", "mamba2", "attention"]
    att = spec.layers[1].block.params["mixer"].params
    assert (att["qkv_bias"], att["qk_norm"], att["qk_norm_weight"], att["qk_norm_after_rotation"], att["cap"], att["value_dim"]) == (True, True, False, True, 20.0, 40)
    assert att["position"].params["style"] == "pairs" and att["position"].params["rot_dim"] == 16
    assert spec.layers[2].block.params["feed_forward"] is None and spec.layers[2].block.params["ff_norm"] is None
    assert spec.layers[0].block.params["mixer_norm"].params["unit_offset"] is True
    model = Model(spec, dtype="float32", device="cpu")
    specs = model.tensor_specs()
    names = set(specs)
    assert {"embed", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.y", "l0.mix.y.b", "l0.mix.x.b", "l0.mix.conv", "l0.mix.conv.b", "l0.mix.ra", "l0.mix.ri.b",
            "l0.mix.lam", "l0.mix.o", "l1.mix.q", "l1.mix.q.b", "l1.mix.k.b", "l1.mix.v.b", "l2.mix.in", "l2.mix.dt_bias", "l2.mix.A_log", "l2.mix.D",
            "l2.mix.norm", "l2.mix.conv.b", "l5.mlp.down"} <= names
    assert not {"head", "l2.norm2", "l1.mix.q.norm", "l1.mix.k.norm", "l2.mlp.gate"} & names
    assert specs["l0.mix.ra"].shape == (5, 16, 16) and specs["l0.mix.ra.b"].shape == (5, 16) and specs["l0.mix.conv"].shape == (80, 4)
    assert specs["l1.mix.v"].shape == (3 * 40, 96) and specs["l1.mix.v.b"].shape == (120,) and specs["l1.mix.o"].shape == (96, 240)
    assert specs["l2.mix.in"].shape == (2 * 120 + 2 * 3 * 24 + 6, 96) and specs["l2.mix.conv"].shape == (120 + 144, 3) and specs["l2.mix.norm"].shape == (120,)
    # the cache: every run has an entry of its own; the recurrent ones a row of float32 (the convolution's inputs, then the state)
    needs = model.needs
    assert len(needs) == 12
    order = [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4, 5]
    assert [getattr(n, "shape", None) for n in needs] == [{0: (3 * 80 + 80,), 1: None, 2: (2 * 264 + 6 * 24 * 20,), 3: (64 + 64,), 4: (4 * (64 + 80) + 4 * 40 * 16,), 5: None}[l]
                                                          for l in order]
    assert (needs[1].n_kv_heads, needs[1].head_dim, needs[1].value_dim, needs[1].window) == (3, 24, 40, None)


@pytest.mark.parametrize("path,value,word", [
    (("width",), None, "width"), (("vocab",), "many", "vocab"), (("norm",), None, "norm"), (("embedding",), None, "embedding"),
    (("embedding", "scale"), None, "scale"), (("layers",), [], "layers"), (("layers", 0, "type"), "convolution", "convolution"),
    (("layers", 1, "mixer", "heads"), 0, "heads"), (("layers", 1, "mixer", "kv_heads"), 4, "kv_heads"), (("layers", 1, "mixer", "vdim"), None, "vdim"),
    (("layers", 1, "mixer", "rot", "dims"), 7, "dims"), (("layers", 1, "mixer", "rot"), None, "rot"), (("layers", 1, "mixer", "scale"), None, "scale"),
    (("layers", 0, "mixer", "blocks"), 7, "blocks"), (("layers", 0, "mixer", "conv"), 0, "conv"), (("layers", 0, "mixer", "conv"), 9, "taps"),
    (("layers", 2, "mixer", "groups"), 4, "groups"), (("layers", 2, "mixer", "norm_groups"), 7, "norm_groups"), (("layers", 2, "mixer", "state"), None, "state"),
    (("layers", 2, "mixer", "state"), 300, "state"), (("layers", 0, "mlp", "kind"), "sparse", "sparse"), (("layers", 0, "mlp", "ff"), -3, "ff"),
    (("loop", "stop"), 7, "loop"), (("loop", "start"), 5, "loop"), (("loop", "times"), 0, "times")])
def test_what_is_missing_or_wrong_is_named(path, value, word):
    raw = copy.deepcopy(C.config_mixed())
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError, match=word):
        spec = spec_from_dict(raw)
        Model(spec, dtype="float32", device="cpu")          # what a part refuses is refused when the model is put together


@pytest.mark.parametrize("make", [C.config_mixed, C.config_ones, C.config_odd])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_and_generation_on_the_null_device(make, dtype):
    cfg = make()
    model = Model.random(cfg, seed=3, dtype=dtype, device="cpu")
    assert not model.on_gpu and model.graph_safe
    engine = Engine(model, max_tokens=6 * PAGE, max_slots=4)
    free0 = [g.pool.n_free for g in engine.cache.kv_groups]
    assert len(engine.cache.state_groups) >= 1 and all(g.state.dtype == torch.float32 for g in engine.cache.state_groups)
    a, b = engine.open(), engine.open()
    out = engine.step([(a, C.tokens(150, cfg["vocab"], 1), [0, 149]), (b, C.tokens(3, cfg["vocab"], 2), [2])])
    assert tuple(out.shape) == (3, cfg["vocab"])
    for step in range(3):
        engine.step([(a, [step], [0]), (b, [step], [0])])
    assert (engine.length(a), engine.length(b)) == (153, 6)
    engine.close(a), engine.close(b)
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0
    engine.cache.check()
    got = generate(engine, [C.tokens(n, cfg["vocab"], 10 + n) for n in (5, 1, 17, 70)], GenerationParams(max_tokens=4, temperature=0.0, repeat_penalty=1.0),
                   eos_ids=(), max_batch=3)
    assert got == [[0] * 4] * 4
    assert [g.pool.n_free for g in engine.cache.kv_groups] == free0


def test_a_model_of_recurrent_layers_alone_holds_no_pages():
    cfg = C.config(40, 16, [(C.rglru(8, 2, 3), 24), (C.mamba2(2, 4, 8, 1, 2, 1), None)], loop=(0, 2, 2))
    engine = Engine(Model.random(cfg, seed=1, dtype="float32", device="cpu"), max_tokens=PAGE, max_slots=3)
    assert not engine.cache.holds_pages and engine.cache.max_slots == 3 and len(engine.cache.kv_groups) == 0
    # two state groups (one per kind of row), each with the rows of both passes
    assert sorted(tuple(g.state.shape[:2]) for g in engine.cache.state_groups) == [(2, 3), (2, 3)]
    s = engine.open()
    engine.step([(s, C.tokens(500, 40, 1), [499])])          # far beyond max_tokens: nothing grows with the sequence
    engine.close(s)


# ---- the plain implementation, pinned by closed forms ----------------------------------------------------
def test_plain_rotation_turns_neighbouring_pairs_of_the_first_elements_only():
    v = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 5.0, 7.0]]]).expand(3, 1, 6)
    r = plain.turn_pairs(v, torch.arange(3), 16.0, 4)          # angles: position, position / 4
    want = [math.cos(2.0), math.sin(2.0), -2.0 * math.sin(0.5), 2.0 * math.cos(0.5), 5.0, 7.0]
    assert torch.allclose(r[2, 0], torch.tensor(want), atol=1e-6)
    assert torch.equal(r[0], v[0]) and torch.equal(plain.turn_pairs(v, torch.arange(3), 16.0, 0), v)


def test_plain_heads_are_unit_normed_after_the_rotation_and_scores_are_capped():
    q = torch.tensor([[[10.0, 0.0]]]).expand(2, 1, 2)
    k = torch.tensor([[[0.0, 0.0]], [[10.0, 0.0]]])
    v = torch.tensor([[[1.0]], [[0.0]]])
    capped = plain.causal_softmax_attention(q, k, v, 1.0, 2.0)[1, 0, 0].item()
    assert abs(capped - 1.0 / (1.0 + math.exp(2.0 * math.tanh(50.0)))) < 1e-6      # scores 0 and 100 become 0 and 2 tanh(50)
    assert torch.allclose(plain.unit_norm(torch.tensor([3.0, 4.0, 0.0, 0.0]), 0.0), torch.tensor([1.2, 1.6, 0.0, 0.0]))
    assert torch.allclose(plain.offset_norm(torch.tensor([2.0, 2.0]), torch.tensor([0.5, -1.0]), 0.0), torch.tensor([1.5, 0.0]))


def test_plain_convolution_weighs_the_token_itself_with_the_last_column():
    x = torch.arange(1.0, 6.0)[:, None]
    out = plain.short_conv(x, torch.tensor([[100.0, 10.0, 1.0]]), torch.tensor([0.5]))
    assert out[:, 0].tolist() == [1.5, 12.5, 123.5, 234.5, 345.5]


def test_plain_gated_recurrence_in_closed_form():
    """One channel, gates held at constants by their biases: S_t = a S_(t-1) + sqrt(1 - a^2) i u_t."""
    w = {"y": torch.zeros(1, 1), "y.b": torch.tensor([30.0]), "x": torch.ones(1, 1), "x.b": torch.zeros(1), "conv": torch.ones(1, 1), "conv.b": torch.zeros(1),
         "ra": torch.zeros(1, 1, 1), "ra.b": torch.tensor([[0.0]]), "ri": torch.zeros(1, 1, 1), "ri.b": torch.tensor([[math.log(3.0)]]),
         "lam": torch.tensor([math.log(math.e - 1.0)]), "o": torch.ones(1, 1)}
    out = plain.rglru(torch.tensor([[1.0], [2.0], [0.0]]), w, "", {"width": 1, "blocks": 1, "conv": 1}, torch.float32)
    a = math.exp(-8.0 * 0.5 * 1.0)          # softplus(lam) = 1, r = 1/2
    m, i = math.sqrt(1.0 - a * a), 0.75
    s1 = m * i * 1.0
    s2 = a * s1 + m * i * 2.0
    assert torch.allclose(out[:, 0], 30.0 * torch.tensor([s1, s2, a * s2]), rtol=1e-5)


def test_plain_state_space_recurrence_in_closed_form():
    """One head, one state row, one value: S_t = e^(-A dt) S_(t-1) + dt B_t x_t and y_t = C_t S_t + D x_t, then the gate and the norm of one value."""
    m = {"heads": 1, "vdim": 1, "state": 1, "groups": 1, "conv": 1, "norm_groups": 1}
    # rows of the product: z, x, B, C, dt, each reading one input
    w = {"in": torch.eye(5), "conv": torch.ones(3, 1), "conv.b": torch.zeros(3), "dt_bias": torch.tensor([0.0]), "A_log": torch.tensor([math.log(2.0)]),
         "D": torch.tensor([0.5]), "norm": torch.tensor([3.0]), "o": torch.ones(1, 1)}
    h = torch.tensor([[1.0, 2.0, 1.0, 1.0, 0.3], [-1.0, 1.0, 2.0, 0.5, 1.0]])
    out = plain.mamba2(h, w, "", m, 0.0, torch.float32)
    silu = lambda z: z / (1.0 + math.exp(-z))
    sp = lambda z: math.log1p(math.exp(z))
    x0, B0, C0, dt0 = silu(2.0), silu(1.0), silu(1.0), sp(0.3)
    x1, B1, C1, dt1 = silu(1.0), silu(2.0), silu(0.5), sp(1.0)
    S0 = dt0 * B0 * x0
    S1 = math.exp(-2.0 * dt1) * S0 + dt1 * B1 * x1
    y0, y1 = (C0 * S0 + 0.5 * x0) * silu(1.0), (C1 * S1 + 0.5 * x1) * silu(-1.0)
    # a part of one value is divided by its own magnitude: what is left is its sign, times the weight
    assert torch.allclose(out[:, 0], torch.tensor([3.0 * math.copysign(1.0, y0), 3.0 * math.copysign(1.0, y1)]), atol=1e-5)
    m2 = dict(m, vdim=2)
    w2 = dict(w, **{"in": torch.eye(7), "conv": torch.ones(4, 1), "conv.b": torch.zeros(4), "norm": torch.ones(2), "o": torch.eye(2)})
    h2 = torch.tensor([[1.0, 1.0, 2.0, 4.0, 1.0, 1.0, 0.3]])
    out2 = plain.mamba2(h2, w2, "", m2, 0.0, torch.float32)
    v = [(C0 * dt0 * B0 * silu(2.0) + 0.5 * silu(2.0)) * silu(1.0), (C0 * dt0 * B0 * silu(4.0) + 0.5 * silu(4.0)) * silu(1.0)]
    rms = math.sqrt((v[0] ** 2 + v[1] ** 2) / 2.0)
    assert torch.allclose(out2[0], torch.tensor([v[0] / rms, v[1] / rms]), atol=1e-5)
