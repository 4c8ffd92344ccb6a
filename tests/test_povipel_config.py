"""Povipel without a GPU: its configuration keys and their errors, the ModelSpec they become (run order, needs, tensor names), steps
and generation of a model in host memory on the null device."""
import copy
import math

import pytest
import torch

import plain_povipel as plain
import povipel_common as C
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import PAGE
from tq_kv_amd.config import ConfigError, config_from_dict, known_architectures
from tq_kv_amd.config.registry import spec_from_dict
from tq_kv_amd.parts.spec import ModelSpec


def test_the_architecture_is_known_by_its_name():
    assert "Povipel" in known_architectures()
    name, typed = config_from_dict(C.config_mixed())
    assert name == "Povipel"
    assert config_from_dict(typed.to_dict())[1] == typed                # round trip through config.json
    assert (typed.vocab, typed.width, typed.norm_eps, typed.embedding_scale, typed.streams, typed.logit_softcap) == (331, 96, 3e-6, 7.5, 3, 18.0)
    assert [l.type for l in typed.layers] == ["parallel", "retention", "parallel", "retention", "parallel"]
    assert typed.run_order() == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4] == plain.run_order(C.config_mixed())
    assert typed.layers[0].mixer["left"]["window"] == 37 and typed.layers[0].mixer["left"]["pool"] == 6 and typed.layers[1].mlp == {"kind": "moe", "ff": 40, "experts": 5, "top": 2}
    # a configuration without the keys: every layer once, one stream with a plain sum, logits as they are
    bare = C.config_single("retention", streams=None)
    del bare["logit_softcap"]
    t = config_from_dict(bare)[1]
    assert t.run_order() == [0] and t.streams is None and t.logit_softcap is None and config_from_dict(t.to_dict())[1] == t


def test_the_spec_names_tensors_parts_and_needs():
    cfg = C.config_mixed()
    spec = spec_from_dict(cfg)
    assert ModelSpec.from_json(spec.to_json()) == spec
    assert spec.embedding_name == "embed" and spec.head_name == "head" and spec.final_norm_prefix == "final.norm" and spec.embedding_scale == 7.5
    assert spec.final_norm.kind == "layer_norm" and spec.logit_cap == 18.0
    assert all(l.block.kind == "multi_stream" and l.block.params["streams"] == 3 and l.block.params["token_shift"] is True for l in spec.layers)
    assert [l.block.params["mixer"].kind for l in spec.layers] == ["parallel", "linear_attention", "parallel", "linear_attention", "parallel"]
    par = spec.layers[0].block.params["mixer"].params
    att, lin = par["first"].params, par["second"].params
    assert (att["window"], att["pool"], att["value_dim"], att["qk_norm"], att["sink"], att["rotate_values"], att["scale"]) == (37, 6, 40, True, True, True, 0.3)
    assert att["position"].params["style"] == "pairs" and att["position"].params["rot_dim"] == 16 and att["value_position"].params["rot_dim"] == 40
    assert (lin["decay"], lin["tau"], lin["norm_weight"], lin["position"]) == ("channels", 5.0, True, None) and abs(lin["q_scale"] - 20 ** -0.5) < 1e-12
    ret = spec.layers[1].block.params["mixer"].params
    assert (ret["decay"], ret["norm_weight"], ret["position"].params["style"]) == ("heads", False, "halves") and abs(ret["k_scale"] - 24 ** -0.5) < 1e-12
    ff = spec.layers[1].block.params["feed_forward"]
    assert ff.kind == "routed_experts" and (ff.params["score"], ff.params["weight_on"], ff.params["top"], ff.params["n_experts"]) == ("sigmoid", "input", 2, 5)
    assert spec.layers[0].block.params["feed_forward"].kind == "activated" and spec.layers[2].block.params["feed_forward"] is None
    model = Model(spec, dtype="float32", device="cpu")
    specs = model.tensor_specs()
    # the names and shapes are those of the weights the tests make, whose low rank (5) no key of the configuration names
    w = C.weights(cfg, 1, rank=5)
    assert set(specs) == set(w)
    free = {"l0.mix.right.a1": 0, "l0.mix.right.a2": 1, "l2.mix.right.a1": 0, "l2.mix.right.a2": 1, "l4.mix.right.a1": 0, "l4.mix.right.a2": 1}
    for name, t in w.items():
        want = list(specs[name].shape)
        if name in free:
            want[free[name]] = 5
        assert list(t.shape) == want, name
    # the cache: every run has an entry of its own; attention's pages with the blocks' rows behind the positions, the states in one row
    needs = model.needs
    assert len(needs) == 11
    assert needs[0].key_page == (3, PAGE + 11, 24) and needs[0].value_page == (3, PAGE + 11, 40) and needs[0].window is None
    assert needs[0].state_shape == (3 * 20 * 12 + 96,) and needs[1].shape == (3 * 24 * 20 + 96,)


@pytest.mark.parametrize("path,value,word", [
    (("width",), None, "width"), (("vocab",), "many", "vocab"), (("norm",), None, "norm"), (("embedding", "scale"), None, "scale"), (("streams",), 0, "streams"),
    (("streams",), 99, "copies"), (("layers",), [], "layers"), (("layers", 0, "type"), "convolution", "convolution"), (("layers", 0, "mixer", "left"), None, "left"),
    (("layers", 0, "mixer", "left", "kv_heads"), 4, "kv_heads"), (("layers", 0, "mixer", "left", "mask", "pool"), 0, "pool"),
    (("layers", 0, "mixer", "left", "mask"), None, "mask"), (("layers", 0, "mixer", "left", "vdim"), 41, "pair"), (("layers", 0, "mixer", "left", "rot", "dims"), 7, "dims"),
    (("layers", 0, "mixer", "right", "tau"), 0, "tau"), (("layers", 0, "mixer", "left", "dim"), 300, "heads of 300"), (("layers", 1, "mixer", "decay"), [0.5], "decay"),
    (("layers", 1, "mixer", "dim"), 600, "key channels"), (("layers", 1, "mixer", "rot", "dims"), 26, "dims"), (("layers", 1, "mlp", "router", "top"), 6, "top"),
    (("layers", 1, "mlp", "expert"), None, "expert"), (("layers", 0, "mlp", "kind"), "sparse", "sparse"), (("loop", "stop"), 7, "loop"), (("loop", "times"), 0, "times")])
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


@pytest.mark.parametrize("make", [C.config_mixed, C.config_ones, C.config_plain_residual])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_and_generation_on_the_null_device(make, dtype):
    cfg = make()
    model = Model.random(cfg, seed=3, dtype=dtype, device="cpu")
    assert not model.on_gpu and model.graph_safe
    engine = Engine(model, max_tokens=6 * PAGE, max_slots=4)
    free0 = [g.pool.n_free for g in engine.cache.kv_groups]
    assert len(engine.cache.kv_groups) >= 1 and all(g.state.dtype == torch.float32 for g in engine.cache.state_groups)
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


def test_a_run_with_pages_and_a_state_row_gets_both():
    """The parallel mixer keeps the attention's pages and, in one row behind each other, the linear attention's state and the block's
    kept token; runs with equal pages share a group of pages whatever their state rows hold."""
    cfg = C.config(40, 16, [(C.parallel(C.left(2, 1, 8, 8, 10, 4, 4), C.right(1, 4, 6)), None), (C.parallel(C.left(2, 1, 8, 8, 10, 4, 4), C.right(2, 4, 6)), None),
                            (C.retention(1, 4, 4, 2, decay=[0.9]), None)], loop=(0, 3, 2))
    engine = Engine(Model.random(cfg, seed=1, dtype="float32", device="cpu"), max_tokens=4 * PAGE, max_slots=3)
    assert len(engine.cache.kv_groups) == 1 and engine.cache.kv_groups[0].runs == [0, 1, 3, 4]
    assert sorted((tuple(g.runs), g.state.shape[-1]) for g in engine.cache.state_groups) == [((0, 3), 24 + 16), ((1, 4), 48 + 16), ((2, 5), 16 + 16)]
    for run in (0, 1, 3, 4):
        e = engine.cache.entry(run)
        assert e.keys is not None and e.state is not None


# ---- the plain implementation, pinned by closed forms ----------------------------------------------------
def test_plain_window_and_blocks_in_closed_form():
    """Keys that are all alike give every visible position and block the same weight: the output is the mean of what is seen."""
    T, W, P = 40, 5, 4
    q = torch.ones(T, 1, 2)
    k = torch.ones(T, 1, 2)
    v = torch.arange(T, dtype=torch.float32).view(T, 1, 1)
    out = plain.pooled_window_attention(q, k, v, 1.0, W, P, None)[:, 0, 0]
    for i in (0, 3, 4, 7, 8, 9, 39):
        seen = [float(j) for j in range(max(0, i - W + 1), i + 1)]
        seen += [b * P + (P - 1) / 2.0 for b in range(T // P) if b * P + P - 1 <= i - W]
        assert abs(out[i].item() - sum(seen) / len(seen)) < 1e-4, i
    # a sink as large as the scores halves the weight of everything when one position is seen
    one = plain.pooled_window_attention(q[:1], k[:1], torch.ones(1, 1, 1), 1.0, W, P, torch.tensor([2.0]))
    assert abs(one.item() - 0.5) < 1e-6


def test_plain_decaying_state_in_closed_form():
    q = torch.ones(3, 1, 2)
    k = torch.tensor([[[1.0, 2.0]], [[0.0, 1.0]], [[1.0, 0.0]]])
    v = torch.tensor([[[1.0]], [[10.0]], [[100.0]]])
    decay = torch.tensor([0.5, 0.25]).view(1, 1, 2).expand(3, 1, 2)
    out = plain.decayed_state_attention(q, k, v, decay)[:, 0, 0].tolist()
    s0 = (1.0, 2.0)
    s1 = (0.5 * s0[0], 0.25 * s0[1] + 10.0)
    s2 = (0.5 * s1[0] + 100.0, 0.25 * s1[1])
    assert out == pytest.approx([sum(s0), sum(s1), sum(s2)])


def test_plain_layer_norm_rotation_and_shift_in_closed_form():
    x = torch.tensor([[1.0, 3.0]])
    assert torch.allclose(plain.layer_norm(x, torch.tensor([2.0, 2.0]), torch.tensor([0.5, 0.5]), 0.0), torch.tensor([[-1.5, 2.5]]))
    v = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 5.0, 7.0]]]).expand(3, 1, 6)
    ang = plain.angles(torch.arange(3), 16.0, 4)                 # position, position / 4
    assert torch.allclose(ang[2], torch.tensor([2.0, 0.5]))
    pairs = plain.turn(v, ang, "pairs")[2, 0]
    assert torch.allclose(pairs, torch.tensor([math.cos(2.0), math.sin(2.0), -2.0 * math.sin(0.5), 2.0 * math.cos(0.5), 5.0, 7.0]), atol=1e-6)
    halves = plain.turn(v, ang, "halves")[2, 0]                  # element 0 with 2, 1 with 3
    assert torch.allclose(halves, torch.tensor([math.cos(2.0), -2.0 * math.sin(0.5), math.sin(2.0), 2.0 * math.cos(0.5), 5.0, 7.0]), atol=1e-6)
    assert torch.allclose(plain.turn(plain.turn(v, ang, "pairs"), -ang, "pairs"), v, atol=1e-6)
    n = torch.tensor([[1.0, 10.0], [3.0, 20.0], [5.0, 40.0]])
    assert torch.allclose(plain.token_shift(n, torch.tensor([0.5, 0.0])), torch.tensor([[0.5, 10.0], [2.0, 20.0], [4.0, 40.0]]))
