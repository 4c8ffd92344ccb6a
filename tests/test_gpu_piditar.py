"""The Piditar decoder through the library against the plain implementation (plain_piditar.py): each mixer alone through its
part, then whole models through Engine.step and generate() with every way of cutting and batching, on configurations made here."""
import json
import os
import random
import subprocess
import sys

import pytest
import torch

import piditar_common as C
import plain_piditar as plain
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import Cache
from tq_kv_amd.engine.context import StepContext
from tq_kv_amd.parts import BuildEnv, PartSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(autouse=True)
def _seeded():
    torch.manual_seed(1234)


# ---- each mixer alone ------------------------------------------------------------------------------------
def mixer_spec(kind, m, hidden, eps):
    if kind == "attention":
        pos = (PartSpec("rotary", {"theta": m["rot"]["base"], "rot_dim": m["rot"]["dims"], "max_positions": 512, "style": "pairs"})
               if m["rot"]["dims"] else PartSpec("none", {"max_positions": 512}))
        return PartSpec("attention", {"hidden": hidden, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
                                      "scale": m["scale"], "qkv_bias": True, "qk_norm": True, "qk_norm_weight": False, "qk_norm_after_rotation": True,
                                      "eps": eps, "cap": m["softcap"], "position": pos,
                                      "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b"}})
    if kind == "rglru":
        return PartSpec("rglru", {"hidden": hidden, "width": m["width"], "blocks": m["blocks"], "conv": m["conv"],
                                  "names": {"y": "y", "y_bias": "y.b", "x": "x", "x_bias": "x.b", "conv": "conv", "conv_bias": "conv.b", "gate_a": "ra",
                                            "gate_a_bias": "ra.b", "gate_i": "ri", "gate_i_bias": "ri.b", "decay": "lam", "o": "o"}})
    return PartSpec("mamba2", {"hidden": hidden, "heads": m["heads"], "head_dim": m["vdim"], "state": m["state"], "groups": m["groups"], "conv": m["conv"],
                               "norm_groups": m["norm_groups"], "eps": eps,
                               "names": {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D", "norm": "norm", "o": "o"}})


MIXERS = [C.attention(6, 3, 24, 40, 16, base=40.0), C.attention(1, 1, 8, 8, 2, base=2.0, softcap=1.0), C.attention(3, 3, 10, 14, 6, softcap=9.0),
          C.attention(4, 1, 32, 16, 32), C.attention(8, 2, 64, 64, 0), C.attention(16, 2, 96, 128, 64, scale=0.5), C.attention(2, 1, 160, 200, 40),
          C.rglru(80, 5, 4), C.rglru(8, 1, 1), C.rglru(36, 3, 3), C.rglru(512, 2, 2), C.rglru(640, 1, 8),
          C.mamba2(6, 20, 24, 3, 3, 4), C.mamba2(1, 8, 1, 1, 1, 1), C.mamba2(3, 14, 10, 3, 4, 3), C.mamba2(8, 64, 128, 1, 4, 2), C.mamba2(4, 32, 200, 2, 2, 1)]


def step_ctx(cache, items):
    sizes = [(s, len(t)) for s, t in items]
    cache.reserve(sizes)
    return StepContext([(s, cache.length(s), t) for s, t in items], [[] for _ in items], cache, DEV), sizes


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mix", MIXERS, ids=lambda m: m[0] + "-" + "x".join(str(v) for v in m[1].values() if isinstance(v, int)))
def test_a_mixer_alone(dtype, mix):
    """Two sequences in shared steps: one in portions of 230, 26, 2 and 2 tokens and then token by token, across pages' borders; the other whole
    beside the first portion.  Then the slots are given back and taken again: nothing of the first use may be left."""
    kind, m = mix
    hidden, eps = 88, 1e-5
    cfg = C.config(50, hidden, [(mix, None)])
    w_all = C.weights(cfg, 3)
    w = {k[len("l0.mix."):]: v for k, v in w_all.items() if k.startswith("l0.mix.")}
    env = BuildEnv(DEV, DT[dtype])
    part = env.build("mixer", mixer_spec(kind, m, hidden, eps))
    assert part.graph_safe and sorted(part.tensors()) == sorted(w)
    part.load({k: v.to(DT[dtype]).to(DEV) for k, v in w.items()})
    cache = Cache([part.cache_need()], [None], 64 * 8, 2, DT[dtype], DEV)
    assert (len(cache.state_groups) == 1) == (kind != "attention")
    xs = [torch.randn(n, hidden).to(DT[dtype]) for n in (300, 40)]
    want = [plain.mixer(kind, x.float(), C.as_float(w), "", m, eps, torch.arange(x.shape[0]), DT[dtype]) for x in xs]
    # (the first step is long enough for the recurrences to run in chunks, beside a sequence shorter than a chunk; the second is not)
    plan = [[(0, 0, 230), (1, 0, 40)], [(0, 230, 256)], [(0, 256, 258)], [(0, 258, 260)]] + [[(0, t, t + 1)] for t in range(260, 300)]
    for use in range(2):
        slots = [cache.acquire(), cache.acquire()]
        got = [[], []]
        for step in plan:
            ctx, sizes = step_ctx(cache, [(slots[i], [0] * (b - a)) for i, a, b in step])
            y = part.forward(torch.cat([xs[i][a:b] for i, a, b in step]).to(DEV), ctx, cache.entry(0))
            cache.commit(sizes)
            off = 0
            for i, a, b in step:
                got[i].append(y[off:off + b - a])
                off += b - a
        for i in range(2):
            e = C.row_errors(torch.cat(got[i]), want[i])
            assert e.max().item() < (2e-5 if dtype == "float32" else 0.02), "use %d, sequence %d: %.3g" % (use, i, e.max().item())
        for s in slots:
            cache.release(s)


@pytest.mark.parametrize("style", ["pairs", "halves"])
@pytest.mark.parametrize("m", [C.attention(6, 2, 64, 40, 24), C.attention(2, 1, 160, 16, 160), C.attention(4, 4, 24, 24, 0)], ids=lambda m: "x".join(str(v) for v in m[1].values() if isinstance(v, int)))
def test_long_steps_turn_and_norm_heads_as_short_ones_do(style, m):
    """Steps of more than 64 tokens add the biases, turn and norm the heads in pieces of several elements and store the values with the
    lanes along the tokens; shorter steps go element by element.  Both orders of rotation, the same tokens either way."""
    hidden, eps = 72, 1e-5
    spec = mixer_spec("attention", m[1], hidden, eps)
    if m[1]["rot"]["dims"]:
        spec.params["position"].params["style"] = style
    cfg = C.config(50, hidden, [(m, None)])
    w = {k[len("l0.mix."):]: v for k, v in C.weights(cfg, 5).items() if k.startswith("l0.mix.")}
    env = BuildEnv(DEV, torch.bfloat16)
    part = env.build("mixer", spec)
    part.load({k: v.to(DEV) for k, v in w.items()})
    cache = Cache([part.cache_need()], [None], 64 * 8, 2, torch.bfloat16, DEV)
    x = torch.randn(200, hidden).to(torch.bfloat16)
    got = []
    for cuts in ([200], [40, 40, 40, 40, 40]):
        slot, a, out = cache.acquire(), 0, []
        for n in cuts:
            ctx, sizes = step_ctx(cache, [(slot, [0] * n)])
            out.append(part.forward(x[a:a + n].to(DEV), ctx, cache.entry(0)))
            cache.commit(sizes)
            a += n
        cache.release(slot)
        got.append(torch.cat(out).float())
    assert C.row_errors(got[0], got[1]).max().item() < 0.02
    if style == "pairs":
        want = plain.mixer("attention", x.float(), C.as_float(w), "", m[1], eps, torch.arange(200), torch.bfloat16)
        assert C.row_errors(got[0], want).max().item() < 0.02


def test_the_convolution_reads_its_first_inputs_from_the_state_and_zeros_before_the_start():
    """One channel group with weights 1, 10, 100, 1000 on the four taps and no recurrence to speak of (the decay is driven to zero): what a token's
    output holds of each earlier input can be read off, whole and in portions of one token."""
    hidden, width = 8, 8
    m = {"width": width, "blocks": 1, "conv": 4}
    env = BuildEnv(DEV, torch.float32)
    part = env.build("mixer", mixer_spec("rglru", m, hidden, 1e-5))
    w = {n: torch.zeros(*s.shape) for n, s in part.tensors().items()}
    w["x"] = torch.eye(width, hidden)
    w["conv"] = torch.tensor([1.0, 10.0, 100.0, 1000.0]).repeat(width, 1)
    w["lam"] = torch.full((width,), 40.0)
    w["ri.b"] = torch.full((1, width), 40.0)           # the input gate is open
    w["y.b"] = torch.full((width,), 30.0)              # gelu_tanh(30) = 30
    w["o"] = torch.eye(hidden, width) / 30.0
    part.load({k: v.to(DEV) for k, v in w.items()})
    cache = Cache([part.cache_need()], [None], 64, 1, torch.float32, DEV)
    x = torch.arange(1.0, 7.0)[:, None].repeat(1, hidden)          # inputs 1 .. 6
    want = torch.tensor([1000.0, 2100.0, 3210.0, 4321.0, 5432.0, 6543.0])[:, None].repeat(1, hidden)
    for cuts in ([6], [1, 1, 1, 1, 1, 1], [2, 1, 3], [4, 2]):
        s = cache.acquire()
        out, a = [], 0
        for n in cuts:
            ctx, sizes = step_ctx(cache, [(s, [0] * n)])
            out.append(part.forward(x[a:a + n].to(DEV), ctx, cache.entry(0)))
            cache.commit(sizes)
            a += n
        torch.testing.assert_close(torch.cat(out).cpu(), want, rtol=1e-6, atol=0)
        cache.release(s)


# ---- whole models ----------------------------------------------------------------------------------------
_MODELS = {}
MAKERS = {"mixed": C.config_mixed, "ones": C.config_ones, "odd": C.config_odd, "attention": lambda: C.config_single("attention"),
          "attention_equal": lambda: C.config_single("attention_equal"),
          "rglru": lambda: C.config_single("rglru"), "mamba2": lambda: C.config_single("mamba2")}


def model(name, tmp_path_factory, memory="some"):
    key = (name, memory)
    if key not in _MODELS:
        cfg = MAKERS[name]()
        w = C.weights(cfg, seed=11 + len(name), memory=memory)
        folder = C.write_folder(str(tmp_path_factory.mktemp("piditar_%s" % name)), cfg, w)
        _MODELS[key] = (cfg, w, folder, {})
    return _MODELS[key]


def engine(name, dtype, tmp_path_factory, memory="some", max_tokens=4096, slots=8):
    cfg, w, folder, engines = model(name, tmp_path_factory, memory)
    if dtype not in engines:
        engines[dtype] = Engine(Model.from_dir(folder, dtype=dtype), max_tokens=max_tokens, max_slots=slots)
    return cfg, w, engines[dtype]


def run_cut(eng, toks, cuts):
    """One request alone, its tokens in portions that end at `cuts`; the logits of every position."""
    s = eng.open()
    out, a = [], 0
    for b in list(cuts) + [len(toks)]:
        b = min(b, len(toks))
        if b > a:
            out.append(eng.step([(s, toks[a:b], list(range(b - a)))]))
            a = b
    eng.close(s)
    return torch.cat(out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "ones", "odd"])
def test_whole_prompts_and_every_cut(name, dtype, tmp_path_factory):
    cfg, w, eng = engine(name, dtype, tmp_path_factory)
    assert eng.model.spec.architecture == "Piditar" and eng.model.graph_safe
    toks = C.tokens(200, cfg["vocab"], 5)
    layers = []
    want = plain.forward(cfg, C.as_float(w), toks, layers_out=layers)
    assert len(layers) == len(eng.model.spec.order) == len(plain.run_order(cfg))
    whole = run_cut(eng, toks, [])
    C.close(whole, want, dtype, "whole")
    C.close(whole[:3], want[:3], dtype, "the first tokens")
    for cuts in ([64], [63, 65], [1, 3, 128, 130], [150, 152, 154] + list(range(155, 200)), list(range(2, 200, 2)), list(range(1, 200))):
        got = run_cut(eng, toks, cuts)
        C.close(got, want, dtype, "cuts %s" % cuts[:4])
        if dtype == "float32":          # no sum depends on the cut: states are carried exactly
            assert torch.equal(got, whole), "float32 logits depend on the cut %s" % cuts[:4]


def poison(eng):
    """NaN into every page that no sequence holds and into the state rows of every slot that is free: nothing may read them
    (a slot's state is cleared when the slot is taken)."""
    for g in eng.cache.kv_groups:
        held = {p for pages in g.pages.values() for p in pages if p >= 0}
        free = [p for p in range(g.pool.n) if p not in held]
        if free:
            g.keys[:, torch.tensor(free, device=g.keys.device)] = float("nan")
            g.values[:, torch.tensor(free, device=g.keys.device)] = float("nan")
    free = [s for s in range(eng.cache.max_slots) if not eng.cache.slots.is_held(s)]
    for g in eng.cache.state_groups:
        if free:
            g.state[:, torch.tensor(free, device=g.state.device)] = float("nan")


@pytest.mark.parametrize("dtype", DTYPES)
def test_batches_of_unequal_requests_and_reused_slots(dtype, tmp_path_factory):
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory, max_tokens=64 * 12, slots=4)
    reqs = [C.tokens(n, cfg["vocab"], 30 + n) for n in (130, 7, 66, 1, 95, 64, 20)]
    want = [C.plain_logits(cfg, w, t) for t in reqs]
    alone = [run_cut(eng, t, []) for t in reqs]
    # three batches one after the other in a cache that only holds them because ended requests give pages and slots back;
    # what they leave behind is overwritten with NaN as soon as nobody holds it
    for batch in ([0, 1, 2, 3], [4, 5, 6, 1], [2, 0, 4]):
        heads = {i: max(1, len(reqs[i]) - 3 - 5 * k) for k, i in enumerate(batch)}
        slots = {i: eng.open() for i in batch}
        poison(eng)
        got = eng.step([(slots[i], reqs[i][:heads[i]], list(range(heads[i]))) for i in batch])
        off = 0
        for i in batch:
            C.close(got[off:off + heads[i]], want[i][:heads[i]], dtype, "prompt of %d in a batch" % i)
            if dtype == "float32":
                assert torch.equal(got[off:off + heads[i]], alone[i][:heads[i]])
            off += heads[i]
        pos, live = dict(heads), [i for i in batch if heads[i] < len(reqs[i])]
        for i in batch:
            if i not in live:
                eng.close(slots[i])
        while live:
            poison(eng)
            got = eng.step([(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            for k, i in enumerate(live):
                C.close(got[k:k + 1], want[i][pos[i]:pos[i] + 1], dtype, "request %d decoded at %d" % (i, pos[i]))
                if dtype == "float32":
                    assert torch.equal(got[k], alone[i][pos[i]])
                pos[i] += 1
            for i in live:
                if pos[i] == len(reqs[i]):
                    eng.close(slots[i])
            live = [i for i in live if pos[i] < len(reqs[i])]
    eng.cache.check()


def logits_of(eng, tokens, how, n):
    if how == "prompt":
        return run_cut(eng, tokens, [])
    if how == "portions":
        return run_cut(eng, tokens, [61, 63, 130])
    return run_cut(eng, tokens, [100] + list(range(101, n)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["attention", "attention_equal"])
def test_a_token_reaches_every_later_position_through_attention_and_none_before(name, dtype, tmp_path_factory):
    """One attention layer with a scale that lets single keys carry the output: changing the token at j changes the logits at i if and only
    if j <= i.  Queries in a prompt, in a later portion, and decoded one by one; keys at the sequence's start, at page borders and far away."""
    cfg, w, eng = engine(name, dtype, tmp_path_factory)
    n = 200
    toks = C.tokens(n, cfg["vocab"], 8)
    for how in ("prompt", "portions", "decoded"):
        base = logits_of(eng, toks, how, n)
        C.close(base, C.plain_logits(cfg, w, toks), dtype, how)
        for i in (130, 191, 199):
            for j in sorted({0, 1, 63, 64, 65, 127, 128, i - 1, i, i + 1}):
                if j >= n:
                    continue
                changed = list(toks)
                changed[j] = (toks[j] + 1 + j) % cfg["vocab"]
                got = logits_of(eng, changed, how, n)[i]
                moved = (got - base[i]).abs().max().item()
                if j <= i:
                    assert moved > 0.0 or dtype == "bfloat16", "%s: query %d does not see the token at %d" % (how, i, j)
                else:
                    assert moved == 0.0, "%s: query %d sees the later token at %d" % (how, i, j)


@pytest.mark.parametrize("vdim", [24, 64])
def test_one_key_far_away_among_hundreds_carries_the_output(vdim, tmp_path_factory):
    """Two tokens have an element of the embedding to themselves; the keys of the one and the queries of the other read it with one and the
    same long vector, so that this key's score stands far above three hundred random ones: the output at the query is that token's value,
    wherever the token stands (first, at a page's border, far back) and however the query comes (in the prompt or decoded)."""
    cfg = C.config(60, 32, [(C.attention(2, 1, 64, vdim, 0, scale=1.0, softcap=100.0), None)], scale=1.0)
    n, special, asker = 330, 7, 11
    toks = [t if t not in (special, asker) else 20 for t in C.tokens(n, cfg["vocab"], 2)]
    f = C.as_float(C.weights(cfg, 4))
    f["embed"][:, 0] = 0.0
    f["embed"][special, 0] = f["embed"][asker, 0] = 3.0
    direction = torch.randn(64)
    f["l0.mix.k"][:, 0] = 3.0 * direction
    f["l0.mix.q"][:, 0] = 3.0 * direction.repeat(2)
    f["l0.mix.v"] = f["l0.mix.v"] * 3.0
    w = {k: v.to(torch.bfloat16) for k, v in f.items()}
    folder = C.write_folder(str(tmp_path_factory.mktemp("piditar_far")), cfg, w)
    for dtype in DTYPES:
        eng = Engine(Model.from_dir(folder, dtype=dtype), max_tokens=1024, max_slots=2)
        for place in (0, 1, 63, 64, 128, 200):
            seq = list(toks)
            seq[place], seq[n - 1] = special, asker
            want = C.plain_logits(cfg, w, seq)[-1:]
            other = list(seq)
            other[place] = 21
            assert C.row_errors(C.plain_logits(cfg, w, other)[-1:], want).item() > 0.2          # the one key matters
            C.close(run_cut(eng, seq, [])[-1:], want, dtype, "prompt, key at %d" % place)
            C.close(run_cut(eng, seq, [300] + list(range(301, n)))[-1:], want, dtype, "decoded, key at %d" % place)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["rglru", "mamba2"])
def test_a_forgetful_recurrence_sees_exactly_the_convolutions_reach(kind, dtype, tmp_path_factory):
    """One recurrent layer whose decay is driven to zero: the state forgets everything at once, and what is left is the short convolution.
    Changing the token at j changes the logits at i if and only if i - taps < j <= i; in prompts, across portions' borders, and decoded."""
    cfg, w, eng = engine(kind, dtype, tmp_path_factory, memory="none")
    taps = cfg["layers"][0]["mixer"]["conv"]
    n = 140
    toks = C.tokens(n, cfg["vocab"], 9)
    for how in ("prompt", "portions", "decoded"):
        base = logits_of(eng, toks, how, n)
        # (with the state gone a position's output hangs on few numbers, and bfloat16 products move a row here and there by a fifth of
        # the spread: bfloat16 is held to the plain implementation with its products rounded the same way)
        C.close(base, C.plain_logits(cfg, w, toks, DT[dtype]), dtype, how)
        for i in (2, 62, 63, 64, 65, 101, 130, 131, 139):
            for back in (0, 1, taps - 1, taps, taps + 1, 60):
                j = i - back
                if j < 0:
                    continue
                changed = list(toks)
                changed[j] = (toks[j] + 1 + j) % cfg["vocab"]
                moved = (logits_of(eng, changed, how, n)[i] - base[i]).abs().max().item()
                if back < taps:
                    assert moved > 0.0, "%s: position %d does not hold the token %d back" % (how, i, back)
                else:
                    assert moved == 0.0, "%s: position %d holds the token %d back (moved %.3g)" % (how, i, back, moved)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["rglru", "mamba2"])
def test_a_recurrence_carries_the_first_token_to_the_last(kind, dtype, tmp_path_factory):
    """With decays near one the state remembers: the first token moves the logits hundreds of positions on, decoded or not."""
    cfg, w, eng = engine(kind, dtype, tmp_path_factory, memory="long")
    n = 260
    toks = C.tokens(n, cfg["vocab"], 10)
    changed = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    want, want_changed = C.plain_logits(cfg, w, toks), C.plain_logits(cfg, w, changed)
    assert C.row_errors(want_changed[-1:], want[-1:]).item() > 2e-3          # ten times what float32 is held to
    for cuts in ([], [200] + list(range(201, n))):
        C.close(run_cut(eng, toks, cuts), want, dtype, "cuts %s" % cuts[:2])
        C.close(run_cut(eng, changed, cuts), want_changed, dtype, "another first token, cuts %s" % cuts[:2])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "odd"])
def test_long_decoding(name, dtype, tmp_path_factory):
    """A prompt of some pages, then a hundred and fifty tokens decoded one by one (replayed from a captured graph)."""
    cfg, w, eng = engine(name, dtype, tmp_path_factory)
    toks = C.tokens(500, cfg["vocab"], 21)
    want = C.plain_logits(cfg, w, toks)
    s = eng.open()
    got = [eng.step([(s, toks[:350], [0, 1, 2, 300, 349])])]
    for t in range(350, 500):
        got.append(eng.step([(s, [toks[t]], [0])]))
    eng.close(s)
    C.close(torch.cat(got), want[[0, 1, 2, 300, 349] + list(range(350, 500))], dtype, "a long sequence")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_loop(dtype, tmp_path_factory):
    cfg, w, eng = engine("mixed", dtype, tmp_path_factory)
    prompts = [C.tokens(n, cfg["vocab"], 50 + n) for n in (1, 9, 70, 33, 128)]
    params = GenerationParams(max_tokens=12, temperature=0.0, repeat_penalty=1.0)
    out = generate(eng, prompts, params, eos_ids=(), max_batch=3)
    for p, o in zip(prompts, out):
        assert len(o) == 12
        seq = list(p)
        for k, t in enumerate(o):
            z = C.plain_logits(cfg, w, seq)[-1]
            if int(z.argmax()) != t:        # a step whose two best logits are closer than rounding may go either way
                assert dtype == "bfloat16" and (z.max() - z[t]).item() < 0.05 * z.std().item(), "token %d of a prompt of %d" % (k, len(p))
            seq.append(t)
    again = generate(eng, prompts[::-1], params, eos_ids=(), max_batch=2)
    assert again[::-1] == out or dtype == "bfloat16"


# ---- configurations drawn at random -------------------------------------------------------------------------
def draw(seed):
    r = random.Random(seed)
    width = r.choice([48, 64, 96, 160, 200, 256])
    layers = []
    for _ in range(r.randint(1, 5)):
        kind = r.choice(["attention", "rglru", "mamba2"])
        if kind == "attention":
            kv = r.choice([1, 2, 3, 4])
            dim = r.choice([8, 12, 16, 24, 32, 48, 64, 80, 96, 128])
            mix = C.attention(kv * r.choice([1, 1, 2, 3, 4, 8]), kv, dim, r.choice([8, 12, 16, 32, 48, 64, 96, 136]), r.choice([0, 2, dim // 4 * 2, dim]),
                              base=r.choice([10.0, 500.0, 10000.0, 1e6]), scale=r.uniform(0.5, 1.5) / dim ** 0.5, softcap=r.choice([2.0, 8.0, 30.0, 50.0]))
        elif kind == "rglru":
            blocks = r.choice([1, 2, 3, 4, 8])
            mix = C.rglru(blocks * r.choice([4, 8, 12, 16, 40, 64]), blocks, r.choice([1, 2, 3, 4, 5]))
        else:
            groups = r.choice([1, 2, 3])
            heads = groups * r.choice([1, 2, 4])
            vdim = r.choice([8, 12, 16, 32, 64])
            parts = r.choice([d for d in (1, 2, 3, 4, heads) if (heads * vdim) % d == 0])
            mix = C.mamba2(heads, vdim, r.choice([1, 8, 16, 40, 64, 100, 128]), groups, r.choice([1, 2, 3, 4]), parts)
        layers.append((mix, r.choice([None, 24, 64, 100, 256])))
    n = len(layers)
    start = r.randint(0, n)
    stop = r.randint(start, n)
    loop = r.choice([None, (start, stop, r.randint(1, 3))])
    return C.config(r.choice([64, 101, 256, 500]), width, layers, loop=loop, eps=r.choice([1e-6, 1e-5, 1e-3]), scale=r.choice([1.0, 3.0, 12.0]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(16))
def test_random_configuration(seed, dtype, tmp_path):
    cfg = draw(3000 + seed)
    w = C.weights(cfg, seed)
    eng = Engine(Model.from_dir(C.write_folder(str(tmp_path), cfg, w), dtype=dtype), max_tokens=64 * 24, max_slots=4)
    a, b = C.tokens(150 + 7 * seed, cfg["vocab"], seed), C.tokens(40 + seed, cfg["vocab"], 100 + seed)
    want_a, want_b = C.plain_logits(cfg, w, a), C.plain_logits(cfg, w, b)
    s = eng.open()
    whole = eng.step([(s, a, list(range(len(a))))])
    eng.close(s)
    C.close(whole, want_a, dtype, "whole")
    # two portions, then single tokens, with the second request alongside from its first token to its end
    sa, sb = eng.open(), eng.open()
    cut1, cut2 = 70 + seed, len(a) - 20
    got_a = [eng.step([(sa, a[:cut1], list(range(cut1)))])]
    both = eng.step([(sa, a[cut1:cut2], list(range(cut2 - cut1))), (sb, b[:-10], list(range(len(b) - 10)))])
    got_a.append(both[:cut2 - cut1])
    got_b = [both[cut2 - cut1:]]
    for i in range(20):
        items = [(sa, [a[cut2 + i]], [0])]
        if i < 10:
            items.append((sb, [b[len(b) - 10 + i]], [0]))
        out = eng.step(items)
        got_a.append(out[:1])
        if i < 10:
            got_b.append(out[1:])
        if i == 9:
            eng.close(sb)
    eng.close(sa)
    C.close(torch.cat(got_a), want_a, dtype, "portions and single tokens")
    C.close(torch.cat(got_b), want_b, dtype, "the request alongside")
    if dtype == "float32":
        assert torch.equal(torch.cat(got_a), whole)


# ---- the programs a user runs ---------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_of_steps_and_the_command_line(dtype, tmp_path_factory):
    """bin/trace_run fed steps on standard input (a request whole, then its last tokens one by one beside a second request), and bin/tq
    generate on the same folder: logits and greedy tokens of the plain implementation."""
    from test_gpu_trace_run import Replay
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    cfg = C.config_odd()
    w = C.weights(cfg, seed=77)
    folder = C.write_folder(str(tmp_path_factory.mktemp("piditar_replay")), cfg, w)
    a, b = C.tokens(150, cfg["vocab"], 1), C.tokens(9, cfg["vocab"], 2)
    want_a, want_b = C.plain_logits(cfg, w, a), C.plain_logits(cfg, w, b)
    r = Replay(folder, dtype, str(tmp_path_factory.mktemp("out")), max_tokens=64 * 6)
    got = r.step([("x", a, list(range(150)))], end=["x"])
    C.close(got.view(-1, cfg["vocab"]), want_a, dtype, "whole")
    assert r.step([("y", a[:140], []), ("z", b[:5], [])]) is None
    for t in range(10):
        live = [("y", [a[140 + t]], [0])] + ([("z", [b[5 + t]], [0])] if t < 4 else [])
        got = r.step(live, end=(["y"] if t == 9 else []) + (["z"] if t == 3 else [])).view(-1, cfg["vocab"])
        C.close(got[0:1], want_a[140 + t:141 + t], dtype, "one by one at %d" % t)
        if t < 4:
            C.close(got[1:2], want_b[5 + t:6 + t], dtype, "the second request at %d" % t)
    r.finish()
    if dtype != "float32":
        return
    cmd = [sys.executable, os.path.join(root, "bin", "tq"), "--fp32", "generate", folder, "--prompt-ids", ",".join(str(t) for t in b), "-n", "5", "-t", "0",
           "--repeat-penalty", "1.0", "--json"]
    out = subprocess.run(cmd, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr
    tokens = json.loads(out.stdout.strip().splitlines()[-1])["outputs"][0]
    seq = list(b)
    for t in tokens:
        assert int(C.plain_logits(cfg, w, seq)[-1].argmax()) == t
        seq.append(t)
