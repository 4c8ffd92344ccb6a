"""The Povipel decoder through the library against the plain implementation (plain_povipel.py): each mechanism alone through its
part, then whole models through Engine.step and generate() with every way of cutting and batching, on configurations made here."""
import pytest
import torch

import plain_povipel as plain
import povipel_common as C
from tq_kv_amd import Engine, GenerationParams, Model, generate
from tq_kv_amd.cache import Cache
from tq_kv_amd.engine.context import StepContext
from tq_kv_amd.parts import BuildEnv, PartSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
DTYPES = ["float32", "bfloat16"]
MAXPOS = 1024


@pytest.fixture(autouse=True)
def _seeded():
    torch.manual_seed(1234)


def rotary(base, dims, style):
    return None if dims == 0 else PartSpec("rotary", {"theta": base, "rot_dim": dims, "max_positions": MAXPOS, "style": style})


def left_spec(m, hidden, eps):
    return PartSpec("pooled_attention", {"hidden": hidden, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
                                         "scale": m["scale"], "window": m["mask"]["size"], "pool": m["mask"]["pool"], "qk_norm": True, "eps": eps, "sink": True,
                                         "rotate_values": True, "position": rotary(m["rot"]["base"], m["rot"]["dims"], "pairs"),
                                         "value_position": rotary(m["rot"]["base"], m["vdim"], "pairs"),
                                         "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink"}})


def right_spec(m, hidden, eps):
    return PartSpec("linear_attention", {"hidden": hidden, "heads": m["heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "decay": "channels", "tau": m["tau"],
                                         "q_scale": m["dim"] ** -0.5, "norm_weight": True, "eps": eps, "position": None,
                                         "names": {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}})


def retention_spec(m, hidden, eps):
    return PartSpec("linear_attention", {"hidden": hidden, "heads": m["heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "decay": "heads",
                                         "head_decay": m["decay"], "k_scale": m["dim"] ** -0.5, "norm_weight": False, "eps": eps,
                                         "position": rotary(m["rot"]["base"], m["rot"]["dims"], "halves"),
                                         "names": {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}})


def mixer_spec(kind, m, hidden, eps):
    if kind == "retention":
        return retention_spec(m, hidden, eps)
    return PartSpec("parallel", {"hidden": hidden, "first": left_spec(m["left"], hidden, eps), "second": right_spec(m["right"], hidden, eps), "eps": eps, "scale": 0.5,
                                 "names": {"first": "left.", "second": "right.", "first_norm": "left.out", "second_norm": "right.out"}})


MIXERS = [C.parallel(C.left(6, 3, 24, 40, 37, 6, 16, base=40.0, scale=0.3), C.right(3, 20, 12, tau=5.0)),
          C.parallel(C.left(1, 1, 8, 2, 1, 1, 2, base=2.0), C.right(1, 1, 1, tau=1.0)),
          C.parallel(C.left(4, 4, 10, 14, 64, 64, 0), C.right(2, 6, 10)),
          C.parallel(C.left(8, 2, 64, 64, 130, 8, 64), C.right(4, 64, 64, tau=16.0)),
          C.parallel(C.left(2, 1, 160, 200, 70, 100, 40, scale=0.05), C.right(2, 130, 70)),
          C.parallel(C.left(2, 2, 32, 64, 33, 5, 16), C.right(1, 32, 32)), C.parallel(C.left(6, 3, 96, 32, 100, 3, 96, scale=0.2), C.right(2, 16, 48)),
          C.retention(3, 24, 20, 16, base=300.0), C.retention(1, 2, 1, 0, decay=[0.5]), C.retention(3, 10, 14, 6), C.retention(4, 128, 128, 128),
          C.retention(2, 200, 136, 64, decay=[0.999, 0.9])]


def step_ctx(cache, items):
    sizes = [(s, len(t)) for s, t in items]
    cache.reserve(sizes)
    return StepContext([(s, cache.length(s), t) for s, t in items], [[] for _ in items], cache, DEV), sizes


def mixer_ids(m):
    flat = m[1] if m[0] == "retention" else dict(m[1]["left"], **{"r" + k: v for k, v in m[1]["right"].items()})
    return m[0] + "-" + "x".join(str(v) for v in flat.values() if isinstance(v, int))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mix", MIXERS, ids=mixer_ids)
def test_a_mixer_alone(dtype, mix):
    """Two sequences in shared steps: one in portions of 230, 26, 2 and 2 tokens and then token by token, across pages' borders, over the
    window's edge and into pooled blocks; the other whole beside the first portion.  Then the slots are given back and taken again:
    nothing of the first use may be left."""
    kind, m = mix
    hidden, eps = 88, 1e-5
    cfg = C.config(50, hidden, [(mix, None)])
    w_all = C.weights(cfg, 3, rank=3)
    w = {k[len("l0.mix."):]: v for k, v in w_all.items() if k.startswith("l0.mix.")}
    env = BuildEnv(DEV, DT[dtype])
    part = env.build("mixer", mixer_spec(kind, m, hidden, eps))
    assert part.graph_safe and sorted(part.tensors()) == sorted(w)
    part.load({k: v.to(DT[dtype]).to(DEV) for k, v in w.items()})
    need = part.cache_need()
    cache = Cache([need], [None], 64 * 8, 2, DT[dtype], DEV)
    assert len(cache.state_groups) == 1 and len(cache.kv_groups) == (1 if kind == "parallel" else 0)
    xs = [torch.randn(n, hidden).to(DT[dtype]) for n in (300, 40)]
    layer = {"type": kind, "mixer": m}
    one_value = (m if kind == "retention" else m["right"])["vdim"] == 1
    want = [plain.mixer(layer, x.float(), C.as_float(w), "", eps, torch.arange(x.shape[0]), DT[dtype]) for x in xs]
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
            # (a head of one value is divided by its own magnitude: next to zero, rounding decides how much of the sign is left)
            limit = (5e-5 if dtype == "float32" else 0.03) * (6.0 if one_value else 1.0)
            assert e.max().item() < limit, "use %d, sequence %d: %.3g" % (use, i, e.max().item())
        for s in slots:
            cache.release(s)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(88, 40, 5, 2), (64, 64, 8, 1), (52, 20, 3, 3), (32, 8, 1, 1), (256, 128, 16, 4)], ids=str)
def test_experts_scored_one_by_one_with_the_weight_on_their_input(dtype, sizes):
    hidden, ff, n, top = sizes
    mlp = C.moe(ff, n, top)
    cfg = C.config(50, hidden, [(C.retention(1, 2, 2, 0), mlp)])
    w = {k[len("l0.mlp."):]: v for k, v in C.weights(cfg, 9).items() if k.startswith("l0.mlp.")}
    part = BuildEnv(DEV, DT[dtype]).build("feed_forward", PartSpec("routed_experts", {
        "hidden": hidden, "inter": ff, "n_experts": n, "top": top, "router_scale": 1.0, "gate": "silu", "score": "sigmoid", "weight_on": "input", "shared": None,
        "names": {"router": "router", "expert": "e%d.", "gate": "gate", "up": "up", "down": "down"}}))
    assert sorted(part.tensors()) == sorted(w)
    part.load({k: v.to(DT[dtype]).to(DEV) for k, v in w.items()})
    for rows in (1, 7, 150):
        x = (2.0 * torch.randn(rows, hidden)).to(DT[dtype])
        want = plain.experts_ff(x.float(), C.as_float(w), "", mlp, DT[dtype])
        e = C.row_errors(part.forward(x.to(DEV)), want)
        assert e.max().item() < (2e-5 if dtype == "float32" else 0.03), "%d rows: %.3g" % (rows, e.max().item())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("size", [1, 52, 192, 1000])
def test_layer_norm_with_weight_and_bias(dtype, size):
    part = BuildEnv(DEV, DT[dtype]).build("norm", PartSpec("layer_norm", {"size": size, "eps": 1e-5, "tensor": "", "bias_tensor": ".b"}))
    w, b = 1.0 + 0.3 * torch.randn(size), 0.2 * torch.randn(size)
    part.load({"": w.to(DT[dtype]).to(DEV), ".b": b.to(DT[dtype]).to(DEV)})
    x = (3.0 + 2.0 * torch.randn(9, size)).to(DT[dtype])
    want = plain.layer_norm(x.float(), w.to(DT[dtype]).float(), b.to(DT[dtype]).float(), 1e-5)
    got = part.forward(x.to(DEV)).float().cpu()
    assert (got - want).abs().max().item() < (1e-4 if dtype == "float32" else 0.06)


# ---- whole models ----------------------------------------------------------------------------------------
_MODELS = {}
MAKERS = {"mixed": C.config_mixed, "ones": C.config_ones, "plain_residual": C.config_plain_residual,
          "parallel": lambda: C.config_single("parallel"), "retention": lambda: C.config_single("retention", streams=6)}


def model(name, tmp_path_factory):
    if name not in _MODELS:
        cfg = MAKERS[name]()
        w = C.weights(cfg, seed=11 + len(name), rank=1 if name == "ones" else 5)
        folder = C.write_folder(str(tmp_path_factory.mktemp("povipel_%s" % name)), cfg, w)
        _MODELS[name] = (cfg, w, folder, {})
    return _MODELS[name]


def engine(name, dtype, tmp_path_factory, max_tokens=4096, slots=8):
    cfg, w, folder, engines = model(name, tmp_path_factory)
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


def close(got, want, dtype, what=""):
    assert got.shape == want.shape, "%s: shapes %s and %s" % (what, tuple(got.shape), tuple(want.shape))
    got, want = got.float().cpu(), want.float().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.std().clamp_min(1e-6)
    assert torch.isfinite(e).all(), "%s: logits are not finite" % what
    if dtype == "float32":
        assert e.max().item() <= 3e-4, "%s: row error %.3g at row %d" % (what, e.max().item(), int(e.argmax()))
        return
    # bfloat16: a router whose two best scores are closer than rounding may send a token to another expert than the plain computation
    # does; such rows are few, and float32 (which runs the same kernels' indexing) is held to every row
    over = int((e > 0.12).sum())
    assert over <= max(1, e.numel() // 50) and e.max().item() <= 1.0, "%s: %d rows of %d over, the worst %.3g at row %d" % (what, over, e.numel(), e.max().item(), int(e.argmax()))


def plain_logits(cfg, w, toks):
    return plain.forward(cfg, C.as_float(w), toks)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "ones", "plain_residual"])
def test_whole_prompts_and_every_cut(name, dtype, tmp_path_factory):
    cfg, w, eng = engine(name, dtype, tmp_path_factory)
    assert eng.model.spec.architecture == "Povipel" and eng.model.graph_safe
    toks = C.tokens(200, cfg["vocab"], 5)
    layers = []
    want = plain.forward(cfg, C.as_float(w), toks, layers_out=layers)
    assert len(layers) == len(eng.model.spec.order) == len(plain.run_order(cfg))
    whole = run_cut(eng, toks, [])
    close(whole, want, dtype, "whole")
    close(whole[:3], want[:3], dtype, "the first tokens")
    for cuts in ([64], [63, 65], [1, 3, 128, 130], [150, 152, 154] + list(range(155, 200)), list(range(2, 200, 2)), list(range(1, 200))):
        got = run_cut(eng, toks, cuts)
        close(got, want, dtype, "cuts %s" % cuts[:4])
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
    want = [plain_logits(cfg, w, t) for t in reqs]
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
            close(got[off:off + heads[i]], want[i][:heads[i]], dtype, "prompt of %d in a batch" % i)
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
                close(got[k:k + 1], want[i][pos[i]:pos[i] + 1], dtype, "request %d decoded at %d" % (i, pos[i]))
                if dtype == "float32":
                    assert torch.equal(got[k], alone[i][pos[i]])
                pos[i] += 1
            for i in live:
                if pos[i] == len(reqs[i]):
                    eng.close(slots[i])
            live = [i for i in live if pos[i] < len(reqs[i])]
    eng.cache.check()


def attention_only(tmp_path_factory, window, pool, n_vocab=60):
    """One layer whose attention alone carries anything from token to token: the linear attention's output product is zero, nothing of
    the previous token is mixed in, one copy of the stream."""
    key = "edges_%d_%d" % (window, pool)
    if key not in _MODELS:
        cfg = C.config(n_vocab, 48, [(C.parallel(C.left(4, 2, 16, 12, window, pool, 8, base=100.0, scale=0.5), C.right(2, 8, 8)), C.dense(32))], streams=2, scale=3.0)
        f = C.as_float(C.weights(cfg, 21))
        f["l0.mix.right.o"].zero_()
        f["l0.shift"].zero_()
        w = {k: v.to(torch.bfloat16) for k, v in f.items()}
        _MODELS[key] = (cfg, w, C.write_folder(str(tmp_path_factory.mktemp("povipel_" + key)), cfg, w), {})
    return key


def logits_of(eng, tokens, how, n, head):
    if how == "prompt":
        return run_cut(eng, tokens, [])
    if how == "portions":
        return run_cut(eng, tokens, [61, 63, 130])
    return run_cut(eng, tokens, [head] + list(range(head + 1, n)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,pool", [(37, 6), (64, 8), (5, 16), (1, 1)])
def test_what_a_position_sees_through_the_window_and_the_blocks(window, pool, dtype, tmp_path_factory):
    """Changing the token at j changes the logits at i if and only if j lies in i's window or in a block that ends at or before
    i - window: keys just inside and just outside the window, in the block that is just seen and in the one that is not yet, at the
    sequence's start and at pages' borders; queries in a prompt, in a later portion, and decoded one by one."""
    cfg, w, eng = engine(attention_only(tmp_path_factory, window, pool), dtype, tmp_path_factory)
    n = 200
    toks = C.tokens(n, cfg["vocab"], 8)

    def sees(i, j):
        return 0 <= i - j < window or (j <= i and (j // pool) * pool + pool - 1 <= i - window)

    for how in ("prompt", "portions", "decoded"):
        base = logits_of(eng, toks, how, n, 120)
        close(base, plain_logits(cfg, w, toks), dtype, how)
        for i in (130, 191, 199):
            edge = i - window
            first_unseen = (edge + 1) // pool * pool          # the first position of the first block that is not yet seen
            for j in sorted({0, 1, 63, 64, 65, 127, 128, edge - 1, edge, edge + 1, edge + 2, first_unseen - 1, first_unseen, first_unseen + pool - 1, i - 1, i, i + 1}):
                if j < 0 or j >= n:
                    continue
                changed = list(toks)
                changed[j] = (toks[j] + 1 + j) % cfg["vocab"]
                got = logits_of(eng, changed, how, n, 120)[i]
                moved = (got - base[i]).abs().max().item()
                if sees(i, j):
                    assert moved > 0.0 or dtype == "bfloat16", "%s: query %d does not see the token at %d" % (how, i, j)
                else:
                    assert moved == 0.0, "%s: query %d sees the token at %d" % (how, i, j)


def test_one_key_far_away_in_a_pooled_block_carries_the_output(tmp_path_factory):
    """Two tokens have an element of the embedding to themselves; the keys of the one and the queries of the other read it with one and
    the same long vector, so that the block that holds this key (or, inside the window, the key itself) stands far above
    everything else the query sees: the output at the query is that block's value, wherever the token stands (in the first block, at a
    page's border, far back, in the last block that is seen, in the one that is not yet and is seen as a position), however the query
    comes (in the prompt or decoded)."""
    window, pool = 40, 2
    cfg = C.config(60, 32, [(C.parallel(C.left(2, 1, 64, 24, window, pool, 0, scale=0.5), C.right(1, 4, 4)), None)], streams=1, scale=1.0)
    n, special, asker = 330, 7, 11
    toks = [t if t not in (special, asker) else 20 for t in C.tokens(n, cfg["vocab"], 2)]
    f = C.as_float(C.weights(cfg, 4))
    # the two elements are zero for every other token, and stay zero through the layer norm because a row's other elements add up to nothing
    f["embed"][:, :2] = 0.0
    f["embed"][:, 2:] -= f["embed"][:, 2:].mean(1, keepdim=True)
    f["embed"][special, 0] = f["embed"][asker, 1] = 3.0
    for k in ("l0.norm1", "l0.hc1.in", "l0.hc1.out", "l0.hc1.mix", "l0.mix.left.q.norm", "l0.mix.left.k.norm"):
        f[k].fill_(1.0)
    f["l0.norm1.b"].zero_()
    f["l0.shift"].zero_()
    f["l0.mix.right.o"].zero_()
    f["l0.mix.left.sink"].fill_(-5.0)
    direction = torch.randn(64)
    f["l0.mix.left.k"][:, 0] = 6.0 * direction
    f["l0.mix.left.q"][:, 1] = 6.0 * direction.repeat(2)
    f["l0.mix.left.v"] = f["l0.mix.left.v"] * 3.0
    w = {k: v.to(torch.bfloat16) for k, v in f.items()}
    folder = C.write_folder(str(tmp_path_factory.mktemp("povipel_far")), cfg, w)
    for dtype in DTYPES:
        eng = Engine(Model.from_dir(folder, dtype=dtype), max_tokens=1024, max_slots=2)
        for place in (0, 1, 2, 63, 64, 128, 200, n - 1 - window - pool, n - 1 - window, n - window):
            seq = list(toks)
            seq[place], seq[n - 1] = special, asker
            want = plain_logits(cfg, w, seq)[-1:]
            other = list(seq)
            other[place] = 21
            assert C.row_errors(plain_logits(cfg, w, other)[-1:], want).item() > 0.2           # the one key matters
            close(run_cut(eng, seq, [])[-1:], want, dtype, "prompt, key at %d" % place)
            close(run_cut(eng, seq, [300] + list(range(301, n)))[-1:], want, dtype, "decoded, key at %d" % place)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["retention", "parallel"])
def test_a_state_carries_the_first_token_to_the_last(name, dtype, tmp_path_factory):
    """Far more tokens than any window: the first token still moves the last logits (through the decaying states), and the library
    agrees with the plain implementation there, in a prompt and after two hundred decoded tokens."""
    cfg, w, eng = engine(name, dtype, tmp_path_factory)
    n = 500
    toks = C.tokens(n, cfg["vocab"], 17)
    want = plain_logits(cfg, w, toks)
    other = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    assert (plain_logits(cfg, w, other)[-1] - want[-1]).abs().max().item() > 0.0
    close(run_cut(eng, toks, []), want, dtype, "prompt")
    close(run_cut(eng, toks, [300] + list(range(301, n))), want, dtype, "decoded")


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
            # float32 against the plain computation; bfloat16 (where rounding may send a token to another expert) against the engine's own
            # step function on the same tokens: the loop, the scheduler and the sampler add nothing of their own
            z = plain_logits(cfg, w, seq)[-1] if dtype == "float32" else run_cut(eng, seq, [])[-1].float().cpu()
            if int(z.argmax()) != t:        # a step whose two best logits are closer than rounding may go either way
                assert dtype == "bfloat16" and (z.max() - z[t]).item() < 0.05 * z.std().item(), "token %d of a prompt of %d" % (k, len(p))
            seq.append(t)
    again = generate(eng, prompts[::-1], params, eos_ids=(), max_batch=2)
    assert again[::-1] == out or dtype == "bfloat16"


@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_of_steps_and_the_command_line(dtype, tmp_path_factory):
    """bin/trace_run fed steps on standard input (a request whole, then its last tokens one by one beside a second request), and bin/tq
    generate on the same folder: logits and greedy tokens of the plain implementation."""
    import json
    import os
    import subprocess
    import sys
    from test_gpu_trace_run import Replay
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    cfg = C.config_plain_residual()
    w = C.weights(cfg, seed=77)
    folder = C.write_folder(str(tmp_path_factory.mktemp("povipel_replay")), cfg, w)
    a, b = C.tokens(150, cfg["vocab"], 1), C.tokens(9, cfg["vocab"], 2)
    want_a, want_b = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    r = Replay(folder, dtype, str(tmp_path_factory.mktemp("out")), max_tokens=64 * 6)
    got = r.step([("x", a, list(range(150)))], end=["x"])
    close(got.view(-1, cfg["vocab"]), want_a, dtype, "whole")
    assert r.step([("y", a[:140], []), ("z", b[:5], [])]) is None
    for t in range(10):
        live = [("y", [a[140 + t]], [0])] + ([("z", [b[5 + t]], [0])] if t < 4 else [])
        got = r.step(live, end=(["y"] if t == 9 else []) + (["z"] if t == 3 else [])).view(-1, cfg["vocab"])
        close(got[0:1], want_a[140 + t:141 + t], dtype, "one by one at %d" % t)
        if t < 4:
            close(got[1:2], want_b[5 + t:6 + t], dtype, "the second request at %d" % t)
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
        assert int(plain_logits(cfg, w, seq)[-1].argmax()) == t
        seq.append(t)
