"""Shared by the Piditar tests: small configurations made here, random weights of a sensible size, model folders written
with the safetensors package, and how logits are compared."""
import json
import math
import os

import torch
from safetensors.torch import save_file

import plain_piditar as plain


def attention(heads, kv_heads, dim, vdim, rot_dims, base=10000.0, scale=None, softcap=20.0):
    return ("attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": rot_dims},
                          "scale": scale if scale is not None else 1.0 / math.sqrt(dim), "softcap": softcap})


def rglru(width, blocks, conv):
    return ("rglru", {"width": width, "blocks": blocks, "conv": conv})


def mamba2(heads, vdim, state, groups, conv, norm_groups):
    return ("mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups})


def config(vocab, width, layers, loop=None, eps=1e-5, scale=4.0):
    """layers: ((type, mixer), ff or None) pairs; loop: (start, stop, times) or None for a configuration without the key."""
    c = {"architecture": "Piditar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
         "layers": [{"type": t, "mixer": m, "mlp": None if f is None else {"kind": "dense", "ff": f}} for (t, m), f in layers]}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


# Sizes chosen away from each other: a looped span in the middle that runs three times, a layer before and one after it, a layer
# without a feed-forward, heads in groups, values larger and smaller than keys, part of a head rotated, convolutions of 2 to 5 taps.
def config_mixed():
    return config(331, 96, [(rglru(80, 5, 4), 72), (attention(6, 3, 24, 40, 16, base=5000.0), 56), (mamba2(6, 20, 24, 3, 3, 4), None),
                            (rglru(64, 2, 2), 40), (mamba2(4, 16, 40, 1, 5, 1), 88), (attention(4, 1, 32, 16, 32, base=300.0, softcap=7.0), 64)],
                  loop=(1, 4, 3), eps=3e-6, scale=7.5)


# The smallest of everything: one head, one group, one block, a convolution of one tap (no inputs kept), a state of one row,
# two rotated elements, a span of one layer that runs once.
def config_ones():
    return config(67, 32, [(attention(1, 1, 8, 8, 2, base=2.0, softcap=1.0), 16), (rglru(8, 1, 1), 16), (mamba2(1, 8, 1, 1, 1, 1), None)],
                  loop=(1, 2, 1), eps=1e-4, scale=1.0)


# Sizes that are no multiples of 8; every layer inside the span, twice; as many groups as heads; no rotation in one layer.
def config_odd():
    return config(101, 52, [(mamba2(3, 14, 10, 3, 4, 3), 44), (attention(3, 3, 10, 14, 6, base=777.0, softcap=9.0), None), (rglru(36, 3, 3), 20),
                            (attention(6, 2, 12, 12, 0, softcap=50.0), 28)], loop=(0, 4, 2), eps=1e-5, scale=3.0)


# One layer of one kind and a configuration without a loop.
def config_single(kind, width=64):
    # ("attention_equal": keys and values of one size, which the plain prompt kernel takes with the cap as an option)
    mix = {"attention": attention(4, 2, 16, 24, 8, base=50.0, scale=1.0, softcap=30.0),
           "attention_equal": attention(6, 2, 32, 32, 12, base=50.0, scale=0.7, softcap=30.0), "rglru": rglru(48, 3, 4), "mamba2": mamba2(4, 12, 16, 2, 4, 2)}[kind]
    return config(97, width, [(mix, 48)], scale=5.0)


def weights(cfg, seed, store=torch.bfloat16, memory="some"):
    """name -> tensor of the store dtype.  Products keep the size of what they read (std 1/sqrt(inputs)).  memory "none": the
    recurrences' decays are driven to zero, so that a token's output depends on the convolution's reach alone; "long": decays
    close to one, so that the state holds a token for hundreds of positions."""
    forgetful, lasting = memory == "none", memory == "long"
    g = torch.Generator().manual_seed(seed)

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(store)

    def vec(n, around=0.0, spread=0.1):
        return (around + spread * torch.randn(n, generator=g)).to(store)

    D = cfg["width"]
    w = {"embed": lin(cfg["vocab"], D, math.sqrt(D) / cfg["embedding"]["scale"] * 1.0), "final.norm": vec(D)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f, kind = "l%d." % i, layer["mixer"], layer["mlp"], layer["type"]
        w[p + "norm1"] = vec(D)
        q = p + "mix."
        if kind == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                w[q + n] = lin(rows, D)
                w[q + n + ".b"] = vec(rows, 0.0, 0.3)
            w[q + "o"] = lin(D, H * dv)
        elif kind == "rglru":
            W, nb = m["width"], m["blocks"]
            bs = W // nb
            for n in ("y", "x"):
                w[q + n] = lin(W, D)
                w[q + n + ".b"] = vec(W, 0.0, 0.3)
            w[q + "conv"] = (torch.randn(W, m["conv"], generator=g) * 0.5).to(store)
            w[q + "conv.b"] = vec(W, 0.0, 0.2)
            for n in ("ra", "ri"):
                w[q + n] = (torch.randn(nb, bs, bs, generator=g) / math.sqrt(bs)).to(store)
                w[q + n + ".b"] = (0.5 * torch.randn(nb, bs, generator=g)).to(store)
            if forgetful:
                w[q + "ra.b"] = w[q + "ra.b"] + 12.0            # r is 1 but for rounding, whatever the input
            w[q + "lam"] = vec(W, 40.0 if forgetful else -6.0 if lasting else -2.0, 1.0 if not lasting else 0.3)
            w[q + "o"] = lin(D, W)
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * P, H * P + 2 * G * N
            w[q + "in"] = lin(2 * inner + 2 * G * N + H, D)
            w[q + "conv"] = (torch.randn(ch, m["conv"], generator=g) * 0.5).to(store)
            w[q + "conv.b"] = vec(ch, 0.0, 0.2)
            w[q + "dt_bias"] = vec(H, 30.0 if forgetful else -3.0 if lasting else -1.0, 0.5)
            w[q + "A_log"] = vec(H, 2.0 if forgetful else -2.0 if lasting else -0.5, 0.5)
            w[q + "D"] = vec(H, 1.0, 0.3)
            w[q + "norm"] = vec(inner, 1.0, 0.1)
            w[q + "o"] = lin(D, inner)
        if f is None:
            continue
        w[p + "norm2"] = vec(D)
        for n, (o, k) in {"gate": (f["ff"], D), "up": (f["ff"], D), "down": (D, f["ff"])}.items():
            w[p + "mlp." + n] = lin(o, k)
    return w


def write_folder(path, cfg, w):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def as_float(w):
    return {k: v.to(torch.float32) for k, v in w.items()}


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def row_errors(got, want):
    """Per row: root mean square of the difference (means taken off), over the spread of the wanted logits."""
    got, want = got.float().cpu(), want.float().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.std().clamp_min(1e-6)


def close(got, want, dtype, what=""):
    """float32: every row within 2e-4 of the spread (the recurrences add rounding of their own over hundreds of tokens).
    bfloat16: every row within 0.1 of it."""
    assert got.shape == want.shape, "%s: shapes %s and %s" % (what, tuple(got.shape), tuple(want.shape))
    e = row_errors(got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1]))
    assert torch.isfinite(e).all(), "%s: logits are not finite" % what
    limit = 2e-4 if dtype == "float32" else 0.1
    assert e.max().item() <= limit, "%s: row error %.3g" % (what, e.max().item())


def plain_logits(cfg, w, toks, low=torch.float32):
    return plain.forward(cfg, as_float(w), toks, low)
