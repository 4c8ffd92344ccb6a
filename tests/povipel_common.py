"""Shared by the Povipel tests: small configurations made here, random weights of a sensible size, model folders written with the
safetensors package, and how logits are compared."""
import json
import math
import os

import torch
from safetensors.torch import save_file


def left(heads, kv_heads, dim, vdim, window, pool, rot_dims, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window, "pool": pool},
            "rot": {"base": base, "dims": rot_dims}, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}


def right(heads, dim, vdim, tau=8.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}


def parallel(l, r):
    return ("parallel", {"left": l, "right": r})


def retention(heads, dim, vdim, rot_dims, base=10000.0, decay=None):
    return ("retention", {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": rot_dims},
                          "decay": decay if decay is not None else [1.0 - 2.0 ** (-3 - h) for h in range(heads)]})


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(vocab, width, layers, streams=3, loop=None, eps=1e-5, scale=4.0, softcap=25.0, rank=None):
    """layers: ((type, mixer), mlp or None) pairs; loop: (start, stop, times) or None for a configuration without the key;
    streams None: a configuration without the key (a plain residual sum); rank: of the decay's low-rank product (not a key of
    the configuration: the tensors' shapes give it)."""
    c = {"architecture": "Povipel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
         "layers": [{"type": t, "mixer": m, "mlp": f} for (t, m), f in layers]}
    if streams is not None:
        c["streams"] = streams
    if softcap is not None:
        c["logit_softcap"] = softcap
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


# Sizes chosen away from each other: a looped span that runs three times with a layer before and after it, a layer without a
# feed-forward, heads in groups, values larger and smaller than keys, part of a head turned, a window that is no multiple of the
# pooled block, a block that does not divide the page, two experts a token.
def config_mixed():
    return config(331, 96, [
        (parallel(left(6, 3, 24, 40, 37, 6, 16, base=5000.0, scale=0.3), right(3, 20, 12, tau=5.0)), dense(72)),
        (retention(3, 24, 20, 16, base=300.0), moe(40, 5, 2)),
        (parallel(left(4, 1, 32, 16, 50, 16, 32, base=777.0), right(4, 8, 24, tau=16.0)), None),
        (retention(2, 40, 36, 40, base=1e6), moe(24, 7, 3)),
        (parallel(left(2, 2, 16, 16, 20, 4, 8), right(2, 16, 16)), moe(32, 4, 1)),
    ], streams=3, loop=(1, 4, 3), eps=3e-6, scale=7.5, softcap=18.0)


# The smallest of everything: one stream, one head, one group, a window of one position, blocks of one position, a rank of one, one
# expert of which one is chosen, two turned elements, a span of one layer that runs once, nothing that is turned in the retention.
def config_ones():
    return config(67, 32, [(parallel(left(1, 1, 8, 2, 1, 1, 2, base=2.0), right(1, 1, 1, tau=1.0)), moe(8, 1, 1)),
                           (retention(1, 2, 1, 0, decay=[0.5]), dense(16))], streams=1, loop=(1, 2, 1), eps=1e-4, scale=1.0, softcap=None)


# No streams at all (the plain residual sum), sizes that are no multiples of 8, every layer inside the span, twice.
def config_plain_residual():
    return config(101, 52, [(retention(3, 10, 14, 6, base=777.0), dense(44)),
                            (parallel(left(3, 3, 10, 14, 9, 3, 6), right(2, 6, 10, tau=3.0)), moe(20, 3, 2))], streams=None, loop=(0, 2, 2), scale=3.0)


def config_single(kind, width=64, streams=2):
    mix = {"parallel": parallel(left(4, 2, 16, 24, 24, 8, 8, base=50.0, scale=0.4), right(2, 12, 20, tau=4.0)),
           "retention": retention(3, 12, 20, 8, base=50.0)}[kind]
    return config(97, width, [(mix, dense(48))], streams=streams, scale=5.0)


def weights(cfg, seed, store=torch.bfloat16, rank=5):
    """name -> tensor of the store dtype.  Products keep the size of what they read (std 1/sqrt(inputs))."""
    g = torch.Generator().manual_seed(seed)

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(store)

    def vec(n, around=0.0, spread=0.1):
        return (around + spread * torch.randn(n, generator=g)).to(store)

    D, S = cfg["width"], cfg.get("streams")
    w = {"embed": lin(cfg["vocab"], D, math.sqrt(D) / cfg["embedding"]["scale"]), "head": lin(cfg["vocab"], D, 3.0),
         "final.norm": vec(D, 1.0), "final.norm.b": vec(D)}
    for i, layer in enumerate(cfg["layers"]):
        p, m, f = "l%d." % i, layer["mixer"], layer["mlp"]
        for q in (1, 2) if f is not None else (1,):
            w[p + "norm%d" % q] = vec(D, 1.0)
            w[p + "norm%d.b" % q] = vec(D)
            if S is not None:
                w[p + "hc%d.in" % q] = vec(S, 1.0 / S, 0.2)
                w[p + "hc%d.out" % q] = vec(S, 1.0, 0.3)
                w[p + "hc%d.mix" % q] = (torch.eye(S) + 0.2 * torch.randn(S, S, generator=g)).to(store)
        w[p + "shift"] = vec(D, 0.4, 0.3)
        x = p + "mix."
        if layer["type"] == "parallel":
            a, b = m["left"], m["right"]
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            w.update({x + "left.q": lin(H * d, D), x + "left.k": lin(G * d, D), x + "left.v": lin(G * dv, D), x + "left.o": lin(D, H * dv),
                      x + "left.q.norm": vec(d, 1.0, 0.2), x + "left.k.norm": vec(d, 1.0, 0.2), x + "left.sink": vec(H, 0.0, 1.0),
                      x + "left.out": vec(D, 1.0), x + "right.out": vec(D, 1.0)})
            H, d, dv = b["heads"], b["dim"], b["vdim"]
            w.update({x + "right.q": lin(H * d, D), x + "right.k": lin(H * d, D), x + "right.v": lin(H * dv, D), x + "right.g": lin(H * dv, D),
                      x + "right.o": lin(D, H * dv), x + "right.norm": vec(dv, 1.0), x + "right.a1": lin(rank, D), x + "right.a2": lin(H * d, rank, 2.0),
                      x + "right.a2.b": vec(H * d, 2.0, 1.0)})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            w.update({x + "q": lin(H * d, D), x + "k": lin(H * d, D), x + "v": lin(H * dv, D), x + "g": lin(H * dv, D), x + "o": lin(D, H * dv)})
        if f is None:
            continue
        y = p + "mlp."
        if f["kind"] == "dense":
            w.update({y + "up": lin(f["ff"], D), y + "down": lin(D, f["ff"])})
        else:
            w[y + "router"] = lin(f["router"]["experts"], D, 2.0)
            for e in range(f["router"]["experts"]):
                w.update({y + "e%d.gate" % e: lin(f["expert"]["ff"], D), y + "e%d.up" % e: lin(f["expert"]["ff"], D), y + "e%d.down" % e: lin(D, f["expert"]["ff"])})
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
    """Per row: the root mean square of the difference over that of the wanted row."""
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    return torch.sqrt(((got - want) ** 2).mean(-1)) / torch.sqrt((want ** 2).mean(-1) + 1e-12)
