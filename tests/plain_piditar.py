"""A plain, slow implementation of the Piditar decoder, one function per mechanism.

Whole sequences, float32 (or a low dtype for products and their activations), no cache, no batching, every
recurrence a Python loop over the tokens.  It shares no code with the library; the GPU tests compare the library with it.

Notation: T tokens, D the model's width.

    x_0      = s E[t]                                          (s the embedding's scale; E doubles as the head)
    layer:     x = x + mix(n1(x));  x = x + ff(n2(x))          (ff may be absent)
    n(x)     = x / sqrt(mean(x^2) + eps) (1 + w)
    ff(h)    = W_down (silu(W_gate h) * (W_up h))
    a span of layers [start, stop) runs `times` times with the same weights; from the second pass on x_0 is added to x
    right before the pass's first layer
    logits   = E n_final(x)

The three mixers:

    attention  q, k, v = W h + b;  the first r elements of every q and k head are turned pair by pair, (e_2i, e_2i+1) by the
               angle p base^(-2i/r);  then q and k heads are divided by their root mean square;  s_ij = c tanh(scale q_i.k_j / c)
               over j <= i, softmax, times v;  W_o on the heads side by side
    rglru      y = gelu_tanh(W_y h + b_y);  u = conv(W_x h + b_x);  per diagonal block r = sigmoid(A u + b_a), i = sigmoid(B u + b_i);
               a = exp(-8 r softplus(lam));  S_t = a S_(t-1) + sqrt(1 - a^2) (i u);  W_o (S y)
    mamba2     [z | x | B | C | dt] = W_in h;  (x, B, C) = silu(conv(x, B, C));  dt = softplus(dt + dt_bias);
               per head S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T,  y_t = S_t^T C_t + D x_t;
               v = y silu(z), divided part by part by its root mean square, times w;  W_o v
    conv       out_t[c] = b[c] + sum_k w[c][k] in_(t - (taps - 1 - k))[c], zeros before the sequence

A weight dict maps the checkpoint's tensor names to float32 tensors (the bfloat16 values exactly).  `low` names the
dtype the products are rounded to (float32: nothing is).
"""
import math

import torch

F32 = torch.float32
DECAY_SCALE = 8.0


def rnd(x, low):
    return x if low == F32 else x.to(low).to(F32)


def product(x, w, low, bias=None):
    """x W^T with operands of the low dtype and float32 sums, rounded to the low dtype; a bias is added after that, in float32."""
    y = rnd(rnd(x, low) @ w.T, low)
    return y if bias is None else y + bias


def unit_norm(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    return unit_norm(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def turn_pairs(v, positions, base, dims):
    """v [T, heads, d]: elements 2i and 2i + 1 (i < dims / 2) are turned by the angle position * base^(-2i/dims)."""
    if dims == 0:
        return v
    out = v.clone()
    for i in range(dims // 2):
        ang = positions.to(F32) * torch.pow(torch.tensor(float(base), dtype=F32), torch.tensor(-2.0 * i / dims, dtype=F32))
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        a, b = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def causal_softmax_attention(q, k, v, scale, cap):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; scores and weights in float32."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F32)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            s = (k[:i + 1, g] @ q[i, h]) * scale
            if cap is not None:
                s = cap * torch.tanh(s / cap)
            out[i, h] = torch.softmax(s, 0) @ v[:i + 1, g]
    return out


def attention(h, w, p, m, eps, positions, low):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = product(h, w[p + "q"], low, w[p + "q.b"]).reshape(T, H, d)
    k = product(h, w[p + "k"], low, w[p + "k.b"]).reshape(T, G, d)
    v = product(h, w[p + "v"], low, w[p + "v.b"]).reshape(T, G, dv)
    q = unit_norm(turn_pairs(q, positions, m["rot"]["base"], m["rot"]["dims"]), eps)
    k = unit_norm(turn_pairs(k, positions, m["rot"]["base"], m["rot"]["dims"]), eps)
    o = causal_softmax_attention(rnd(q, low), rnd(k, low), rnd(v, low), m["scale"], m.get("softcap"))
    return product(o.reshape(T, H * dv), w[p + "o"], low)


def short_conv(x, w, b):
    """x [T, C], w [C, taps] whose last column weighs the token itself, b [C]."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F32)
    for t in range(T):
        acc = b.clone()
        for k in range(taps):
            src = t - (taps - 1 - k)
            if src >= 0:
                acc = acc + w[:, k] * x[src]
        out[t] = acc
    return out


def rglru(h, w, p, m, low):
    width, blocks = m["width"], m["blocks"]
    bs = width // blocks
    y = gelu_tanh(product(h, w[p + "y"], low, w[p + "y.b"]))
    u = short_conv(product(h, w[p + "x"], low, w[p + "x.b"]), w[p + "conv"], w[p + "conv.b"])
    decay = DECAY_SCALE * torch.nn.functional.softplus(w[p + "lam"])
    S = torch.zeros(width, dtype=F32)
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        r = torch.zeros(width, dtype=F32)
        g = torch.zeros(width, dtype=F32)
        for b in range(blocks):
            part = u[t, b * bs:(b + 1) * bs]
            r[b * bs:(b + 1) * bs] = torch.sigmoid(w[p + "ra"][b] @ part + w[p + "ra.b"][b])
            g[b * bs:(b + 1) * bs] = torch.sigmoid(w[p + "ri"][b] @ part + w[p + "ri.b"][b])
        a = torch.exp(-decay * r)
        S = a * S + torch.sqrt(1.0 - a * a) * (g * u[t])
        out[t] = S
    return product(out * y, w[p + "o"], low)


def mamba2(h, w, p, m, eps, low):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    every = product(h, w[p + "in"], low)
    z, rest, dt = every[:, :inner], every[:, inner:2 * inner + 2 * G * N], every[:, 2 * inner + 2 * G * N:]
    rest = silu(short_conv(rest, w[p + "conv"], w[p + "conv.b"]))
    x = rest[:, :inner].reshape(T, H, P)
    B = rest[:, inner:inner + G * N].reshape(T, G, N)
    C = rest[:, inner + G * N:].reshape(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[p + "dt_bias"])
    rate = torch.exp(w[p + "A_log"])
    S = torch.zeros(H, N, P, dtype=F32)
    y = torch.zeros(T, H, P, dtype=F32)
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = torch.exp(-rate[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + w[p + "D"][hd] * x[t, hd]
    v = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    v = unit_norm(v.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return product(v, w[p + "o"], low)


def dense_ff(h, w, p, low):
    return product(silu(product(h, w[p + "gate"], low)) * product(h, w[p + "up"], low), w[p + "down"], low)


def run_order(cfg):
    """(layer, whether the embedding's output is added in front of it) for every run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    order = [(i, False) for i in range(loop["start"])]
    for turn in range(loop["times"]):
        order += [(i, turn > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def mixer(kind, h, w, p, m, eps, positions, low):
    if kind == "attention":
        return attention(h, w, p, m, eps, positions, low)
    if kind == "rglru":
        return rglru(h, w, p, m, low)
    return mamba2(h, w, p, m, eps, low)


def forward(cfg, w, tokens, low=F32, layers_out=None):
    """Logits [T, vocab] of one sequence from its first token."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][tokens] * cfg["embedding"]["scale"]
    x = x0.clone()
    positions = torch.arange(tokens.shape[0])
    for i, again in run_order(cfg):
        if again:
            x = x + x0
        layer = cfg["layers"][i]
        p = "l%d." % i
        x = x + mixer(layer["type"], rnd(offset_norm(x, w[p + "norm1"], eps), low), w, p + "mix.", layer["mixer"], eps, positions, low)
        if layer.get("mlp"):
            x = x + dense_ff(rnd(offset_norm(x, w[p + "norm2"], eps), low), w, p + "mlp.", low)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rnd(offset_norm(x, w["final.norm"], eps), low) @ w["embed"].T
