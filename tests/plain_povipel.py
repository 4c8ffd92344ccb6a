"""A plain, slow implementation of the Povipel decoder, one function per mechanism.

Whole sequences, float32 (or a low dtype for products and their activations), no cache, no batching, every recurrence a
Python loop over the tokens.  It shares no code with the library; the GPU tests compare the library with it.

Notation: T tokens, D the model's width, S streams.

    X_0[s]   = c E[t] for every stream s                       (c the embedding's scale)
    sublayer:  u = sum_s a[s] X[s];  y = part(LN(u));  X'[t] = sum_s M[s, t] X[s] + b[t] y       (a, M, b per sublayer)
               the first sublayer of a layer is its mixer, the second its feed-forward (which may be absent)
    without streams: x' = x + part(LN(x))
    LN(u)    = (u - mean) / sqrt(var + eps) w + beta
    shift:     what a mixer reads is n_t + (n_(t-1) - n_t) mu with n = LN(u) and n_(-1) = 0
    a span of layers [start, stop) runs `times` times with the same weights
    logits   = cap tanh(H LN_final(sum_s X[s]) / cap)

Mixers:

    windowed attention with pooled blocks ("left")
               q, k, v = W h;  q and k heads are divided by their root mean square and multiplied by a weight, then their first
               r elements are turned pair by pair, (e_2i, e_2i+1) by p base^(-2i/r);  v of position j is turned by j over all its
               elements, pair m by j base^(-2m/dv);  position i sees the positions j with 0 <= i - j < W and, for every block
               of P positions that ends at or before i - W, one key and value that are the means of the block's;  the softmax's
               denominator also holds exp(sink_h);  the head's output is turned back by -i
    gated linear attention ("right")
               q = W_q h / sqrt(d), k = W_k h, v = W_v h;  alpha = sigmoid(W_a2 W_a1 h + b)^(1/tau) per key channel;
               S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  o is normed per head with a weight, times silu(W_g h), W_o
    parallel   (n_l(left(h)) + n_r(right(h))) / 2 with n an RMS norm over the width with a weight
    retention  q, k turned in halves (e_i with e_(i + r/2)), k / sqrt(d);  S_t = g_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t;  o is
               divided per head by its root mean square, times silu(W_g h), W_o

Feed-forwards: dense W_down gelu_tanh(W_up h); experts: s = sigmoid(W_r h), the `top` largest are chosen, the output is
sum_e E_e(s_e h) with E(z) = W_down (silu(W_gate z) * (W_up z)).

A weight dict maps the checkpoint's tensor names to float32 tensors (the bfloat16 values exactly).  `low` names the dtype
the products are rounded to (float32: nothing is).
"""
import math

import torch

F32 = torch.float32


def rnd(x, low):
    return x if low == F32 else x.to(low).to(F32)


def product(x, w, low):
    return rnd(rnd(x, low) @ w.T, low)


def layer_norm(x, w, b, eps):
    m = x.mean(-1, keepdim=True)
    d = x - m
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def unit_norm(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def angles(positions, base, dims):
    """[T, dims / 2]: position * base^(-2i/dims)"""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    return (positions.to(torch.float64)[:, None] * f[None, :]).to(F32)


def turn(v, ang, layout):
    """v [T, heads, d]; the first 2 * ang.shape[1] elements of each head are turned by ang [T, n]; layout 'pairs' joins 2i with
    2i + 1, 'halves' i with i + n."""
    n = ang.shape[1]
    if n == 0:
        return v
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = v.clone()
    if layout == "pairs":
        a, b = v[..., 0:2 * n:2], v[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = a * c - b * s
        out[..., 1:2 * n:2] = b * c + a * s
    else:
        a, b = v[..., :n], v[..., n:2 * n]
        out[..., :n] = a * c - b * s
        out[..., n:2 * n] = b * c + a * s
    return out


def token_shift(n, mu):
    prev = torch.cat([torch.zeros_like(n[:1]), n[:-1]], 0)
    return n + (prev - n) * mu


def pooled_window_attention(q, k, v, scale, window, pool, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv] as the cache holds them -> [T, H, dv].  A loop over the positions."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F32)
    n_blocks = T // pool
    kb = k[:n_blocks * pool].reshape(n_blocks, pool, G, -1).mean(1) if n_blocks else k[:0]
    vb = v[:n_blocks * pool].reshape(n_blocks, pool, G, -1).mean(1) if n_blocks else v[:0]
    for i in range(T):
        lo = max(0, i - window + 1)
        seen = sum(1 for b in range(n_blocks) if b * pool + pool - 1 <= i - window)
        for h in range(H):
            g = h // (H // G)
            keys = torch.cat([kb[:seen, g], k[lo:i + 1, g]], 0)
            vals = torch.cat([vb[:seen, g], v[lo:i + 1, g]], 0)
            s = (keys @ q[i, h]) * scale
            m = torch.maximum(s.max(), sink[h]) if sink is not None else s.max()
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e / den) @ vals
    return out


def left_attention(h, w, p, m, eps, positions, low):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = product(h, w[p + "q"], low).view(T, H, d)
    k = product(h, w[p + "k"], low).view(T, G, d)
    v = product(h, w[p + "v"], low).view(T, G, dv)
    q = unit_norm(q, eps) * w[p + "q.norm"]
    k = unit_norm(k, eps) * w[p + "k.norm"]
    ang = angles(positions, m["rot"]["base"], m["rot"]["dims"])
    q, k = turn(q, ang, "pairs"), turn(k, ang, "pairs")
    vang = angles(positions, m["rot"]["base"], dv)
    v = turn(v, vang, "pairs")
    q, k, v = rnd(q, low), rnd(k, low), rnd(v, low)
    o = pooled_window_attention(q, k, v, m["scale"], m["mask"]["size"], m["mask"]["pool"], w[p + "sink"])
    o = turn(o, -vang, "pairs")
    return product(o.reshape(T, H * dv), w[p + "o"], low)


def decayed_state_attention(q, k, v, decay):
    """S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k [T, H, d], v [T, H, dv], decay [T, H, d]."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F32)
    out = torch.zeros(T, H, v.shape[2], dtype=F32)
    for t in range(T):
        S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def right_attention(h, w, p, m, eps, low):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = product(h, w[p + "q"], low).view(T, H, d) * d ** -0.5
    k = product(h, w[p + "k"], low).view(T, H, d)
    v = product(h, w[p + "v"], low).view(T, H, dv)
    z = product(product(h, w[p + "a1"], low), w[p + "a2"], low) + w[p + "a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / m["tau"]).view(T, H, d)
    o = decayed_state_attention(q, k, v, alpha)
    o = unit_norm(o, eps) * w[p + "norm"]
    o = rnd(o.reshape(T, H * dv), low) * silu(product(h, w[p + "g"], low))
    return product(o, w[p + "o"], low)


def parallel(h, w, p, m, eps, positions, low):
    a = left_attention(h, w, p + "left.", m["left"], eps, positions, low)
    b = right_attention(h, w, p + "right.", m["right"], eps, low)
    return 0.5 * (unit_norm(a, eps) * w[p + "left.out"] + unit_norm(b, eps) * w[p + "right.out"])


def retention(h, w, p, m, eps, positions, low):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = product(h, w[p + "q"], low).view(T, H, d)
    k = product(h, w[p + "k"], low).view(T, H, d)
    v = product(h, w[p + "v"], low).view(T, H, dv)
    ang = angles(positions, m["rot"]["base"], m["rot"]["dims"])
    q, k = turn(q, ang, "halves"), turn(k, ang, "halves") * d ** -0.5
    decay = torch.tensor(m["decay"], dtype=F32)[None, :, None].expand(T, H, d)
    o = unit_norm(decayed_state_attention(q, k, v, decay), eps)
    o = rnd(o.reshape(T, H * dv), low) * silu(product(h, w[p + "g"], low))
    return product(o, w[p + "o"], low)


def dense_ff(h, w, p, low):
    return product(rnd(gelu_tanh(product(h, w[p + "up"], low)), low), w[p + "down"], low)


def experts_ff(h, w, p, mlp, low):
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.sigmoid(h @ w[p + "router"].T)
    chosen = torch.topk(s, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            z = (s[t, e] * h[t])[None]
            a = rnd(silu(product(z, w[p + f"e{e}.gate"], low)) * product(z, w[p + f"e{e}.up"], low), low)
            out[t] += product(a, w[p + f"e{e}.down"], low)[0]
    return out


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    span = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + span * loop["times"] + list(range(loop["stop"], n))


def mixer(layer, h, w, p, eps, positions, low):
    if layer["type"] == "parallel":
        return parallel(h, w, p, layer["mixer"], eps, positions, low)
    if layer["type"] == "retention":
        return retention(h, w, p, layer["mixer"], eps, positions, low)
    raise ValueError(layer["type"])


def feed_forward(layer, h, w, p, low):
    if layer["mlp"]["kind"] == "dense":
        return dense_ff(h, w, p, low)
    return experts_ff(h, w, p, layer["mlp"], low)


def forward(cfg, w, tokens, low=F32, layers_out=None):
    """tokens: a list of ids; returns logits [T, vocab] in float32.  layers_out: a list that receives the stream (the sum of
    the streams) after every run of a layer."""
    T = len(tokens)
    eps = cfg["norm"]["eps"]
    positions = torch.arange(T)
    x0 = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    S = cfg.get("streams")
    X = x0[None].repeat(S, 1, 1) if S else x0

    def sublayer(X, pre, hc, norm, part, shift=None):
        u = torch.einsum("s,std->td", w[pre + hc + ".in"], X) if S else X
        n = layer_norm(u, w[pre + norm], w[pre + norm + ".b"], eps)
        if shift is not None:
            n = token_shift(n, shift)
        y = part(rnd(n, low))
        if S:
            return torch.einsum("sr,std->rtd", w[pre + hc + ".mix"], X) + w[pre + hc + ".out"][:, None, None] * y[None]
        return X + y

    for li in run_order(cfg):
        layer, pre = cfg["layers"][li], f"l{li}."
        X = sublayer(X, pre, "hc1", "norm1", lambda h: mixer(layer, h, w, pre + "mix.", eps, positions, low), w[pre + "shift"])
        if layer["mlp"] is not None:
            X = sublayer(X, pre, "hc2", "norm2", lambda h: feed_forward(layer, h, w, pre + "mlp.", low))
        if layers_out is not None:
            layers_out.append(X.sum(0) if S else X.clone())
    x = X.sum(0) if S else X
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    logits = product(x, w["head"], low)
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
