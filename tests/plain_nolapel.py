"""The Nolapel design in plain float64: one function per mechanism, whole sequences, token by token
where the design is a recurrence.  Slow on purpose; shares no code with the engine.

Notation: x [T, d] the stream, n the normed stream that a mixer reads, W the weights by checkpoint name
(float64), positions 0 .. T-1, cfg the dict that config.json holds.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def dyt(x, W, name):
    """The tanh norm: tanh(alpha x) * w + b, element by element."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


# ------------------------------------------------------------------ embedding
def bigram_rows(tokens, bg):
    """Row of the bigram table for every token: a hash of (previous, current), the last row for the first."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(bg["buckets"] if t == 0 else (tokens[t - 1] * bg["mul_prev"] + tok * bg["mul_cur"]) % bg["buckets"])
    return rows


def embedding(tokens, W, cfg):
    x = W["embed"][torch.tensor(tokens)]
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + W["bigram"][torch.tensor(bigram_rows(list(tokens), bg))]
    return x


# ------------------------------------------------------------------ short convolution over time
def causal_conv(u, w, bias=None):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start.  u [T, C], w [C, taps]."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y if bias is None else y + bias


# ------------------------------------------------------------------ softmax attention
def softmax_attention(q, k, v, scale, sink=None, window=None, slopes=None):
    """q [T, H, D], k [T, G, D], v [T, G, V].  Query i reads keys j <= i (with ``window``: i - j < window);
    score = q.k * scale - slope_h (i - j); the denominator holds exp(sink_h) beside the keys' terms."""
    T, H, D = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    seen = (j <= i) if window is None else ((j <= i) & (i - j < window))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if slopes is not None:
            s = s - slopes[h] * (i - j).to(F64)
        s = s.masked_fill(~seen, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].expand_as(m))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def conv_attention(n, W, p, mx, eps):
    """The 'attention' mixer: convolved q and k, values = keys before their norm, a head norm, a query
    temperature that grows with the position, a distance bias, a window, a sink of score 0."""
    T = n.shape[0]
    H, G, D = mx["heads"], mx["kv_heads"], mx["dim"]
    q, k = n @ W[p + "q"].T, n @ W[p + "k"].T
    if mx.get("conv"):
        q, k = causal_conv(q, W[p + "q.conv"]), causal_conv(k, W[p + "k.conv"])
    v = k.view(T, G, D)
    q = unit_rms(q.view(T, H, D), eps) * W[p + "q.norm"]
    k = unit_rms(k.view(T, G, D), eps) * W[p + "k.norm"]
    qt = mx.get("q_temp")
    if qt:
        pos = torch.arange(T)
        q = q * (1.0 + qt["coef"] * torch.log(torch.floor((pos + 1) / qt["every"]).to(F64) + 1.0)).view(T, 1, 1)
    slopes = [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]
    window = (mx.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, mx["scale"], sink=torch.zeros(H, dtype=F64), window=window, slopes=slopes)
    return o.reshape(T, -1) @ W[p + "o"].T


def rotate_halves(x, rot):
    """x [T, heads, D]: the first ``dims`` elements of a head turn, element i with element i + dims/2."""
    if not rot:
        return x
    dims, base = rot["dims"], rot["base"]
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = torch.arange(T, dtype=F64).view(T, 1, 1) * f
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def sink_attention(n, W, p, mx):
    """The left half of the 'parallel' mixer: rotated q and k, every earlier key, a learned sink a head."""
    T = n.shape[0]
    H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = rotate_halves((n @ W[p + "q"].T).view(T, H, D), mx.get("rot"))
    k = rotate_halves((n @ W[p + "k"].T).view(T, G, D), mx.get("rot"))
    v = (n @ W[p + "v"].T).view(T, G, V)
    o = softmax_attention(q, k, v, mx["scale"], sink=W[p + "sink"])
    return o.reshape(T, -1) @ W[p + "o"].T


# ------------------------------------------------------------------ time mixing with a decayed state
def time_mix(n, W, p, mx, eps):
    """The right half: every projection reads its own blend of the row and the row before; per head
    o_t = (S + diag(u) k_t v_t^T)^T r_t, then S <- diag(w_t) S + k_t v_t^T."""
    T, d = n.shape
    H, D = mx["heads"], mx["dim"]
    before = torch.cat([torch.zeros(1, d, dtype=F64), n[:-1]], 0)
    blend = {s: n + (before - n) * W[p + "mu." + s] for s in "rkvgw"}
    r = (blend["r"] @ W[p + "r"].T).view(T, H, D)
    k = (blend["k"] @ W[p + "k"].T).view(T, H, D)
    v = (blend["v"] @ W[p + "v"].T).view(T, H, D)
    gate = silu(blend["g"] @ W[p + "g"].T)
    w = torch.exp(-torch.exp(torch.tanh(blend["w"] @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).view(T, H, D)
    u = W[p + "u"]
    S = torch.zeros(H, D, D, dtype=F64)
    o = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        kv = k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = ((S + u.unsqueeze(-1) * kv) * r[t].unsqueeze(-1)).sum(1)
        S = w[t].unsqueeze(-1) * S + kv
    o = unit_rms(o, eps).reshape(T, H * D) * W[p + "norm"]
    return (o * gate) @ W[p + "o"].T


def parallel_mixer(n, W, p, mx, eps):
    return mx["left_scale"] * sink_attention(n, W, p + "left.", mx["left"]) + \
        mx["right_scale"] * time_mix(n, W, p + "right.", mx["right"], eps)


# ------------------------------------------------------------------ state-space mixer
def ssm(n, W, p, mx, eps):
    T = n.shape[0]
    H, P, N, G = mx["heads"], mx["vdim"], mx["state"], mx["groups"]
    inner = H * P
    row = n @ W[p + "in"].T
    z, xbc, dt = row[:, :inner], row[:, inner:2 * inner + 2 * G * N], row[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    a = torch.exp(-torch.exp(W[p + "A_log"]) * dt)                      # [T, H]
    S = torch.zeros(H, N, P, dtype=F64)
    y = torch.zeros(T, H, P, dtype=F64)
    for t in range(T):
        for h in range(H):
            g = h // (H // G)
            S[h] = a[t, h] * S[h] + dt[t, h] * B[t, g].unsqueeze(-1) * x[t, h].unsqueeze(0)
            y[t, h] = S[h].T @ C[t, g] + W[p + "D"][h] * x[t, h]
    y = y.reshape(T, inner) * silu(z)
    parts = mx["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


# ------------------------------------------------------------------ experts
def expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def router_choice(n, W, p, top):
    """(experts [T, top], their sigmoid scores): the largest scores, the lowest index among equals."""
    s = torch.sigmoid(n @ W[p + "router"].T)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, s.gather(1, order)


def experts(n, W, p, mlp, take=None):
    """The weight multiplies an expert's input; the scores are not renormalized; the shared expert reads n."""
    T = n.shape[0]
    top = mlp["router"]["top"]
    chosen, score = router_choice(n, W, p, top)
    if take is not None:
        chosen = take
        score = torch.sigmoid(n @ W[p + "router"].T).gather(1, take)
    out = torch.zeros_like(n)
    for t in range(T):
        for j in range(top):
            out[t] += expert(score[t, j] * n[t:t + 1], W, f"{p}e{int(chosen[t, j])}.")[0]
    if mlp.get("shared"):
        out = out + expert(n, W, p + "shared.")
    return out, chosen


# ------------------------------------------------------------------ the model
MIXERS = {"attention": lambda n, W, p, mx, eps: conv_attention(n, W, p, mx, eps),
          "parallel": parallel_mixer, "mamba2": ssm}


def layer_order(cfg):
    """[(layer, pass or None)]: the looped span ``times`` times in a row, the rest once."""
    L, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(L)]
    a, b, n = loop["start"], loop["stop"], loop["times"]
    return [(i, None) for i in range(a)] + [(i, t) for t in range(n) for i in range(a, b)] + [(i, None) for i in range(b, L)]


def forward(tokens, W, cfg, take=None, streams=None, chosen=None):
    """Logits [T, vocab] of one sequence from its first token.  ``streams``: a list that receives the
    stream after every layer run; ``take``: experts per layer run instead of the routers' choice;
    ``chosen``: a list that receives the experts taken."""
    eps = cfg["norm"]["eps"]
    x0 = embedding(tokens, W, cfg)
    x = x0
    loop = cfg.get("loop")
    run = 0
    for i, t in layer_order(cfg):
        if t is not None and i == loop["start"]:
            x = torch.cat([x, x0], -1) @ W["loop.in"].T + W["loop.step"][t]
        L, p = cfg["layers"][i], f"l{i}."
        x = x + dyt(MIXERS[L["type"]](dyt(x, W, p + "norm1"), W, p + "mix.", L["mixer"], eps), W, p + "norm1b")
        if L.get("mlp"):
            f, c = experts(dyt(x, W, p + "norm2"), W, p + "mlp.", L["mlp"], None if take is None else take[run])
            x = x + dyt(f, W, p + "norm2b")
            if chosen is not None:
                chosen.append(c)
            run += 1
        if streams is not None:
            streams.append(x.clone())
    logits = dyt(x, W, "final.norm") @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
