"""The Tebalorn design in plain float64: one function per mechanism, whole sequences, token by token
where the design is a recurrence.  Slow on purpose; shares no code with the engine.

Notation: x [T, d] the stream, n = unit_rms(x) * w the normed stream, W the weights by checkpoint name
(float64), p the positions 0 .. T-1.
"""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return unit_rms(x, eps) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------ linear attention
def recurrence(q, k, v, decay):
    """o_t = S_t^T q_t with S_t = diag(decay_t) S_(t-1) + k_t v_t^T, S_0 = 0.
    q, k, decay [T, H, D]; v [T, H, V]; returns [T, H, V] and the last state [H, D, V]."""
    T, H, D = q.shape
    V = v.shape[-1]
    S = torch.zeros(H, D, V, dtype=torch.float64)
    out = torch.zeros(T, H, V, dtype=torch.float64)
    for t in range(T):
        S = decay[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = (S * q[t].unsqueeze(-1)).sum(1)
    return out, S


def channel_decay(n, W, p, tau):
    """sigmoid(z)^(1/tau), z = W_a2 (W_a1 n) + b."""
    z = (n @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    return torch.sigmoid(z) ** (1.0 / tau)


def gla(n, W, p, mx, eps):
    T = n.shape[0]
    H, D, V = mx["heads"], mx["dim"], mx["vdim"]
    q = (n @ W[p + "q"].T).view(T, H, D) / math.sqrt(D)
    k = (n @ W[p + "k"].T).view(T, H, D)
    v = (n @ W[p + "v"].T).view(T, H, V)
    a = channel_decay(n, W, p, mx["tau"]).view(T, H, D)
    o, _ = recurrence(q, k, v, a)
    o = unit_rms(o, eps) * W[p + "norm"]                       # every head on its own, one weight for all
    return (o.reshape(T, H * V) * silu(n @ W[p + "g"].T)) @ W[p + "o"].T


def lightning(n, W, p, mx, eps):
    T = n.shape[0]
    H, D, V = mx["heads"], mx["dim"], mx["vdim"]
    q = silu(n @ W[p + "q"].T).view(T, H, D)
    k = silu(n @ W[p + "k"].T).view(T, H, D)
    v = silu(n @ W[p + "v"].T).view(T, H, V)
    a = torch.tensor(mx["decay"], dtype=torch.float64).view(1, H, 1).expand(T, H, D)
    o, _ = recurrence(q, k, v, a)
    o = unit_rms(o.reshape(T, H * V), eps) * W[p + "norm"]     # the heads together
    return (o * torch.sigmoid(n @ W[p + "g"].T)) @ W[p + "o"].T


# ------------------------------------------------------------------ softmax attention
def rotation_table(rot):
    """(frequencies [dims/2], the constant on sine and cosine)."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0
    index = lambda turns: dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo, hi = max(math.floor(index(sc["fast"])), 0), min(math.ceil(index(sc["slow"])), dims - 1)
    for i in range(dims // 2):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        f[i] = (1.0 - r) * f[i] + r * f[i] / sc["factor"]
    return torch.tensor(f, dtype=torch.float64), 0.1 * math.log(sc["factor"]) + 1.0


def turn(x, pos, rot):
    """x [T, heads, D]: pairs (i, i + dims/2) of the first ``dims`` elements turn by pos * f_i."""
    f, mag = rotation_table(rot)
    half = rot["dims"] // 2
    ang = pos.double().unsqueeze(-1) * f
    c, s = (torch.cos(ang) * mag).unsqueeze(1), (torch.sin(ang) * mag).unsqueeze(1)
    a, b = x[..., :half], x[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., 2 * half:]], dim=-1)


def visible(pos, chunk):
    i, j = pos.unsqueeze(1), pos.unsqueeze(0)
    ok = j <= i
    if chunk is not None:
        ok = ok & (torch.div(i, chunk, rounding_mode="floor") == torch.div(j, chunk, rounding_mode="floor"))
    return ok


def sink_softmax(scores, ok, sink):
    """Weights over the keys with one more term exp(sink) in the denominator."""
    s = scores.masked_fill(~ok, float("-inf"))
    m = torch.maximum(s.max(-1, keepdim=True).values, torch.full_like(s[:, :1], float(sink)))
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + math.exp(float(sink)) / torch.exp(m))


def attention(n, W, p, mx, pos):
    T = n.shape[0]
    H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (n @ W[p + "q"].T).view(T, H, D)
    k = (n @ W[p + "k"].T).view(T, G, D)
    v = (n @ W[p + "v"].T).view(T, G, V)
    if mx.get("rot"):
        q, k = turn(q, pos, mx["rot"]), turn(k, pos, mx["rot"])
    ok = visible(pos, mx["mask"]["size"] if mx.get("mask") else None)
    heads = []
    for h in range(H):
        g = h // (H // G)
        w = sink_softmax(q[:, h] @ k[:, g].T * mx["scale"], ok, W[p + "sink"][h])
        heads.append(w @ v[:, g])
    return torch.cat(heads, dim=-1) @ W[p + "o"].T


# ------------------------------------------------------------------ feed-forward, token input
def gated(n, W, p, act):
    return (act(n @ W[p + "gate"].T) * (n @ W[p + "up"].T)) @ W[p + "down"].T


def route(n, W, p, ml):
    """(experts [T, top], weights [T, top]): the largest logits, softmax over the taken ones."""
    z = n @ W[p + "router"].T
    val, idx = torch.topk(z, ml["router"]["top"], dim=-1)
    return idx, torch.softmax(val, dim=-1)


def experts(n, W, p, ml, taken=None, chosen=None):
    """``taken`` [T, top]: experts to take instead of the router's own choice (their weights still come
    from their own logits); ``chosen``: a list that receives the experts."""
    if taken is None:
        idx, w = route(n, W, p, ml)
    else:
        idx = taken
        w = torch.softmax((n @ W[p + "router"].T).gather(1, idx), dim=-1)
    if chosen is not None:
        chosen.append(idx)
    out = torch.zeros_like(n)
    for t in range(n.shape[0]):
        for j in range(idx.shape[1]):
            out[t] += w[t, j] * gated(n[t:t + 1], W, f"{p}e{int(idx[t, j])}.", silu)[0]
    if ml.get("shared"):
        out = out + gated(n, W, p + "shared.", silu)
    return out


def token_input(x, W, p, tokens, layer, dim, eps):
    rows = W["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ W[p + "side.gate"].T) * rows) @ W[p + "side.proj"].T
    return x + unit_rms(y, eps) * W[p + "side.norm"]


# ------------------------------------------------------------------ the model
def forward(cfg, W, tokens, upto=None, taken=None, chosen=None):
    """Logits [T, vocab] of a whole sequence, or, with ``upto``, the stream after that many layers.
    ``taken``: {layer: experts [T, top]} to take; ``chosen``: a dict that receives them."""
    tok = torch.tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(tokens))
    eps = cfg["norm"]["eps"]
    x = W["embed"][tok] * (cfg.get("embedding") or {}).get("scale", 1.0)
    for i, L in enumerate(cfg["layers"]):
        if upto is not None and i >= upto:
            return x
        p = f"l{i}."
        n = norm(x, W[p + "norm1"], eps)
        mix = {"gla": lambda: gla(n, W, p + "mix.", L["mixer"], eps),
               "lightning": lambda: lightning(n, W, p + "mix.", L["mixer"], eps),
               "attention": lambda: attention(n, W, p + "mix.", L["mixer"], pos)}[L["type"]]()
        ml = L.get("mlp")
        if ml is None:
            ff = 0.0
        elif ml["kind"] == "dense":
            ff = gated(n, W, p + "mlp.", torch.relu)
        else:
            got = []
            ff = experts(n, W, p + "mlp.", ml, None if taken is None else taken[i], got)
            if chosen is not None:
                chosen[i] = got[0]
        x = x + (mix + ff)
        if cfg.get("token_side"):
            x = token_input(x, W, p, tok, i, cfg["token_side"]["dim"], eps)
    if upto is not None:
        return x
    return norm(x, W["final.norm"], eps) @ W["head"].T * cfg.get("logit_scale", 1.0)


def greedy(row):
    return int(torch.argmax(row))
