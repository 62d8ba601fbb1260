"""The Nolapel design in the engine against the plain implementation (``plain_nolapel``): every mechanism's
kernel alone, whole prompts, decoding through the state rows and the cache, portions down to two tokens, mixed
batches with pages and slots used again, window edges, far keys and far tokens, the first tokens, generation."""
from __future__ import annotations

import copy
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
import plain_nolapel as plain


# ------------------------------------------------------------------------------------------ configurations
def _attention(heads, kv, dim, scale, window, conv=3, q_temp=(0.2, 16)):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if conv:
        m["conv"] = conv
    if window is not None:
        m["mask"] = {"size": window}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return "attention", m


def _parallel(heads, kv, dim, vdim, scale, rot, rheads, rdim, ls=1.1, rs=0.7):
    left = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        left["rot"] = {"base": rot[0], "dims": rot[1]}
    return "parallel", {"left": left, "right": {"heads": rheads, "dim": rdim}, "left_scale": ls, "right_scale": rs}


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return "mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _moe(experts, top, ff, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff},
            "shared": None if shared is None else {"ff": shared}}


def _layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


# odd sizes that no fast kernel takes; every kind of mixer, a layer without feed-forward, a loop that starts at layer 1
SMALL = {"architecture": "Nolapel", "vocab": 96, "width": 40, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
         "embedding": {"bigram": {"buckets": 53, "mul_prev": 31, "mul_cur": 7}},
         "loop": {"start": 1, "stop": 3, "times": 2},
         "layers": [_layer(_ssm(3, 10, 6, 3, 3, 1), _moe(5, 2, 12, shared=20)),
                    _layer(_attention(4, 2, 12, 0.3, 9, conv=3, q_temp=(0.4, 5)), _moe(4, 1, 8)),
                    _layer(_parallel(3, 3, 8, 6, 0.4, (100.0, 4), 2, 10), None),
                    _layer(_attention(3, 1, 10, 0.25, None, conv=2, q_temp=None), _moe(3, 3, 8, shared=8)),
                    _layer(_ssm(4, 5, 9, 2, 5, 4), _moe(6, 2, 8))]}
# sizes that the matrix-unit kernels take in bfloat16 (heads of 64 and 128, pages of 32)
WIDE = {"architecture": "Nolapel", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "logit_softcap": 20.0,
        "embedding": {"bigram": {"buckets": 211, "mul_prev": 101, "mul_cur": 13}},
        "loop": {"start": 0, "stop": 2, "times": 3},
        "layers": [_layer(_ssm(4, 32, 64, 2, 4, 2), _moe(4, 2, 64, shared=64)),
                   _layer(_attention(4, 2, 64, 0.125, 40, conv=4, q_temp=(0.3, 32)), _moe(6, 1, 32, shared=64)),
                   _layer(_parallel(4, 1, 64, 64, 0.2, (10000.0, 32), 2, 64), _moe(4, 2, 64)),
                   _layer(_attention(2, 1, 128, 0.1, None, conv=4, q_temp=(0.1, 64)), _moe(4, 1, 64, shared=32))]}
# values that are 1, equal or absent where the other configurations have them apart
ONES = {"architecture": "Nolapel", "vocab": 50, "width": 24, "norm": {"eps": 1e-3},
        "loop": {"start": 0, "stop": 1, "times": 1},
        "layers": [_layer(_attention(1, 1, 2, 1.0, 1, conv=0, q_temp=(1.0, 1)), _moe(1, 1, 8)),
                   _layer(_ssm(1, 2, 2, 1, 1, 1), None),
                   _layer(_parallel(1, 1, 2, 2, 1.0, None, 1, 2, ls=1.0, rs=1.0), _moe(2, 2, 4, shared=4)),
                   _layer(_attention(5, 5, 4, 0.5, 2, conv=2, q_temp=None), _moe(2, 1, 4))]}
CONFIGS = {"small": SMALL, "wide": WIDE, "ones": ONES}
PAGE = {"small": 16, "wide": 32, "ones": 4}
LENGTHS = {"small": [1, 45, 23, 60, 2, 31, 17], "wide": [90, 1, 140, 33, 75], "ones": [30, 1, 44, 9]}


def planted(cfg, seed, gain=3.0, std=0.08):
    """Random tensors with sharper attention, routers that tell experts apart, sinks of the size of a score,
    decays spread over (0, 1), step sizes around 1, convolutions whose taps all count, alphas around 1."""
    from spite_amd.weights.random_init import random_tensors
    t = random_tensors(cfg, seed, std)
    g = torch.Generator().manual_seed(seed)
    rnd = lambda shape, s=1.0: torch.randn(shape, generator=g) * s
    d = cfg["width"]
    for name in ("embed", "bigram"):                       # rows large enough to bend the tanh norms
        if name in t:
            t[name] = t[name] * (0.6 / std)
    for name in list(t):
        if name.endswith(".alpha"):
            t[name] = torch.tensor(0.7) + 0.3 * torch.rand((), generator=g)
        elif name.endswith(".b") and ("norm" in name):
            t[name] = rnd(t[name].shape, 0.1)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}.mix."
        mx = L["mixer"]
        if L["type"] == "attention":
            t[p + "q"] = t[p + "q"] * gain
            for s in ("q", "k"):
                if p + s + ".conv" in t:
                    t[p + s + ".conv"] = rnd(t[p + s + ".conv"].shape, 0.5)
                t[p + s + ".norm"] = 1.0 + rnd(t[p + s + ".norm"].shape, 0.3)
        elif L["type"] == "parallel":
            t[p + "left.q"] = t[p + "left.q"] * gain
            t[p + "left.sink"] = rnd(t[p + "left.sink"].shape, 1.5)
            r = p + "right."
            n = mx["right"]["heads"] * mx["right"]["dim"]
            for s in "rkvgw":
                t[r + "mu." + s] = torch.rand(d, generator=g)
            t[r + "w1"] = rnd(t[r + "w1"].shape, 0.3)
            t[r + "w2"] = rnd(t[r + "w2"].shape, 0.5)
            t[r + "w0"] = rnd((n,), 1.0) - 2.0
            t[r + "u"] = rnd(t[r + "u"].shape, 0.5)
            t[r + "norm"] = 1.0 + rnd((n,), 0.3)
            for s in "rkv":
                t[r + s] = t[r + s] * gain
        else:
            Hh = mx["heads"]
            t[p + "conv"] = rnd(t[p + "conv"].shape, 0.5)
            t[p + "conv.b"] = rnd(t[p + "conv.b"].shape, 0.2)
            t[p + "dt_bias"] = rnd((Hh,), 1.0)
            t[p + "A_log"] = rnd((Hh,), 1.0) - 1.0
            t[p + "D"] = 1.0 + rnd((Hh,), 0.5)
            t[p + "norm"] = 1.0 + rnd(t[p + "norm"].shape, 0.3)
            t[p + "in"] = t[p + "in"] * gain
        if L["mlp"]:
            t[f"l{i}.mlp.router"] = t[f"l{i}.mlp.router"] * 8.0
    if "loop.step" in t:
        t["loop.step"] = rnd(t["loop.step"].shape, 0.3)
        t["loop.in"] = torch.cat([torch.eye(d), torch.zeros(d, d)], 1) * 0.7 + rnd((d, 2 * d), 0.1)
    return t


def make_model(folder, cfg, seed, dtype, **kw):
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(folder), cfg, seed, dtype=dtype, overrides=planted(cfg, seed, **kw))
    return H.read_weights(str(folder))


def requests(vocab, lengths, seed):
    return {f"r{i}": H.random_tokens(vocab, n, seed + 13 * i) for i, n in enumerate(lengths)}


def expert_runs(cfg):
    """How many layer runs of a step have experts (a looped layer counts once a pass)."""
    return sum(1 for i, _ in plain.layer_order(cfg) if cfg["layers"][i]["mlp"])


def tops(cfg):
    return [cfg["layers"][i]["mlp"]["router"]["top"] for i, _ in plain.layer_order(cfg) if cfg["layers"][i]["mlp"]]


def plain_rows(cfg, weights, reqs, taken=None, chosen=None):
    """{(request, position): logits}; ``taken``: {request: [experts [T, top] per layer run]}; ``chosen`` receives them."""
    rows = {}
    for rid, toks in reqs.items():
        got = []
        out = plain.forward(toks, weights, cfg, take=None if taken is None else taken[rid], chosen=got).to(torch.float32).numpy()
        if chosen is not None:
            chosen[rid] = got
        for i in range(len(toks)):
            rows[(rid, i)] = out[i]
    return rows


def experts_of(cfg, steps, routing):
    """{request: [experts [T, top] per layer run]} from what a replay recorded step by step."""
    tk, parts = tops(cfg), {}
    for rec in steps:
        off = 0
        for e in rec["entries"]:
            n = len(e["tokens"])
            for k, top in enumerate(tk):
                parts.setdefault(e["id"], [[] for _ in tk])[k].append(np.asarray(routing[rec["step"]][k]).reshape(-1, top)[off:off + n])
            off += n
    return {rid: [torch.from_numpy(np.concatenate(v).astype(np.int64)) for v in per] for rid, per in parts.items()}


def experts_for(cfg, steps, experts):
    """{step: [experts of the step's tokens, one array per layer run]}: ``experts`` cut as ``steps`` cuts."""
    n_runs, fed, take = expert_runs(cfg), {}, {}
    for rec in steps:
        per = [[] for _ in range(n_runs)]
        for e in rec["entries"]:
            at, n = fed.get(e["id"], 0), len(e["tokens"])
            for k in range(n_runs):
                per[k].append(experts[e["id"]][k][at:at + n].numpy())
            fed[e["id"]] = at + n
        take[rec["step"]] = [np.concatenate(x).astype(np.int32) if x else np.zeros((0,), np.int32) for x in per]
    return take


def engine(folder, dtype, name, **kw):
    from spite_amd import Engine
    kw.setdefault("page_size", PAGE[name])
    kw.setdefault("cache_tokens", 1024)
    kw.setdefault("max_requests", 4)
    return Engine(str(folder), dtype=dtype, device="cuda:0", **kw)


def poison(eng):
    """Every cache row and every state row holds NaN (integer rows: a large number) until it is written or cleared."""
    for g in eng.cache.groups:
        for half in g.halves():
            if half is not None and half.numel():
                half.fill_(float("nan"))
    for st in eng.cache.states.values():
        st.fill_(float("nan") if st.is_floating_point() else 12345)


def rows_over(a, b, limit):
    return [k for k in a if not float(np.max(np.abs(a[k].astype(np.float64) - b[k].astype(np.float64)))) <= limit]


def close_in_16_bits(rows, ref, scale, tol):
    """bfloat16 against the plain implementation: every row within 4 ``tol``, all but one in fifty within ``tol``."""
    far, near = rows_over(rows, ref, 4 * tol * scale), rows_over(rows, ref, tol * scale)
    assert not far and len(near) <= max(1, len(rows) // 50), f"{len(near)} of {len(rows)} rows over {tol * scale}, {far[:3]} far over (scale {scale})"


def scale_of(rows):
    return max(float(np.abs(v).max()) for v in rows.values())


# ------------------------------------------------------------------------------------------ without a GPU
def test_registry_and_tensor_names():
    from spite_amd.config import read_config
    from spite_amd.config.nolapel import NolapelConfig
    from spite_amd.engine.model import Model
    from spite_amd.engine.context import Env
    arch, cfg = read_config(SMALL)
    assert arch.name == "Nolapel" and isinstance(cfg, NolapelConfig)
    assert cfg.layers[1].mixer.window == 9 and cfg.layers[3].mixer.window is None and cfg.layers[2].mlp is None
    assert cfg.layers[1].mixer.q_temp == (0.4, 5) and cfg.layers[3].mixer.q_temp is None and cfg.loop.times == 2
    assert cfg.layers[0].mlp.shared_ff == 20 and cfg.layers[1].mlp.shared_ff is None and cfg.bigram.buckets == 53
    spec = arch.build_spec(cfg)
    model = Model(spec, Env(torch.float32, torch.device("cpu")))
    names = {n: ps.shape for n, ps, _, _ in model.tensor_plan()}
    assert {"embed", "bigram", "loop.in", "loop.step", "final.norm", "final.norm.b", "final.norm.alpha", "head",
            "l0.mix.in", "l0.mix.conv", "l0.mix.conv.b", "l0.mix.dt_bias", "l0.mix.A_log", "l0.mix.D", "l0.mix.norm", "l0.mix.o",
            "l1.mix.q.conv", "l1.mix.k.norm", "l2.mix.left.sink", "l2.mix.right.mu.w", "l2.mix.right.w0", "l2.mix.right.u",
            "l0.mlp.router", "l0.mlp.e4.down", "l0.mlp.shared.up", "l0.norm1b.alpha", "l0.norm2b.b"} <= set(names)
    assert "l2.norm2" not in names and "l2.mlp.router" not in names and "l1.mlp.shared.up" not in names and "l1.mix.v" not in names
    assert names["bigram"] == (54, 40) and names["loop.in"] == (40, 80) and names["loop.step"] == (2, 40) and names["l0.norm1.alpha"] == ()
    assert names["l0.mix.in"] == (2 * 30 + 2 * 18 + 3, 40) and names["l0.mix.conv"] == (30 + 36, 3) and names["l0.mix.norm"] == (30,)
    assert names["l1.mix.q"] == (48, 40) and names["l1.mix.k"] == (24, 40) and names["l1.mix.q.conv"] == (48, 3) and names["l1.mix.q.norm"] == (12,)
    assert names["l2.mix.left.v"] == (18, 40) and names["l2.mix.right.r"] == (20, 40) and names["l2.mix.right.u"] == (2, 10)
    # the order of a step: layer 0, then twice (reentry, layers 1 and 2), then layers 3 and 4; every pass its own caches
    assert [c.block for c in spec.order] == [0, 5, 1, 2, 5, 1, 2, 3, 4] and [c.arg for c in spec.order if c.block == 5] == [0, 1]
    ids = [cid for c in spec.order for cid in c.cache_ids().values()]
    assert len(ids) == len(set(ids))
    needs = model.cache_needs()
    assert needs[0].state.shape == (3, 6, 10) and needs[1].state.shape == (2, 66)
    assert needs[2].kv.visibility == "window" and needs[2].kv.span == 9 and needs[2].state.shape == (2, 72)
    assert needs[3].kv.visibility == "full" and needs[3].kv.value_dim == 6 and needs[4].state.shape == (2, 10, 10) and needs[5].state.shape == (40,)
    assert needs[-1].state.dtype == torch.int32 and needs[-1].state.shape == ()
    # without the optional keys: a plain embedding, no loop, no cap
    bare = {k: v for k, v in SMALL.items() if k not in ("embedding", "loop", "logit_softcap")}
    arch, cfg = read_config(bare)
    spec = arch.build_spec(cfg)
    assert spec.embedding is None and not spec.keep_embedding and [c.block for c in spec.order] == [0, 1, 2, 3, 4]


def test_config_errors_are_collected():
    from spite_amd.config import read_config, ConfigError
    bad = copy.deepcopy(SMALL)
    del bad["vocab"]
    bad["layers"][0]["mixer"]["groups"] = 2
    bad["layers"][1]["mixer"]["kv_heads"] = 3
    bad["layers"][1]["mixer"]["vdim"] = 7
    bad["layers"][2]["mixer"]["left"]["rot"]["dims"] = 7
    bad["layers"][3]["mlp"]["router"]["top"] = 9
    bad["layers"][4]["type"] = "other"
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError) as e:
        read_config(bad)
    msg = str(e.value)
    for word in ("vocab", "groups", "kv_heads", "vdim", "rot.dims", "router.top", "type", "loop"):
        assert word in msg, word


def test_plain_mechanisms():
    g = torch.Generator().manual_seed(0)
    f64 = torch.float64
    # the convolution as written out by hand; zeros before the start
    u, w = torch.rand(5, 2, generator=g, dtype=f64), torch.rand(2, 3, generator=g, dtype=f64)
    y = plain.causal_conv(u, w)
    assert float((y[0] - w[:, 2] * u[0]).abs().max()) < 1e-12
    assert float((y[3] - (w[:, 0] * u[1] + w[:, 1] * u[2] + w[:, 2] * u[3])).abs().max()) < 1e-12
    # the hashed row, and the last row for the first token
    assert plain.bigram_rows([5, 9, 2], {"buckets": 7, "mul_prev": 3, "mul_cur": 4}) == [7, (5 * 3 + 9 * 4) % 7, (9 * 3 + 2 * 4) % 7]
    # the tanh norm
    W = {"n": torch.tensor([2.0, 3.0], dtype=f64), "n.b": torch.tensor([0.5, -0.5], dtype=f64), "n.alpha": torch.tensor(0.5, dtype=f64)}
    assert float((plain.dyt(torch.tensor([[1.0, -2.0]], dtype=f64), W, "n") - torch.tensor([[2 * math.tanh(0.5) + 0.5, 3 * math.tanh(-1.0) - 0.5]], dtype=f64)).abs().max()) < 1e-12
    # softmax with a sink of score zero: one more 1 in the denominator; the slope counts the distance; the window
    q, k = torch.ones(3, 1, 1, dtype=f64), torch.tensor([0.0, 1.0, 2.0], dtype=f64).view(3, 1, 1)
    v = torch.tensor([1.0, 10.0, 100.0], dtype=f64).view(3, 1, 1)
    o = plain.softmax_attention(q, k, v, 1.0, sink=torch.zeros(1, dtype=f64), window=2, slopes=[0.5])
    den = 1.0 + math.exp(2.0) + math.exp(1.0 - 0.5)
    assert abs(float(o[2, 0, 0]) - (100.0 * math.exp(2.0) + 10.0 * math.exp(0.5)) / den) < 1e-12
    assert abs(float(o[0, 0, 0]) - 1.0 / 2.0) < 1e-12
    # the state-space recurrence as a sum over earlier tokens with the decays' products
    T, Hh, P, N = 6, 2, 3, 4
    cfg_mx = {"heads": Hh, "vdim": P, "state": N, "groups": 1, "conv": 1, "norm_groups": 1}
    inner = Hh * P
    Wm = {"in": torch.randn(2 * inner + 2 * N + Hh, 5, generator=g, dtype=f64), "conv": torch.ones(inner + 2 * N, 1, dtype=f64),
          "conv.b": torch.zeros(inner + 2 * N, dtype=f64), "dt_bias": torch.randn(Hh, generator=g, dtype=f64),
          "A_log": torch.randn(Hh, generator=g, dtype=f64), "D": torch.zeros(Hh, dtype=f64), "norm": torch.ones(inner, dtype=f64),
          "o": torch.eye(inner, dtype=f64)}
    n = torch.randn(T, 5, generator=g, dtype=f64)
    row = n @ Wm["in"].T
    z, xbc, dt = row[:, :inner], plain.silu(row[:, inner:2 * inner + 2 * N]), plain.softplus(row[:, 2 * inner + 2 * N:] + Wm["dt_bias"])
    x, B, C = xbc[:, :inner].view(T, Hh, P), xbc[:, inner:inner + N], xbc[:, inner + N:]
    a = torch.exp(-torch.exp(Wm["A_log"]) * dt)
    t = T - 1
    want = torch.zeros(Hh, P, dtype=f64)
    for s in range(t + 1):
        for h in range(Hh):
            want[h] += float(C[t] @ B[s]) * dt[s, h] * float(torch.prod(a[s + 1:t + 1, h])) * x[s, h]
    want = plain.unit_rms((want.reshape(1, inner) * plain.silu(z[t:t + 1])), 1e-5)
    got = plain.ssm(n, {"p." + k: v for k, v in Wm.items()}, "p.", cfg_mx, 1e-5)[t:t + 1]
    assert float((got - want).abs().max()) < 1e-10
    # the order of layers under a loop
    assert plain.layer_order(SMALL) == [(0, None), (1, 0), (2, 0), (1, 1), (2, 1), (3, None), (4, None)]


# ------------------------------------------------------------------------------------------ kernels alone
def _meta(lens, slots):
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32).cuda()
    sot = torch.tensor(np.repeat(np.arange(len(lens)), lens), dtype=torch.int32).cuda()
    return cu, sot, torch.tensor(slots, dtype=torch.int32).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [40, 37, 256])
def test_tanh_norm_kernel(dtype, d):
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(d)
    dt = getattr(torch, dtype)
    T = 9
    h, d1, d2, yn = (torch.randn(T, d, generator=g) for _ in range(4))
    w, b, wn, bn = (torch.randn(d, generator=g) for _ in range(4))
    al, an = torch.tensor([0.8]), torch.tensor([1.3])
    hd = h.cuda()
    out, out32 = torch.empty(T, d, dtype=dt, device="cuda:0"), torch.empty(T, d, device="cuda:0")
    hipops.add_tanh_norm(hd, w.cuda(), b.cuda(), al.cuda(), out=out, out32=out32, d1=d1.cuda(), d2=d2.cuda(),
                         normed=(yn.cuda(), wn.cuda(), bn.cuda(), an.cuda(), 0.5))
    v = h.double() + d1.double() + d2.double() + 0.5 * (torch.tanh(1.3 * yn.double()) * wn.double() + bn.double())
    want = torch.tanh(0.8 * v) * w.double() + b.double()
    assert float((hd.cpu().double() - v).abs().max()) < 1e-5
    assert float((out32.cpu().double() - want).abs().max()) < 1e-5
    assert float((out.cpu().double() - want).abs().max()) < (1e-5 if dtype == "float32" else 3e-2)
    # gathered rows do not change the stream; the stream itself in the products' dtype
    rows = torch.tensor([7, 2], dtype=torch.int32).cuda()
    o2 = torch.empty(2, d, dtype=dt, device="cuda:0")
    before = hd.clone()
    hipops.add_tanh_norm(hd, w.cuda(), b.cuda(), al.cuda(), out=o2, rows=rows, write_h=False)
    assert torch.equal(hd, before) and float((o2.cpu().double() - want[[7, 2]]).abs().max()) < (1e-5 if dtype == "float32" else 3e-2)
    hipops.add_tanh_norm(hd, None, None, None, out=out)
    assert float((out.cpu().double() - v).abs().max()) < (1e-5 if dtype == "float32" else 3e-2)
    if d % 4 == 0:
        # small fp32 products of the normed rows in the same pass (router logits)
        proj = torch.randn(5, d, generator=g)
        h2, po = h.cuda(), torch.empty(T, 5, device="cuda:0")
        hipops.add_tanh_norm(h2, w.cuda(), b.cuda(), al.cuda(), out=out, d1=d1.cuda(), d2=d2.cuda(),
                             normed=(yn.cuda(), wn.cuda(), bn.cuda(), an.cuda(), 0.5), proj=proj.cuda(), proj_out=po)
        assert float((h2.cpu().double() - v).abs().max()) < 1e-5
        assert float((out.cpu().double() - want).abs().max()) < (1e-5 if dtype == "float32" else 3e-2)
        assert float((po.cpu().double() - want @ proj.double().T).abs().max()) < 1e-4


@pytest.mark.gpu
def test_hashed_embedding_kernels():
    """Two steps over slots that lie apart: the first token of a request takes the last row, the first token of a
    later portion hashes with the request's last token of the step before."""
    from spite_amd.csrc import hipops
    V, d, buckets, mp, mc = 30, 12, 11, 1009, 23
    g = torch.Generator().manual_seed(1)
    table, pairs = torch.randn(V, d, generator=g), torch.randn(buckets + 1, d, generator=g)
    seqs = [H.random_tokens(V, n, 3 + n) for n in (7, 1, 9)]
    slots = [4, 1, 2]
    state = torch.full((6,), 999, dtype=torch.int32).cuda()
    cuts = [(0, [3, 1, 2]), (1, [4, 0, 7])]
    fed = [0, 0, 0]
    for step, lens in cuts:
        live = [i for i, n in enumerate(lens) if n]
        ids = [seqs[i][fed[i]:fed[i] + lens[i]] for i in live]
        pos = [list(range(fed[i], fed[i] + lens[i])) for i in live]
        cu, sot, sl = _meta([lens[i] for i in live], [slots[i] for i in live])
        flat = torch.tensor(sum(ids, []), dtype=torch.int32).cuda()
        T = flat.numel()
        rows = torch.empty(T, dtype=torch.int32, device="cuda:0")
        hipops.hash_rows(flat, torch.tensor(sum(pos, []), dtype=torch.int32).cuda(), sot, cu, sl, state, rows, mp, mc, buckets)
        h = torch.empty(T, d, device="cuda:0")
        hipops.embed_sum(flat, table.cuda(), rows, pairs.cuda(), h)
        want_rows = sum([plain.bigram_rows(seqs[i], {"buckets": buckets, "mul_prev": mp, "mul_cur": mc})[fed[i]:fed[i] + lens[i]] for i in live], [])
        assert rows.cpu().tolist() == want_rows
        want = table[flat.cpu().long()] + pairs[torch.tensor(want_rows)]
        assert float((h.cpu() - want).abs().max()) < 1e-6
        for i in live:
            fed[i] += lens[i]
    assert state.cpu().tolist() == [999, seqs[1][0], seqs[2][8], 999, seqs[0][6], 999]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps,C,bias,act", [(4, 24, True, "silu"), (2, 7, False, None), (1, 5, True, None), (7, 300, False, "silu")])
def test_convolution_kernel(dtype, taps, C, bias, act):
    """Three steps of portions shorter and longer than the taps, single tokens, slots apart, NaN in the rows of others."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(taps * C)
    dt = getattr(torch, dtype)
    lens_by_step = [[2, 1, 9], [1, 1, 1], [taps + 3, 2, 1]]
    total = [sum(x[i] for x in lens_by_step) for i in range(3)]
    u = [torch.randn(n, C, generator=g).to(dt) for n in total]
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g) if bias else None
    want = [plain.causal_conv(x.double(), w.double(), None if b is None else b.double()) for x in u]
    if act:
        want = [plain.silu(y) for y in want]
    slots = [5, 0, 3]
    state = None
    if taps > 1:
        state = torch.full((6, taps - 1, C), float("nan"))
        state[slots] = 0.0
        state = state.cuda()
    fed = [0, 0, 0]
    for lens in lens_by_step:
        cu, sot, sl = _meta(lens, slots)
        T = sum(lens)
        wide = torch.zeros(T, C + 5, dtype=dt)
        wide[:, 3:3 + C] = torch.cat([u[i][fed[i]:fed[i] + lens[i]] for i in range(3)])
        wide = wide.cuda()
        y = torch.full((T, C), float("nan"), dtype=dt, device="cuda:0")
        hipops.causal_conv(wide[:, 3:3 + C], w.t().contiguous().cuda(), y, state, sot, cu, sl, bias=None if b is None else b.cuda(), act=act)
        ref = torch.cat([want[i][fed[i]:fed[i] + lens[i]] for i in range(3)])
        tol = 1e-5 if dtype == "float32" else 2e-2
        assert float((y.cpu().double() - ref).abs().max()) <= tol * max(1.0, float(ref.abs().max()))
        for i in range(3):
            fed[i] += lens[i]
    if taps > 1:
        for i, s in enumerate(slots):
            assert torch.equal(state[s].cpu(), u[i][-(taps - 1):].float()) or total[i] < taps - 1
        assert bool(torch.isnan(state[[1, 2, 4]]).all())


@pytest.mark.gpu
@pytest.mark.parametrize("taps", [2, 3, 4])
def test_convolution_kernel_in_tiles(taps):
    """Steps of many tokens run in tiles of tokens: the same bits as the same requests in small portions (a workgroup a
    token), tiles that cross an entry's border and a last tile that is not full included."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(taps)
    C, lens = 40, [301, 5, 263]
    u = [torch.randn(n, C, generator=g).to(torch.bfloat16) for n in lens]
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    wt = w.t().contiguous().cuda()
    want = torch.cat([plain.silu(plain.causal_conv(x.double(), w.double(), b.double())) for x in u])
    slots = [2, 0, 1]

    def run(portion):
        state = torch.zeros(3, taps - 1, C).cuda()
        outs = [[] for _ in lens]
        at = 0
        while at < max(lens):
            cut = [max(0, min(portion, n - at)) for n in lens]
            live = [i for i, n in enumerate(cut) if n]
            cu, sot, sl = _meta([cut[i] for i in live], [slots[i] for i in live])
            rows = torch.cat([u[i][at:at + cut[i]] for i in live]).cuda()
            y = torch.empty_like(rows)
            hipops.causal_conv(rows, wt, y, state, sot, cu, sl, bias=b.cuda(), act="silu")
            o = 0
            for i in live:
                outs[i].append(y[o:o + cut[i]].cpu())
                o += cut[i]
            at += portion
        return torch.cat([torch.cat(x) for x in outs]), state.cpu()
    whole, s1 = run(10 ** 6)
    small, s2 = run(37)
    assert torch.equal(whole, small) and torch.equal(s1, s2)
    assert float((whole.double() - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_blend_with_the_row_before_kernel(dtype):
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(4)
    dt = getattr(torch, dtype)
    d, n = 44, 5
    x = [torch.randn(L, d, generator=g).to(dt) for L in (6, 2, 11)]
    mu = torch.rand(n, d, generator=g)
    slots = [2, 4, 0]
    state = torch.full((5, d), float("nan"))
    state[slots] = 0.0
    state = state.cuda()
    fed = [0, 0, 0]
    for lens in ([3, 1, 4], [3, 1, 7]):
        cu, sot, sl = _meta(lens, slots)
        rows = torch.cat([x[i][fed[i]:fed[i] + lens[i]] for i in range(3)]).cuda()
        y = torch.empty(n, sum(lens), d, dtype=dt, device="cuda:0")
        hipops.shift_mix(rows, mu.cuda(), state, y, sot, cu, sl)
        want = []
        for i in range(3):
            xs = x[i].double()
            before = torch.cat([torch.zeros(1, d, dtype=torch.float64), xs[:-1]])
            want.append((xs.unsqueeze(0) + (before - xs).unsqueeze(0) * mu.double().unsqueeze(1))[:, fed[i]:fed[i] + lens[i]])
        ref = torch.cat(want, 1)
        assert float((y.cpu().double() - ref).abs().max()) <= (1e-6 if dtype == "float32" else 2e-2) * 4
        for i in range(3):
            fed[i] += lens[i]
    assert bool(torch.isnan(state[[1, 3]]).all())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hh,D,lens", [(2, 10, [5, 1, 2]), (2, 64, [70, 1, 33]), (1, 130, [20]), (3, 32, [1, 1, 1])])
def test_recurrence_with_a_bonus_kernel(dtype, Hh, D, lens):
    """o_t = (S + diag(u) k v^T)^T r before the token enters the state, over two steps through state rows apart."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(D)
    dt = getattr(torch, dtype)
    n, slots = len(lens), [3, 0, 5][:len(lens)]
    state = torch.full((6, Hh, D, D), float("nan"))
    state[slots] = 0.0
    state = state.cuda()
    full = [2 * L for L in lens]
    rnd = lambda *s: torch.randn(*s, generator=g)
    r, k, v = ([(rnd(L, Hh, D) * 0.5).to(dt) for L in full] for _ in range(3))
    w = [torch.exp(-torch.exp(rnd(L, Hh, D) - 2.0)) for L in full]
    u = rnd(Hh, D) * 0.5
    want = []
    for i in range(n):
        S = torch.zeros(Hh, D, D, dtype=torch.float64)
        o = torch.zeros(full[i], Hh, D, dtype=torch.float64)
        for t in range(full[i]):
            kv = k[i][t].double().unsqueeze(-1) * v[i][t].double().unsqueeze(-2)
            o[t] = ((S + u.double().unsqueeze(-1) * kv) * r[i][t].double().unsqueeze(-1)).sum(1)
            S = w[i][t].double().unsqueeze(-1) * S + kv
        want.append(o)
    scale = max(float(o.abs().max()) for o in want)
    cu, _, sl = _meta(lens, slots)
    for step in range(2):
        cut = lambda xs: torch.cat([x[step * L:(step + 1) * L] for x, L in zip(xs, lens)])
        T = sum(lens)
        row = torch.cat([cut(r).reshape(T, -1), cut(k).reshape(T, -1), cut(v).reshape(T, -1)], dim=1).cuda()
        n_ = Hh * D
        out = torch.full((T, n_), float("nan"), device="cuda:0")
        hipops.linear_attn_scan(row[:, :n_], row[:, n_:2 * n_], row[:, 2 * n_:], out, state, cu, sl, n, Hh, D, D,
                                decay=cut(w).reshape(T, -1).float().contiguous().cuda(), bonus=u.cuda(), longest=max(lens))
        ref = torch.cat([o[step * L:(step + 1) * L] for o, L in zip(want, lens)]).reshape(T, n_)
        assert float((out.cpu().double() - ref).abs().max()) <= 2e-5 * scale, f"step {step}"
    assert bool(torch.isnan(state[[1, 2, 4]]).all())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hh,G,N,P,lens", [(3, 3, 6, 10, [5, 1, 2]), (4, 2, 64, 32, [70, 1, 33]), (6, 1, 48, 48, [40]), (2, 1, 16, 64, [1, 1])])
def test_recurrence_with_shared_keys_and_step_sizes_kernel(dtype, Hh, G, N, P, lens):
    """Heads of a group share q and k; a head's value row enters the state times the token's step size."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(N + P)
    dt = getattr(torch, dtype)
    n, slots = len(lens), [2, 0, 4][:len(lens)]
    state = torch.zeros(5, Hh, N, P).cuda()
    rnd = lambda *s: torch.randn(*s, generator=g)
    T = sum(lens)
    C, B, x = (rnd(T, G, N) * 0.5).to(dt), (rnd(T, G, N) * 0.5).to(dt), rnd(T, Hh, P).to(dt)
    raw, dt_bias, a_log = rnd(T, Hh).to(dt), rnd(Hh), rnd(Hh) - 1.0
    step = torch.empty(T, Hh, device="cuda:0")
    decay = torch.empty(T, Hh * N, device="cuda:0")
    wide = torch.cat([x.reshape(T, -1), B.reshape(T, -1), C.reshape(T, -1), raw], 1).cuda()
    hipops.step_decay(wide[:, Hh * P + 2 * G * N:], dt_bias.cuda(), a_log.cuda(), step, decay, Hh, N)
    want_dt = plain.softplus(raw.double() + dt_bias.double())
    want_a = torch.exp(-torch.exp(a_log.double()) * want_dt)
    assert float((step.cpu().double() - want_dt).abs().max()) < 1e-5
    assert float((decay.cpu().double().view(T, Hh, N) - want_a.unsqueeze(-1)).abs().max()) < 1e-6
    out = torch.full((T, Hh * P), float("nan"), device="cuda:0")
    cu, _, sl = _meta(lens, slots)
    hipops.linear_attn_scan(wide[:, Hh * P + G * N:Hh * P + 2 * G * N], wide[:, Hh * P:Hh * P + G * N], wide[:, :Hh * P], out, state,
                            cu, sl, n, Hh, N, P, decay=decay, qk_heads=G, v_scale=step, longest=max(lens))
    ref = torch.zeros(T, Hh, P, dtype=torch.float64)
    at = 0
    for L in lens:
        S = torch.zeros(Hh, N, P, dtype=torch.float64)
        for t in range(at, at + L):
            for h in range(Hh):
                gi = h // (Hh // G)
                S[h] = want_a[t, h] * S[h] + want_dt[t, h] * B[t, gi].double().unsqueeze(-1) * x[t, h].double().unsqueeze(0)
                ref[t, h] = S[h].T @ C[t, gi].double()
        at += L
    assert float((out.cpu().double().view(T, Hh, P) - ref).abs().max()) <= 3e-5 * max(1.0, float(ref.abs().max()))
    # the gate before the norm, a direct path from the recurrence's input, a norm in parts
    parts = 2 if (Hh * P) % 2 == 0 else 1
    z, skip_w, w = rnd(T, Hh * P).to(dt), rnd(Hh), rnd(Hh * P)
    y = torch.empty(T, Hh * P, dtype=dt, device="cuda:0")
    hipops.gated_group_norm(out, w.cuda(), y, Hh * P // parts, 1e-4, gate=z.cuda(), act="silu", gate_first=True,
                            skip=wide[:, :Hh * P], skip_weight=skip_w.cuda(), skip_group=P)
    v = (out.cpu().double().view(T, Hh, P) + skip_w.double().view(1, Hh, 1) * x.double()).reshape(T, -1) * plain.silu(z.double())
    want = plain.unit_rms(v.view(T, parts, -1), 1e-4).reshape(T, -1) * w.double()
    assert float((y.cpu().double() - want).abs().max()) <= (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(want.abs().max()))


@pytest.mark.gpu
def test_decay_forms_and_small_row_kernels():
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(3)
    z, b = torch.randn(9, 30, generator=g) * 2.0, torch.randn(30, generator=g)
    dev = z.cuda()
    hipops.channel_decay(dev, b.cuda(), form="exp_exp")
    assert float((dev.cpu().double() - torch.exp(-torch.exp(z.double() + b.double()))).abs().max()) < 1e-6
    x = (torch.randn(7, 50, generator=g) * 40.0).cuda()
    want = 15.0 * torch.tanh(x.cpu().double() / 15.0)
    hipops.softcap_rows(x, 15.0)
    assert float((x.cpu().double() - want).abs().max()) < 1e-5
    a, c = torch.randn(5, 12, generator=g).cuda(), torch.randn(5, 12, generator=g).cuda()
    both = torch.empty(5, 24, dtype=torch.bfloat16, device="cuda:0")
    hipops.concat_rows(a, c, both)
    assert torch.equal(both.cpu(), torch.cat([a.cpu(), c.cpu()], 1).to(torch.bfloat16))
    out = torch.empty(5, 12, device="cuda:0")
    hipops.bias_rows(a, c[0].contiguous(), out)
    assert torch.equal(out.cpu(), a.cpu() + c[0].cpu())
    want = 1.3 * a.cpu().double() + 0.6 * c.cpu().double()
    hipops.axpby_rows(a, c, a, 1.3, 0.6)
    assert float((a.cpu().double() - want).abs().max()) < 1e-6
    for act_in in (torch.randn(6, 16, generator=g) * 3.0,):
        w = torch.randn(8, 16, generator=g)
        for dt in (torch.float32, torch.bfloat16):
            from spite_amd.parts.linear import linear, Weight
            y = torch.empty(6, 8, dtype=dt, device="cuda:0")
            linear(act_in.to(dt).cuda(), Weight(w.to(dt).cuda()), y, act="tanh")
            ref = torch.tanh(act_in.to(dt).double() @ w.to(dt).double().T)
            assert float((y.cpu().double() - ref).abs().max()) < (1e-5 if dt == torch.float32 else 2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,D,page", [("float32", 12, 8), ("bfloat16", 64, 32), ("bfloat16", 20, 16)])
def test_prepare_and_attention_kernels(dtype, D, page):
    """Head norm, query temperature and values taken from the keys in the kernel before the cache; slopes and a sink of
    zero in the plain attention kernel (and, for heads of 64, in the matrix-unit kernels): one request, scattered pages."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(D)
    dt = getattr(torch, dtype)
    Hq, G, T, window, scale, eps = 4, 2, 3 * page + 5, page + 3, 0.2, 1e-5
    rows = torch.randn(T, (Hq + G) * D, generator=g).to(dt)
    wq, wk = torch.rand(D, generator=g) + 0.5, torch.rand(D, generator=g) + 0.5
    n_pages = 8
    tiled = hipops.kv_tiled_ok(dt, D, page)
    kp = torch.zeros(n_pages, G, page, D, dtype=dt, device="cuda:0")
    vp = torch.zeros(n_pages, G, D, page, dtype=dt, device="cuda:0")
    table = torch.tensor([[5, 2, 7, 0]], dtype=torch.int32).cuda()
    pos = torch.arange(T, dtype=torch.int32).cuda()
    slot_map = torch.tensor([[5, 2, 7, 0][p // page] * page + p % page for p in range(T)], dtype=torch.int32).cuda()
    q = torch.empty(T, Hq * D, dtype=dt, device="cuda:0")
    hipops.qkv_prepare(rows.cuda(), q, kp, vp, pos, slot_map, Hq, G, G, D, D, page, norm_q=wq.cuda(), norm_k=wk.cuda(), eps=eps,
                       k_tiled=tiled, v_tiled=tiled, head_norm=True, q_temperature=(0.3, 7), values_from_keys=True)
    r = rows.double()
    qq = plain.unit_rms(r[:, :Hq * D].view(T, Hq, D), eps) * wq.double()
    qq = qq * (1.0 + 0.3 * torch.log(torch.floor((torch.arange(T) + 1) / 7).double() + 1.0)).view(T, 1, 1)
    kk = plain.unit_rms(r[:, Hq * D:].view(T, G, D), eps) * wk.double()
    vv = r[:, Hq * D:].view(T, G, D)
    tol = 1e-5 if dtype == "float32" else 3e-2
    assert float((q.cpu().double().view(T, Hq, D) - qq).abs().max()) < tol * float(qq.abs().max())
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / Hq) for h in range(Hq)])
    sinks = torch.zeros(Hq)
    # the plain implementation on what the kernel stored (rounded to the cache's dtype)
    want = plain.softmax_attention(q.cpu().double().view(T, Hq, D), kk.to(dt).double(), vv.to(dt).double(), scale,
                                   sink=sinks.double(), window=window, slopes=slopes.tolist())
    sot = torch.zeros(T, dtype=torch.int32).cuda()
    out = torch.empty(T, Hq * D, dtype=dt, device="cuda:0")
    hipops.attn_wide(q, kp, vp, out, pos, sot, table, T, Hq, G, G, D, D, page, "window", window, scale, k_tiled=tiled, v_tiled=tiled,
                     sinks=sinks.cuda(), slopes=slopes.cuda())
    assert float((out.cpu().double().view(T, Hq, D) - want).abs().max()) < tol * max(1.0, float(want.abs().max()))
    if tiled and D == 64:
        out2 = torch.empty_like(out)
        counts = np.array([T], dtype=np.int32)
        hipops.attn_prefill(q, kp, vp, out2, pos, torch.tensor([0, T], dtype=torch.int32).cuda(), counts, table, Hq, G, D, page,
                            "window", window, scale, sinks=sinks.cuda(), slopes=slopes.cuda())
        assert float((out2.cpu().double().view(T, Hq, D) - want).abs().max()) < tol * max(1.0, float(want.abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_experts_weighted_at_their_input(dtype):
    """The experts part with the weight on the input against the plain form, the engine's own choice taken."""
    from spite_amd.parts.base import PartSpec, build
    from spite_amd.engine.context import Env, Workspace, StepContext
    g = torch.Generator().manual_seed(2)
    dt = getattr(torch, dtype)
    d, F, E, top, Fs, T = 32, 16, 5, 2, 24, 13
    env = Env(dt, torch.device("cuda:0"))
    part = build("ffn", PartSpec("moe_topk_sigmoid", dict(hidden_size=d, intermediate_size=F, n_experts=E, top_k=top,
                 shared_intermediate_size=Fs, score_bias=False, weight_input=True)), env)
    W = {"router": torch.randn(E, d, generator=g)}
    for e in [f"e{i}" for i in range(E)] + ["shared"]:
        f = Fs if e == "shared" else F
        W.update({f"{e}.gate": torch.randn(f, d, generator=g) * 0.3, f"{e}.up": torch.randn(f, d, generator=g) * 0.3,
                  f"{e}.down": torch.randn(d, f, generator=g) * 0.3})
    part.load({k: (v.cuda() if k == "router" else v.to(dt).cuda()) for k, v in W.items()})
    x = torch.randn(T, d, generator=g).to(dt)
    ctx = StepContext(T=T, n_seqs=1, token_ids=None, positions=None, seq_of_token=None, cu_seqlens=None, seq_slots=None,
                      seq_starts=None, logit_rows=None, n_out=0, host=None, ws=Workspace(torch.device("cuda:0")))
    trace = {}
    ctx.extras["trace"] = trace
    (y,) = part.forward(x.cuda(), x.float().cuda(), ctx)
    took = trace["moe_experts"][0].cpu().long()
    Wd = {"p." + k: (v.double() if k == "router" else v.to(dt).double()) for k, v in W.items()}
    want, chosen = plain.experts(x.double(), Wd, "p.", {"router": {"top": top}, "shared": {"ff": Fs}}, take=took)
    assert float((y.cpu().double() - want).abs().max()) < (1e-4 if dtype == "float32" else 5e-2) * float(want.abs().max())
    own, _ = plain.router_choice(x.double(), Wd, "p.", top)
    assert (torch.sort(own, 1).values == torch.sort(took, 1).values).float().mean() > 0.9


# ------------------------------------------------------------------------------------------ the model in the engine
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            folder = tmp_path_factory.mktemp(f"nolapel_{name}_{dtype}")
            kw = {} if dtype == "float32" else dict(gain=1.5, std=0.05)
            made[(name, dtype)] = (folder, make_model(folder, CONFIGS[name], seed=11 + len(name), dtype=dtype, **kw))
        return made[(name, dtype)]
    return get


def _pending_sum(x, pending):
    for p in pending:
        if hasattr(p, "alpha"):                                # what the next norm adds after a tanh norm of its own
            x += p.mult * (torch.tanh(p.alpha * p.y[:x.shape[0]]) * p.weight + p.bias)
        else:
            x += p[:x.shape[0]]
    return x


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "ones"])
def test_every_layer_against_plain(models, name):
    """The stream after each layer run of a whole prompt, in true 32-bit."""
    from spite_amd.engine.engine import StepEntry, StepMeta
    cfg = CONFIGS[name]
    folder, weights = models(name, "float32")
    toks = H.random_tokens(cfg["vocab"], 37, 3)
    streams = []
    plain.forward(toks, weights, cfg, streams=streams)
    eng = engine(folder, "float32", name)
    slot = eng.admit()
    eng.cache.reserve_all([(slot, len(toks))])
    meta = StepMeta(eng, [StepEntry(slot, toks, [0])])
    eng._step_ws.reset()
    m, state = eng.model, {}
    seen = 0
    layer_blocks = len(cfg["layers"])
    for u in range(m.n_units()):
        kind, _, i, _ = m._units[u]
        m.run_units(u, u + 1, state, meta.ctx, eng.cache, meta, eng._arenas, eng._step_ws)
        if kind == "stage" and m._units[u + 1][2] != i and m.spec.order[i].block < layer_blocks:
            x = _pending_sum(state["h"].clone(), state["pending"])
            ref = streams[seen]
            assert float((x.cpu().double() - ref).abs().max()) <= 2e-5 * float(ref.abs().max()), f"layer run {seen}"
            seen += 1
    assert seen == len(streams) == len(plain.layer_order(cfg))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "wide", "ones"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_float32_against_plain(models, name, schedule):
    """True 32-bit: every schedule gives the plain implementation's logits at every position.  Pools and state
    rows start poisoned and are small: pages and slots are used again in the mixed schedule."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "float32")
    reqs = requests(cfg["vocab"], LENGTHS[name], 5)
    ref = plain_rows(cfg, weights, reqs)
    steps = {"whole": H.schedule_whole, "tail": lambda r: H.schedule_tail_one_by_one(r, tail=28),
             "portions": H.schedule_portions, "mixed": lambda r: H.schedule_mixed(r, seed=3, max_live=4)}[schedule](reqs)
    eng = engine(folder, "float32", name, cache_tokens=4 * (max(LENGTHS[name]) + PAGE[name]))
    poison(eng)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
    err, where = H.max_diff(got, ref)
    assert err <= 2e-4 * scale_of(ref), f"{err} at {where} (scale {scale_of(ref)})"
    assert all(eng.cache.free_pages(g) == eng.cache.total_pages(g) for g in range(eng.cache.n_groups()))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "wide"])
def test_bfloat16_against_plain_and_itself(models, name):
    """bfloat16 through the serving kernels: whole prompts against the plain implementation with the experts that
    the engine took, then the other schedules against the whole prompts with those experts."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "bfloat16")
    reqs = requests(cfg["vocab"], LENGTHS[name], 8)
    eng = engine(folder, "bfloat16", name, cache_tokens=4 * (max(LENGTHS[name]) + PAGE[name]))
    if name == "wide":
        assert not eng.slow_paths, eng.slow_paths
    poison(eng)
    whole, routing = H.schedule_whole(reqs), {}
    rows = H.collect(whole, H.run_trace_inprocess(eng, whole, routing=routing), cfg["vocab"])
    experts = experts_of(cfg, whole, routing)
    ref = plain_rows(cfg, weights, reqs, taken=experts)
    scale = scale_of(ref)
    close_in_16_bits(rows, ref, scale, 0.06)
    own = {}
    plain_rows(cfg, weights, reqs, chosen=own)
    total = sum(int(e.numel()) for per in experts.values() for e in per)
    same = sum(int((torch.sort(a, 1).values == torch.sort(b, 1).values).sum()) for r in experts for a, b in zip(experts[r], own[r]))
    assert same >= 0.85 * total
    for steps in (H.schedule_tail_one_by_one(reqs, tail=28), H.schedule_portions(reqs), H.schedule_mixed(reqs, seed=4, max_live=4)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps, take=experts_for(cfg, steps, experts)), cfg["vocab"])
        err, where = H.max_diff(got, rows)
        assert err <= 0.06 * scale, f"{err} at {where} (scale {scale})"


def _one_layer(mixer, mlp=None, width=40, vocab=64, bigram=True):
    cfg = {"architecture": "Nolapel", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "layers": [_layer(mixer, mlp)]}
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": 29, "mul_prev": 5, "mul_cur": 3}}
    return cfg


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
@pytest.mark.parametrize("decoded", [False, True])
def test_window_edges(tmp_path, dtype, wide, decoded):
    """One layer of attention with a window of W over small pages.  The key at j is made of the tokens j - taps .. j
    (the convolution's taps and the hashed pair), so the logits at i do not move at all when token i - W - taps
    changes and move when token i - W - taps + 1 does; in a prompt and when the positions are decoded one by one."""
    W, taps = (40, 3) if wide else (11, 3)
    mixer = _attention(4, 2, 64, 0.125, W, conv=taps, q_temp=(0.3, 16)) if wide else _attention(3, 3, 12, 0.3, W, conv=taps, q_temp=(0.3, 4))
    cfg = _one_layer(mixer, _moe(2, 1, 16, shared=16), width=128 if wide else 40)
    make_model(tmp_path, cfg, seed=2, dtype=dtype, gain=3.0)
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    n = 3 * W + 9
    base = H.random_tokens(64, n, 1)

    def run(toks):
        reqs = {"a": toks}
        steps = H.schedule_tail_one_by_one(reqs, tail=n - W - 7) if decoded else H.schedule_whole(reqs)
        return H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    ref = run(base)
    for i in (2 * W, 2 * W + 1, 3 * W - 1, 3 * W + 8):
        last_out = i - W - taps
        outside, inside = list(base), list(base)
        outside[last_out] = (base[last_out] + 7) % 64
        inside[last_out + 1] = (base[last_out + 1] + 7) % 64
        a, b = run(outside)[("a", i)], run(inside)[("a", i)]
        assert np.array_equal(a, ref[("a", i)]), f"position {i} sees a key outside its window"
        assert float(np.abs(b - ref[("a", i)]).max()) > 1e-4 * float(np.abs(ref[("a", i)]).max()), f"position {i} misses its window's first key"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
def test_one_far_key_stands_out_and_the_sink_counts(tmp_path, dtype, wide):
    """The left half of a parallel mixer, every earlier key visible.  One token stands at position 3 only; another
    stands hundreds of keys later, in the prompt and among the decoded tokens.  On an element that does not turn the
    queries carry their token's part along the second token's normed input and the keys theirs along the first's:
    the second token's query scores the far key far above every other, less what the sink takes, which is planted
    next to that score.  The plain implementation is shown to depend on both first."""
    mixer = _parallel(4, 2, 64, 64, 0.25, (10000.0, 32), 2, 64, ls=1.0, rs=0.05) if wide else _parallel(3, 3, 12, 10, 0.25, (100.0, 8), 2, 6, ls=1.0, rs=0.05)
    cfg = _one_layer(mixer, None, width=128 if wide else 40, bigram=False)
    mx = cfg["layers"][0]["mixer"]["left"]
    Hh, G, D, key_tok, query_tok, gain = mx["heads"], mx["kv_heads"], mx["dim"], 7, 9, 2.5
    t = planted(cfg, 3, gain=1.0)
    Wd = {k: v.double() for k, v in t.items()}
    normed = lambda tok: plain.dyt(Wd["embed"][tok], Wd, "l0.norm1")
    hk, hq = normed(key_tok), normed(query_tok)
    c0 = D - 1                                                      # behind the elements that turn
    for hh in range(Hh):
        t["l0.mix.left.q"][hh * D + c0] = gain * (hq / hq.norm()).float()
    for g in range(G):
        t["l0.mix.left.k"][g * D + c0] = gain * (hk / hk.norm()).float()
    t["l0.mix.left.v"], t["l0.mix.left.o"] = t["l0.mix.left.v"] * 3.0, t["l0.mix.left.o"] * 3.0
    score = mx["scale"] * gain * gain * float(hq.norm()) * float(hk.norm())
    t["l0.mix.left.sink"] = torch.full((Hh,), score - (0.0 if dtype == "float32" else 2.0))
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(tmp_path), cfg, 3, dtype=dtype, overrides=t)
    weights = H.read_weights(str(tmp_path))
    toks = [x if x not in (key_tok, query_tok) else 11 for x in H.random_tokens(64, 330, 9)]
    toks[3] = key_tok
    toks[280], toks[300], toks[320] = query_tok, query_tok, query_tok
    without = list(toks)
    without[3] = 11
    ref, other = plain.forward(toks, weights, cfg), plain.forward(without, weights, cfg)
    scale = float(ref.abs().max())
    assert score > 5 and float((ref[[280, 300, 320]] - other[[280, 300, 320]]).abs().min(0).values.max()) > 0.02 * scale
    nosink = dict(weights)
    nosink["l0.mix.left.sink"] = torch.full((Hh,), -1e30, dtype=torch.float64)
    assert float((plain.forward(toks, nosink, cfg) - ref).abs().max()) > 0.005 * scale
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    poison(eng)
    steps = H.schedule_tail_one_by_one({"a": toks}, tail=40)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    rows = {("a", i): ref[i].float().numpy() for i in range(len(toks))}
    err, where = H.max_diff(got, rows)
    assert err <= (2e-4 if dtype == "float32" else 0.06) * scale, f"{err} at {where} (scale {scale})"


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["time_mix", "state_space"])
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
def test_a_far_token_stays_in_the_state(tmp_path, kind, dtype, wide):
    """Decays next to 1: what the first tokens wrote into the state is still read hundreds of tokens later, through a
    long prompt in one step and more than a hundred tokens decoded one by one.  Changing tokens 1 to 80 moves the last logits
    of the plain implementation, and the engine follows it at every position."""
    if kind == "time_mix":
        mixer = _parallel(2, 1, 64, 64, 0.1, None, 2, 64, ls=0.05, rs=1.0) if wide else _parallel(1, 1, 4, 4, 0.1, None, 3, 6, ls=0.05, rs=1.0)
    else:
        mixer = _ssm(4, 32, 64, 2, 4, 2) if wide else _ssm(3, 10, 6, 3, 3, 1)
    cfg = _one_layer(mixer, None, width=128 if wide else 40)
    t = planted(cfg, 5, gain=2.0)
    if kind == "time_mix":
        t["l0.mix.right.w0"] = torch.full_like(t["l0.mix.right.w0"], -8.0)          # exp(-exp(-8)): 0.9997 a token
        t["l0.mix.right.w2"] = t["l0.mix.right.w2"] * 0.1
    else:
        t["l0.mix.A_log"] = torch.full_like(t["l0.mix.A_log"], -8.0)
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(tmp_path), cfg, 5, dtype=dtype, overrides=t)
    weights = H.read_weights(str(tmp_path))
    toks = H.random_tokens(64, 420, 6)
    other = list(toks)
    for j in range(1, 81):
        other[j] = (toks[j] + 5) % 64
    ref = plain.forward(toks, weights, cfg)
    scale = float(ref.abs().max())
    assert float((plain.forward(other, weights, cfg)[-1] - ref[-1]).abs().max()) > 1e-3 * scale
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    poison(eng)
    steps = H.schedule_tail_one_by_one({"a": toks}, tail=130)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    rows = {("a", i): ref[i].float().numpy() for i in range(len(toks))}
    err, where = H.max_diff(got, rows)
    assert err <= (2e-4 if dtype == "float32" else 0.06) * scale, f"{err} at {where} (scale {scale})"


@pytest.mark.gpu
def test_a_slot_used_again_starts_from_zeros(models):
    """A request that takes the slot (and the pages) of a finished one reads nothing of it: convolution tails, the
    row before, the recurrent states and the previous token all start anew."""
    cfg = CONFIGS["small"]
    folder, weights = models("small", "float32")
    eng = engine(folder, "float32", "small", max_requests=1, cache_tokens=64)
    a, b = H.random_tokens(cfg["vocab"], 40, 1), H.random_tokens(cfg["vocab"], 25, 2)
    for toks in (a, b, a):
        steps = H.schedule_portions({"x": toks}, sizes=(1, 2, 9))
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
        ref = plain_rows(cfg, weights, {"x": toks})
        err, where = H.max_diff(got, ref)
        assert err <= 2e-4 * scale_of(ref), f"{err} at {where}"


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["small", "wide"])
def test_greedy_generation(models, name):
    """Through the engine's own entry point and scheduler: prompts of unequal length, more new tokens than the
    windows are long, in true 32-bit: the plain implementation's greedy tokens."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "float32")
    prompts = [H.random_tokens(cfg["vocab"], n, 40 + n) for n in (1, 19, 7)]
    eng = engine(folder, "float32", name, cache_tokens=512, max_batch_tokens=16)
    n_new = 30 if name == "small" else 10
    got = eng.generate(prompts, max_tokens=n_new, temperature=0.0)
    for p, g in zip(prompts, got):
        toks = list(p)
        for k in range(n_new):
            last = plain.forward(toks, weights, cfg)[-1]
            top = torch.topk(last, 2).values
            if float(top[0] - top[1]) < 1e-3 * float(last.abs().max()):
                break                                              # a tie at 32-bit precision: what follows may differ
            assert g[k] == int(torch.argmax(last)), f"token {k} of a prompt of {len(p)}"
            toks.append(g[k])
        assert k >= 4


@pytest.mark.gpu
def test_decode_steps_replay_graphs(models):
    """Decode steps of one shape are captured and replayed; every replay gives the eager logits (states, convolution
    tails and the previous token move on inside the graph)."""
    cfg = CONFIGS["wide"]
    folder, _ = models("wide", "bfloat16")
    reqs = requests(cfg["vocab"], [40, 41], 21)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:20], "want": [19]} for r, t in reqs.items()], "end": []}]
    steps += [{"step": 1 + i, "entries": [{"id": r, "tokens": [t[20 + i]], "want": [0]} for r, t in reqs.items()], "end": []} for i in range(20)]
    outs = []
    for graphs in (False, True):
        eng = engine(folder, "bfloat16", "wide", graphs=graphs)
        outs.append(H.run_trace_inprocess(eng, copy.deepcopy(steps)))
        assert (eng.graph_replays > 10) == graphs
    for k in outs[0]:
        assert np.array_equal(outs[0][k], outs[1][k]), f"step {k}"


def random_config(seed, aligned=False):
    """A configuration drawn from a seed: layer count and order, the loop, heads, sizes, windows, taps and constants
    all vary; now and then a value is 1 or sizes are odd.  ``aligned``: sizes that the bfloat16 runs take on the
    matrix units in one kernel or another."""
    rng = np.random.RandomState(seed)
    pick = lambda *xs: xs[rng.randint(len(xs))]
    layers = []
    for _ in range(int(pick(1, 2, 3, 5))):
        kind = pick("attention", "parallel", "mamba2")
        if aligned:
            dim = int(pick(32, 64, 64, 128))
            mlp = pick(None, _moe(int(pick(2, 4, 8)), int(pick(1, 2)), int(pick(32, 64)), pick(None, 32, 64)))
        else:
            dim = int(pick(2, 6, 8, 12, 20))
            mlp = pick(None, _moe(int(pick(1, 3, 5)), 1, int(pick(4, 12)), pick(None, 8)), _moe(int(pick(3, 6)), int(pick(2, 3)), 8, pick(None, 4, 12)))
        kv = int(pick(1, 2, 3))
        heads = kv * int(pick(1, 2, 4))
        if kind == "attention":
            mixer = _attention(heads, kv, dim, float(pick(0.1, 0.25, 0.5)), pick(None, 1, 2, 7, 24, 33, 64), conv=int(pick(0, 2, 3, 4)),
                               q_temp=pick(None, (float(pick(0.1, 0.5)), int(pick(1, 8, 50)))))
        elif kind == "parallel":
            vdim = int(pick(32, 64, 128)) if aligned else int(pick(2, 3, 10, 16))
            dims = int(pick(*[x for x in (2, 4, 8, 16, 32, dim) if x <= dim and x % 2 == 0]))
            mixer = _parallel(heads, kv, dim, vdim, float(pick(0.1, 0.25)), pick(None, (float(pick(100.0, 10000.0, 1e6)), dims)),
                              int(pick(1, 2, 4)), int(pick(16, 32, 64)) if aligned else int(pick(2, 5, 8, 12)),
                              ls=float(pick(1.0, 1.3, 0.5)), rs=float(pick(1.0, 0.8)))
        else:
            groups = int(pick(1, 2))
            h = groups * int(pick(1, 2, 3))
            vdim = int(pick(16, 32, 64)) if aligned else int(pick(2, 5, 8))
            ng = int(pick(*[x for x in (1, 2, h) if (h * vdim) % x == 0]))
            mixer = _ssm(h, vdim, int(pick(16, 64, 128)) if aligned else int(pick(2, 6, 16)), groups, int(pick(1, 2, 4)), ng)
        layers.append(_layer(mixer, mlp))
    cfg = {"architecture": "Nolapel", "vocab": int(pick(50, 128, 257)), "width": int(pick(64, 128, 192)) if aligned else int(pick(24, 37, 48, 64)),
           "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    if pick(True, True, False):
        cfg["embedding"] = {"bigram": {"buckets": int(pick(1, 13, 101)), "mul_prev": int(pick(1, 31, 1000003)), "mul_cur": int(pick(1, 7, 99991))}}
    if pick(True, True, False):
        a = int(rng.randint(len(layers)))
        cfg["loop"] = {"start": a, "stop": int(a + 1 + rng.randint(len(layers) - a)), "times": int(pick(1, 2, 3))}
    if pick(True, False):
        cfg["logit_softcap"] = float(pick(5.0, 40.0))
    return cfg


@pytest.mark.gpu
@pytest.mark.parametrize("seed", list(range(8)) + list(range(100, 108)))
def test_random_configurations(tmp_path, seed):
    """Whatever the configuration says: true 32-bit against the plain implementation, whole prompts and a mixed
    schedule through small pages; then bfloat16 against itself across schedules and, loosely, against the plain
    implementation."""
    cfg = random_config(seed, aligned=seed >= 100)
    page = int(np.random.RandomState(seed + 100).choice([4, 16, 32, 64]))
    weights = make_model(tmp_path / "f32", cfg, seed=seed, dtype="float32", gain=2.0)
    reqs = requests(cfg["vocab"], [41, 1, 70, 2, 19], seed)
    ref = plain_rows(cfg, weights, reqs)
    from spite_amd import Engine
    eng = Engine(str(tmp_path / "f32"), dtype="float32", page_size=page, cache_tokens=4 * (70 + page), max_requests=4, device="cuda:0")
    poison(eng)
    for steps in (H.schedule_whole(reqs), H.schedule_mixed(reqs, seed=seed, max_live=4)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab"])
        err, where = H.max_diff(got, ref)
        assert err <= 3e-4 * scale_of(ref), f"{err} at {where} (scale {scale_of(ref)}): {cfg}"
    del eng
    weights = make_model(tmp_path / "bf16", cfg, seed=seed, dtype="bfloat16", gain=1.5, std=0.05)
    eng = Engine(str(tmp_path / "bf16"), dtype="bfloat16", page_size=page, cache_tokens=4 * (70 + page), max_requests=4, device="cuda:0")
    poison(eng)
    whole, routing = H.schedule_whole(reqs), {}
    rows = H.collect(whole, H.run_trace_inprocess(eng, whole, routing=routing), cfg["vocab"])
    experts = experts_of(cfg, whole, routing) if expert_runs(cfg) else None
    ref = plain_rows(cfg, weights, reqs, taken=experts)
    scale = scale_of(ref)
    close_in_16_bits(rows, ref, scale, 0.08)
    steps = H.schedule_mixed(reqs, seed=seed + 1, max_live=4)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps, take=experts_for(cfg, steps, experts) if experts else None), cfg["vocab"])
    err, where = H.max_diff(got, rows)
    assert err <= 0.08 * scale, f"{err} at {where} (scale {scale}): {cfg}"


@pytest.mark.gpu
def test_replay_program(models):
    """The replay program on a model folder, as a child process: a mixed schedule in true 32-bit gives the plain
    implementation's logits."""
    cfg = CONFIGS["small"]
    folder, weights = models("small", "float32")
    reqs = requests(cfg["vocab"], [30, 1, 47, 12, 22], 77)
    steps = H.schedule_mixed(reqs, seed=9, max_live=4)
    out = H.run_trace_program(str(folder), "float32", steps, max_tokens=4 * 64, extra=["--page-size", "16", "--max-requests", "4"])
    got = H.collect(steps, out, cfg["vocab"])
    ref = plain_rows(cfg, weights, reqs)
    err, where = H.max_diff(got, ref)
    assert err <= 2e-4 * scale_of(ref), f"{err} at {where}"


@pytest.mark.gpu
def test_command_line_and_sampling(models):
    """`spite run` on the model's folder: the greedy tokens of `Engine.generate`; and sampling with a seed through the
    framework's sampler gives the same tokens twice and other tokens than greedy somewhere."""
    cfg = CONFIGS["small"]
    folder, _ = models("small", "float32")
    p = H.random_tokens(cfg["vocab"], 9, 21)
    eng = engine(folder, "float32", "small", cache_tokens=256)
    want = eng.generate([p], max_tokens=12, temperature=0.0)[0]
    out = subprocess.run([sys.executable, os.path.join(H.ROOT, "bin", "spite"), "run", "-m", str(folder), "--prompt-ids",
                          ",".join(map(str, p)), "--max-tokens", "12", "--temperature", "0", "--dtype", "fp32",
                          "--ctx", "64", "--page-size", "16"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in want]
    a = eng.generate([p, p[:4]], max_tokens=12, temperature=1.0, seed=5)
    b = eng.generate([p, p[:4]], max_tokens=12, temperature=1.0, seed=5)
    assert a == b and a[0] != want
