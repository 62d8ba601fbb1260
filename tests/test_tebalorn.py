"""The Tebalorn design in the engine against the plain implementation (``plain_tebalorn``): every
mechanism's kernel alone, whole prompts, decoding through the state rows and the cache, portions down to
two tokens, mixed batches with pages and slots used again, chunk edges, far tokens, sinks, the first
tokens, generation."""
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
import plain_tebalorn as plain


# ------------------------------------------------------------------------------------------ configurations
def _gla(heads, dim, vdim, tau):
    return "gla", {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}


def _lightning(heads, dim, vdim, decay):
    assert len(decay) == heads
    return "lightning", {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def _attention(heads, kv, dim, vdim, scale, chunk, base=10000.0, dims=None, yarn=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
         "rot": {"base": base, "dims": dim if dims is None else dims}}
    if yarn is not None:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), yarn))
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return "attention", m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff},
            "shared": None if shared is None else {"ff": shared}}


def _layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


# odd sizes that no fast kernel takes; every kind of mixer and feed-forward, a layer without one
SMALL = {"architecture": "Tebalorn", "vocab": 96, "width": 40, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
         "logit_scale": 0.5, "token_side": {"dim": 6},
         "layers": [_layer(_gla(3, 6, 10, 8.0), _moe(5, 2, 12, shared=20)),
                    _layer(_attention(4, 2, 12, 10, 0.3, 9, base=100.0, dims=8, yarn=(4.0, 16, 4.0, 1.0)), _dense(24)),
                    _layer(_lightning(2, 8, 6, [0.9, 0.99]), None),
                    _layer(_attention(3, 3, 8, 6, 0.4, None), _moe(4, 1, 8)),
                    _layer(_gla(1, 18, 4, 1.0), _dense(16)),
                    _layer(_lightning(4, 4, 12, [1.0, 0.5, 0.75, 0.97]), _moe(3, 3, 8, shared=8))]}
# sizes that the matrix-unit kernels take in bfloat16 (heads of 64 and 128, pages of 32)
WIDE = {"architecture": "Tebalorn", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
        "logit_scale": 2.0, "token_side": {"dim": 32},
        "layers": [_layer(_lightning(2, 32, 128, [0.95, 0.999]), _moe(4, 2, 64, shared=64)),
                   _layer(_attention(4, 2, 64, 64, 0.125, 40, dims=32, yarn=(8.0, 64, 8.0, 0.5)), _dense(128)),
                   _layer(_gla(2, 64, 64, 12.0), _moe(6, 3, 32)),
                   _layer(_attention(2, 1, 64, 128, 0.2, None, base=1000.0), _dense(64))]}
# values that are 1, equal or absent where the other configurations have them apart
ONES = {"architecture": "Tebalorn", "vocab": 50, "width": 24, "norm": {"eps": 1e-3},
        "layers": [_layer(_attention(1, 1, 2, 2, 1.0, 1, dims=2, yarn=(1.0, 8, 2.0, 1.0)), _moe(1, 1, 8)),
                   _layer(_gla(1, 2, 2, 1.0), None),
                   _layer(_lightning(1, 2, 2, [1.0]), _dense(24)),
                   _layer(_attention(5, 1, 4, 4, 0.5, 2), _moe(2, 2, 4, shared=4))]}
CONFIGS = {"small": SMALL, "wide": WIDE, "ones": ONES}
PAGE = {"small": 16, "wide": 32, "ones": 4}
LENGTHS = {"small": [1, 45, 23, 60, 2, 31, 17], "wide": [90, 1, 140, 33, 75], "ones": [30, 1, 44, 9]}


def planted(cfg, seed, gain=3.0, std=0.08, rank=5):
    """Random tensors with sharper attention, routers that tell experts apart, sinks of the size of a
    score, decay biases that spread the decays over (0, 1), and a decay of inner width ``rank``."""
    from spite_amd.weights.random_init import random_tensors
    t = random_tensors(cfg, seed, std)
    g = torch.Generator().manual_seed(seed)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}.mix."
        if L["type"] == "attention":
            t[p + "q"] = t[p + "q"] * gain
            t[p + "sink"] = torch.randn(t[p + "sink"].shape, generator=g) * 1.5
        elif L["type"] == "gla":
            d, n = cfg["width"], L["mixer"]["heads"] * L["mixer"]["dim"]
            t[p + "a1"] = torch.randn(rank, d, generator=g) * 0.3
            t[p + "a2"] = torch.randn(n, rank, generator=g) * 0.5
            t[p + "a2.b"] = torch.randn(n, generator=g) * 2.0 + 2.0
            t[p + "q"] = t[p + "q"] * gain
        else:
            t[p + "q"] = t[p + "q"] * gain
        if p + "norm" in t:
            t[p + "norm"] = 1.0 + 0.3 * torch.randn(t[p + "norm"].shape, generator=g)
        if L["mlp"] and L["mlp"]["kind"] == "moe":
            t[f"l{i}.mlp.router"] = t[f"l{i}.mlp.router"] * 8.0
    return t


def make_model(folder, cfg, seed, dtype, **kw):
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(folder), cfg, seed, dtype=dtype, overrides=planted(cfg, seed, **kw))
    return H.read_weights(str(folder))


def requests(vocab, lengths, seed):
    return {f"r{i}": H.random_tokens(vocab, n, seed + 13 * i) for i, n in enumerate(lengths)}


def moe_layers(cfg):
    return [i for i, L in enumerate(cfg["layers"]) if L["mlp"] and L["mlp"]["kind"] == "moe"]


def plain_rows(cfg, weights, reqs, taken=None, chosen=None):
    """{(request, position): logits}; ``taken``: {request: {layer: experts [T, top]}} to take;
    ``chosen`` receives what was taken, in the same form."""
    rows = {}
    for rid, toks in reqs.items():
        got = {}
        out = plain.forward(cfg, weights, toks, taken=None if taken is None else taken[rid], chosen=got).to(torch.float32).numpy()
        if chosen is not None:
            chosen[rid] = got
        for i in range(len(toks)):
            rows[(rid, i)] = out[i]
    return rows


def experts_of(cfg, steps, routing):
    """{request: {layer: experts [T, top]}} from what a replay recorded step by step."""
    layers, parts = moe_layers(cfg), {}
    for rec in steps:
        off = 0
        for e in rec["entries"]:
            n = len(e["tokens"])
            for k, L in enumerate(layers):
                parts.setdefault(e["id"], {}).setdefault(L, []).append(np.asarray(routing[rec["step"]][k]).reshape(-1, cfg["layers"][L]["mlp"]["router"]["top"])[off:off + n])
            off += n
    return {rid: {L: torch.from_numpy(np.concatenate(v).astype(np.int64)) for L, v in per.items()} for rid, per in parts.items()}


def experts_for(cfg, steps, experts):
    """{step: [experts of the step's tokens, one array per layer with experts]}: ``experts`` cut as ``steps`` cuts."""
    layers, fed, take = moe_layers(cfg), {}, {}
    for rec in steps:
        per = [[] for _ in layers]
        for e in rec["entries"]:
            at, n = fed.get(e["id"], 0), len(e["tokens"])
            for k, L in enumerate(layers):
                per[k].append(experts[e["id"]][L][at:at + n].numpy())
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
    """Every cache row and every state row holds NaN until it is written or cleared."""
    for g in eng.cache.groups:
        for half in g.halves():
            if half is not None and half.numel():
                half.fill_(float("nan"))
    for st in eng.cache.states.values():
        st.fill_(float("nan"))


def rows_over(a, b, limit):
    """The rows of ``a`` that differ from ``b``'s by more than ``limit`` somewhere."""
    return [k for k in a if not float(np.max(np.abs(a[k].astype(np.float64) - b[k].astype(np.float64)))) <= limit]


def close_in_16_bits(rows, ref, scale, tol):
    """bfloat16 against the plain implementation: every row within 4 ``tol``, all but one in fifty within ``tol``.
    (A head's normed result is a sign times a unit vector wherever the state holds one outer product only, and
    its size does not matter wherever a norm follows: where q . k is next to nothing, its rounding decides.
    The 32-bit runs hold every row.)"""
    far, near = rows_over(rows, ref, 4 * tol * scale), rows_over(rows, ref, tol * scale)
    assert not far and len(near) <= max(1, len(rows) // 50), f"{len(near)} of {len(rows)} rows over {tol * scale}, {far[:3]} far over (scale {scale})"


def scale_of(rows):
    return max(float(np.abs(v).max()) for v in rows.values())


# ------------------------------------------------------------------------------------------ without a GPU
def test_registry_and_tensor_names():
    from spite_amd.config import read_config
    from spite_amd.config.tebalorn import TebalornConfig
    from spite_amd.engine.model import Model
    from spite_amd.engine.context import Env
    arch, cfg = read_config(SMALL)
    assert arch.name == "Tebalorn" and isinstance(cfg, TebalornConfig)
    assert cfg.layers[1].mixer.rot_scaling.factor == 4.0 and cfg.layers[3].mixer.chunk is None and cfg.layers[2].mlp is None
    assert cfg.layers[5].mixer.decay == (1.0, 0.5, 0.75, 0.97) and cfg.layers[0].mlp.shared_ff == 20 and cfg.layers[3].mlp.shared_ff is None
    model = Model(arch.build_spec(cfg), Env(torch.float32, torch.device("cpu")))
    names = {n: ps.shape for n, ps, _, _ in model.tensor_plan()}
    assert {"embed", "side.embed", "final.norm", "head", "l0.mix.a1", "l0.mix.a2", "l0.mix.a2.b", "l0.mix.g", "l0.mix.norm",
            "l1.mix.sink", "l0.mlp.router", "l0.mlp.e4.down", "l0.mlp.shared.up", "l1.mlp.gate", "l5.side.proj", "l2.side.norm"} <= set(names)
    assert "l2.mlp.up" not in names and "l3.mlp.shared.up" not in names and "l1.mix.g" not in names and "l2.mix.a1" not in names
    assert "l0.norm2" not in names
    assert names["l0.mix.q"] == (18, 40) and names["l0.mix.v"] == (30, 40) and names["l0.mix.norm"] == (10,)
    assert names["l2.mix.norm"] == (12,) and names["l1.mix.k"] == (24, 40) and names["l1.mix.v"] == (20, 40) and names["l1.mix.sink"] == (4,)
    assert names["side.embed"] == (96, 6 * 6) and names["l4.side.gate"] == (6, 40) and names["l4.side.proj"] == (40, 6)
    needs = model.cache_needs()
    kinds = [(n.kv is not None, n.state is not None) for n in needs]
    assert kinds == [(False, True), (True, False), (False, True), (True, False), (False, True), (False, True)]
    assert needs[0].state.shape == (3, 6, 10) and needs[4].state.shape == (1, 18, 4) and needs[0].state.dtype == torch.float32
    assert needs[1].kv.visibility == "chunk" and needs[1].kv.span == 9 and needs[3].kv.visibility == "full"
    assert needs[1].kv.head_dim == 12 and needs[1].kv.value_dim == 10


def test_config_errors_are_collected():
    from spite_amd.config import read_config, ConfigError
    bad = copy.deepcopy(SMALL)
    del bad["vocab"]
    bad["layers"][0]["mixer"]["tau"] = 0.0
    bad["layers"][1]["mixer"]["kv_heads"] = 3
    bad["layers"][1]["mixer"]["rot"]["dims"] = 7
    bad["layers"][2]["mixer"]["decay"] = [0.5]
    bad["layers"][3]["mlp"]["router"]["top"] = 9
    bad["layers"][4]["type"] = "other"
    bad["layers"][5]["mlp"]["kind"] = "sparse"
    with pytest.raises(ConfigError) as e:
        read_config(bad)
    msg = str(e.value)
    for word in ("vocab", "tau", "kv_heads", "rot.dims", "decay", "router.top", "type", "kind"):
        assert word in msg, word


def test_plain_mechanisms():
    g = torch.Generator().manual_seed(0)
    T, Hh, D, V = 7, 2, 3, 4
    q, k, a = (torch.rand(T, Hh, D, generator=g, dtype=torch.float64) for _ in range(3))
    v = torch.rand(T, Hh, V, generator=g, dtype=torch.float64)
    o, S = plain.recurrence(q, k, v, a)
    # the same as a sum over the earlier tokens, each key decayed by the product of the decays since
    for t in (0, 3, 6):
        want = torch.zeros(Hh, V, dtype=torch.float64)
        for s in range(t + 1):
            w = k[s].clone()
            for r in range(s + 1, t + 1):
                w = w * a[r]
            want += (w * q[t]).sum(-1, keepdim=True) * v[s]
        assert float((o[t] - want).abs().max()) < 1e-12
    assert S.shape == (Hh, D, V)
    sc = torch.tensor([[0.0, 1.0, 2.0]], dtype=torch.float64)
    ok = torch.tensor([[True, True, False]])
    w = plain.sink_softmax(sc, ok, 0.5)
    den = 1.0 + math.e + math.exp(0.5)
    assert float((w - torch.tensor([[1.0 / den, math.e / den, 0.0]], dtype=torch.float64)).abs().max()) < 1e-12
    assert abs(float(plain.sink_softmax(sc, ok, -1e30).sum()) - 1.0) < 1e-12
    assert plain.visible(torch.arange(7), 3)[5].tolist() == [False, False, False, True, True, True, False]
    assert plain.visible(torch.arange(4), None)[2].tolist() == [True, True, True, False]
    f, mag = plain.rotation_table({"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}})
    # pair 0 turns more than 4 times in 16 positions and keeps its frequency; the others are divided by 4
    assert abs(float(f[0]) - 1.0) < 1e-12 and abs(float(f[1]) - 100.0 ** -0.25 / 4.0) < 1e-12 and abs(float(f[3]) - 100.0 ** -0.75 / 4.0) < 1e-12
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    x = torch.arange(6, dtype=torch.float64).view(1, 1, 6)
    y = plain.turn(x, torch.tensor([2]), {"base": 100.0, "dims": 4})
    assert abs(float(y[0, 0, 0]) - (0 * math.cos(2.0) - 2 * math.sin(2.0))) < 1e-12 and torch.equal(y[0, 0, 4:], x[0, 0, 4:])
    assert abs(float(y[0, 0, 3]) - (3 * math.cos(0.2) + 1 * math.sin(0.2))) < 1e-12
    Wr = {"mlp.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]], dtype=torch.float64)}
    idx, wt = plain.route(torch.tensor([[2.0, 1.0]], dtype=torch.float64), Wr, "mlp.", {"router": {"top": 2}})
    assert idx.tolist() == [[2, 0]] and abs(float(wt[0, 0]) - 1.0 / (1.0 + math.exp(-1.0))) < 1e-12
    assert abs(float(plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["channel", "head"])
@pytest.mark.parametrize("Hh,D,V,lens", [(3, 6, 10, [5, 1, 2, 1]), (2, 64, 64, [150, 1, 67]), (1, 130, 20, [33]), (2, 32, 128, [64, 128]),
                                         (4, 128, 128, [1, 1, 1, 1]), (1, 256, 72, [40, 3])])
def test_linear_attention_kernel(dtype, kind, Hh, D, V, lens):
    """Portions and single tokens of several requests in two steps through state rows that lie apart: the
    second step goes on from what the first left, nobody reads or writes another slot's row."""
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(D + V)
    dt = getattr(torch, dtype)
    n = len(lens)
    slots = [3, 0, 5, 2][:n]
    state = torch.full((6, Hh, D, V), float("nan"))
    state[slots] = 0.0
    state = state.cuda()
    full = [2 * L for L in lens]
    rnd = lambda *s: torch.randn(*s, generator=g)
    q = [(rnd(L, Hh, D) * 0.5).to(dt) for L in full]
    k = [(rnd(L, Hh, D) * 0.5).to(dt) for L in full]
    v = [rnd(L, Hh, V).to(dt) for L in full]
    if kind == "channel":
        a = [torch.sigmoid(rnd(L, Hh, D) * 2.0 + 3.0) for L in full]
        head_decay = None
    else:
        hd = torch.tensor([1.0, 0.9, 0.5, 0.999][:Hh])
        a = [hd.view(1, Hh, 1).expand(L, Hh, D) for L in full]
        head_decay = hd.cuda()
    q_scale = 0.37
    want = [plain.recurrence(q[i].double() * q_scale, k[i].double(), v[i].double(), a[i].double()) for i in range(n)]
    scale = max(float(w[0].abs().max()) for w in want)
    tol = 2e-5 if dtype == "float32" else 2e-5          # the inputs are rounded before both; the sums are 32-bit in both
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32).cuda()
    sl = torch.tensor(slots, dtype=torch.int32).cuda()
    for step in range(2):
        cut = lambda xs: torch.cat([x[step * L:(step + 1) * L] for x, L in zip(xs, lens)])
        T = sum(lens)
        # q, k and v as column ranges of one wider matrix, as the mixer has them
        row = torch.cat([cut(q).reshape(T, -1), cut(k).reshape(T, -1), cut(v).reshape(T, -1)], dim=1).cuda()
        HD, HV = Hh * D, Hh * V
        out = torch.full((T, HV), float("nan"), device="cuda:0")
        dec = cut(a).reshape(T, -1).float().contiguous().cuda() if kind == "channel" else None
        hipops.linear_attn_scan(row[:, :HD], row[:, HD:2 * HD], row[:, 2 * HD:], out, state, cu, sl, n, Hh, D, V,
                                decay=dec, head_decay=head_decay, q_scale=q_scale)
        ref = torch.cat([w[0][step * L:(step + 1) * L] for w, L in zip(want, lens)]).reshape(T, HV)
        err = float((out.cpu().double() - ref).abs().max())
        assert err <= tol * scale, f"step {step}: {err} (scale {scale})"
    last = torch.stack([w[1] for w in want])
    assert float((state[slots].cpu().double() - last).abs().max()) <= tol * max(1.0, float(last.abs().max()))
    others = [s for s in range(6) if s not in slots]
    assert bool(torch.isnan(state[others]).all())


@pytest.mark.gpu
def test_linear_attention_kernel_keeps_nothing_when_told():
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(1)
    Hh, D, V, T = 2, 16, 16, 40
    state = torch.randn(2, Hh, D, V, generator=g).cuda()
    before = state.clone()
    row = torch.randn(T, 3 * Hh * D, generator=g).cuda()
    out = torch.empty(T, Hh * V, device="cuda:0")
    hipops.linear_attn_scan(row[:, :32], row[:, 32:64], row[:, 64:], out, state, torch.tensor([0, T], dtype=torch.int32).cuda(),
                            torch.tensor([1], dtype=torch.int32).cuda(), 1, Hh, D, V, head_decay=torch.tensor([0.9, 0.8]).cuda(), keep=False)
    assert torch.equal(state, before) and bool(torch.isfinite(out).all())


@pytest.mark.gpu
@pytest.mark.parametrize("tau", [1.0, 20.0, 0.5])
def test_channel_decay_kernel(tau):
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(3)
    z = torch.cat([torch.randn(9, 30, generator=g) * 4.0, torch.tensor([[-60.0, 60.0, 0.0] * 10])])
    b = torch.randn(30, generator=g)
    want = torch.sigmoid(z.double() + b.double()) ** (1.0 / tau)
    dev = z.cuda()
    hipops.channel_decay(dev, b.cuda(), tau)
    got = dev.cpu().double()
    assert float((got - want).abs().max()) < 3e-6
    # close to 1 the distance from 1 keeps its leading digits
    near = want > 0.99
    assert float(((1 - got[near]) - (1 - want[near])).abs().max()) < 2e-7


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,group,n_w,act", [(30, 10, 10, "silu"), (24, 24, 24, "sigmoid"), (256, 128, 128, "silu"), (96, 96, 96, None), (1300, 1300, 1300, "sigmoid"), (2048, 1024, 1024, "silu")])
def test_norm_and_gate_kernel(dtype, n, group, n_w, act):
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(n)
    dt = getattr(torch, dtype)
    T, eps = 11, 1e-3
    o = torch.randn(T, n, generator=g) * 3.0
    w = torch.rand(n_w, generator=g) + 0.5
    wide = torch.randn(T, n + 7, generator=g).to(dt)
    y = torch.empty(T, n, dtype=dt, device="cuda:0")
    hipops.gated_group_norm(o.cuda(), w.cuda(), y, group, eps, gate=wide.cuda()[:, 5:5 + n] if act else None, act=act)
    want = plain.unit_rms(o.double().view(T, n // group, group), eps).view(T, n) * w.double().repeat(n // n_w)
    gate = wide[:, 5:5 + n].double()
    if act == "silu":
        want = want * plain.silu(gate)
    elif act == "sigmoid":
        want = want * torch.sigmoid(gate)
    assert float((y.cpu().double() - want).abs().max()) < (1e-5 if dtype == "float32" else 2e-2) * max(1.0, float(want.abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("E,top", [(5, 2), (12, 2), (3, 3), (1, 1), (70, 4)])
def test_router_takes_the_largest_and_weighs_them_among_themselves(E, top):
    from spite_amd.csrc import hipops
    g = torch.Generator().manual_seed(E)
    T = 19
    z = torch.randn(T, E, generator=g) * 3.0
    expert = torch.empty(T * top, dtype=torch.int32, device="cuda:0")
    weight = torch.empty(T * top, device="cuda:0")
    hipops.router_topk(z.cuda(), None, expert, weight, top, scoring="softmax_taken")
    val, idx = torch.topk(z.double(), top, dim=-1)
    want = torch.softmax(val, dim=-1)
    got_e, got_w = expert.cpu().view(T, top).long(), weight.cpu().view(T, top).double()
    order = torch.argsort(got_e, dim=1)
    worder = torch.argsort(idx, dim=1)
    assert torch.equal(got_e.gather(1, order), idx.gather(1, worder))
    assert float((got_w.gather(1, order) - want.gather(1, worder)).abs().max()) < 1e-6
    assert float((got_w.sum(1) - 1.0).abs().max()) < 1e-6


@pytest.mark.gpu
def test_rotation_table_in_the_engine():
    """The engine's frequencies and magnitude are the plain implementation's, for scaled and unscaled tables."""
    from spite_amd.parts.position import inv_frequencies, rotation_magnitude
    for rot in ({"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}},
                {"base": 300000.0, "dims": 48, "scaling": {"factor": 16.0, "original": 1000, "fast": 20.0, "slow": 2.0}},
                {"base": 10000.0, "dims": 6}):
        sc = rot.get("scaling")
        scaling = None if sc is None else dict(sc, rope_type="yarn")
        f, mag = plain.rotation_table(rot)
        got = torch.tensor(inv_frequencies(rot["dims"], rot["base"], scaling), dtype=torch.float64)
        assert float((got / f - 1).abs().max()) < 1e-12 and abs(rotation_magnitude(scaling) - mag) < 1e-12


# ------------------------------------------------------------------------------------------ the model in the engine
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            folder = tmp_path_factory.mktemp(f"tebalorn_{name}_{dtype}")
            kw = {} if dtype == "float32" else dict(gain=1.5, std=0.05)
            if name == "wide":
                kw["rank"] = 16                                    # an inner width that the matrix units take
            made[(name, dtype)] = (folder, make_model(folder, CONFIGS[name], seed=11 + len(name), dtype=dtype, **kw))
        return made[(name, dtype)]
    return get


@pytest.mark.gpu
def test_every_layer_against_plain(models):
    """The stream after each layer of a whole prompt, in true 32-bit."""
    from spite_amd.engine.engine import StepEntry, StepMeta
    cfg = SMALL
    folder, weights = models("small", "float32")
    toks = H.random_tokens(cfg["vocab"], 37, 3)
    eng = engine(folder, "float32", "small")
    slot = eng.admit()
    eng.cache.reserve_all([(slot, len(toks))])
    meta = StepMeta(eng, [StepEntry(slot, toks, [0])])
    eng._step_ws.reset()
    m, state = eng.model, {}
    seen = 0
    for u in range(m.n_units()):
        kind, _, i, _ = m._units[u]
        m.run_units(u, u + 1, state, meta.ctx, eng.cache, meta, eng._arenas, eng._step_ws)
        if kind == "stage" and m._units[u + 1][2] != i:
            x = state["h"].clone()
            for p in state["pending"]:
                if hasattr(p, "weight"):                           # what the next norm adds after a norm of its own
                    y = p.y[:x.shape[0]]
                    x += p.mult * y / torch.sqrt((y * y).mean(-1, keepdim=True) + p.eps) * p.weight
                else:
                    x += p[:x.shape[0]]
            ref = plain.forward(cfg, weights, toks, upto=i + 1)
            assert float((x.cpu().double() - ref).abs().max()) <= 2e-5 * float(ref.abs().max()), f"layer {i}"
            seen += 1
    assert seen == len(cfg["layers"])


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
    """bfloat16 through the serving kernels: whole prompts against the plain implementation with the experts
    that the engine took (their weights are still the plain implementation's own), then the other schedules
    against the whole prompts with those experts."""
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
    close_in_16_bits(rows, ref, scale, 0.05)
    # the engine's choice is the plain implementation's own nearly everywhere
    own = {}
    plain_rows(cfg, weights, reqs, chosen=own)
    total = sum(int(e.numel()) for per in experts.values() for e in per.values())
    same = sum(int((torch.sort(experts[r][L], 1).values == torch.sort(own[r][L], 1).values).sum()) for r in experts for L in experts[r])
    assert same >= 0.9 * total
    for steps in (H.schedule_tail_one_by_one(reqs, tail=28), H.schedule_portions(reqs), H.schedule_mixed(reqs, seed=4, max_live=4)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps, take=experts_for(cfg, steps, experts)), cfg["vocab"])
        err, where = H.max_diff(got, rows)
        assert err <= 0.05 * scale, f"{err} at {where} (scale {scale})"


def _one_layer(mixer, mlp=None, width=40, vocab=64, side=None):
    cfg = {"architecture": "Tebalorn", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
           "layers": [_layer(mixer, mlp)]}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
@pytest.mark.parametrize("decoded", [False, True])
def test_chunk_edges(tmp_path, dtype, wide, decoded):
    """One layer of attention with chunks of 11 (40 in bfloat16) over pages of 8 (32): the logits at i do not move
    at all when the last token of the chunk before changes, and move when the chunk's own first token does; in a
    prompt and when the positions are decoded one by one."""
    C = 40 if wide else 11
    mixer = _attention(4, 2, 64, 64, 0.125, C, dims=32, yarn=(4.0, 32, 4.0, 1.0)) if wide else _attention(3, 3, 12, 10, 0.3, C, dims=8)
    cfg = _one_layer(mixer, _dense(32), width=128 if wide else 40)
    make_model(tmp_path, cfg, seed=2, dtype=dtype, gain=3.0)
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    n = 3 * C + 5
    base = H.random_tokens(64, n, 1)

    def run(toks):
        reqs = {"a": toks}
        steps = H.schedule_tail_one_by_one(reqs, tail=n - C - 3) if decoded else H.schedule_whole(reqs)
        return H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    ref = run(base)
    for i in (2 * C, 2 * C + 1, 3 * C - 1, 3 * C + 4):
        first = i // C * C
        outside, inside = list(base), list(base)
        outside[first - 1] = (base[first - 1] + 7) % 64
        inside[first] = (base[first] + 7) % 64
        a, b = run(outside)[("a", i)], run(inside)[("a", i)]
        assert np.array_equal(a, ref[("a", i)]), f"position {i} sees the chunk before"
        assert float(np.abs(b - ref[("a", i)]).max()) > 1e-4 * float(np.abs(ref[("a", i)]).max()), f"position {i} misses its chunk's first key"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
def test_one_far_key_stands_out_and_the_sink_counts(tmp_path, dtype, wide):
    """One token stands at position 3 only; another stands hundreds of keys later, in the prompt and among the
    decoded tokens.  On an element that does not turn, the queries carry their token's part along the second
    token's normed embedding and the keys theirs along the first's: the second token's query scores the far key
    far above every other, so the result there is the far key's value, less what the sink takes, which is planted
    next to that score.  The test shows both on the plain implementation first."""
    mixer = _attention(4, 2, 64, 64, 0.25, None, dims=32, yarn=(2.0, 128, 8.0, 1.0)) if wide else _attention(3, 3, 12, 10, 0.25, None, dims=8)
    cfg = _one_layer(mixer, None, width=128 if wide else 40)
    mx = cfg["layers"][0]["mixer"]
    Hh, G, D, key_tok, query_tok, gain = mx["heads"], mx["kv_heads"], mx["dim"], 7, 9, 1.5
    t = planted(cfg, 3, gain=1.0)
    normed = lambda tok: plain.norm(t["embed"][tok].double() * cfg["embedding"]["scale"], t["l0.norm1"].double(), cfg["norm"]["eps"])
    hk, hq = normed(key_tok), normed(query_tok)
    c0 = D - 1                                                      # behind the elements that turn
    for hh in range(Hh):
        t["l0.mix.q"][hh * D + c0] = gain * (hq / hq.norm()).float()
    for g in range(G):
        t["l0.mix.k"][g * D + c0] = gain * (hk / hk.norm()).float()
    t["l0.mix.v"], t["l0.mix.o"] = t["l0.mix.v"] * 3.0, t["l0.mix.o"] * 3.0     # what attention adds is as large as the stream
    score = mx["scale"] * gain * gain * float(hq.norm()) * float(hk.norm())     # the second token's query on the first's key
    t["l0.mix.sink"] = torch.full((Hh,), score - (0.0 if dtype == "float32" else 2.0))
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(tmp_path), cfg, 3, dtype=dtype, overrides=t)
    weights = H.read_weights(str(tmp_path))
    toks = [x if x not in (key_tok, query_tok) else 11 for x in H.random_tokens(64, 330, 9)]
    toks[3] = key_tok
    toks[280], toks[300], toks[320] = query_tok, query_tok, query_tok
    without = list(toks)
    without[3] = 11
    ref, other = plain.forward(cfg, weights, toks), plain.forward(cfg, weights, without)
    scale = float(ref.abs().max())
    assert score > 20 and float((ref[[280, 300, 320]] - other[[280, 300, 320]]).abs().min(0).values.max()) > 0.05 * scale      # the far key decides
    nosink = dict(weights)
    nosink["l0.mix.sink"] = torch.full((Hh,), -1e30, dtype=torch.float64)
    assert float((plain.forward(cfg, nosink, toks) - ref).abs().max()) > 0.01 * scale                   # and the sink counts
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    if wide:
        assert not eng.slow_paths, eng.slow_paths
    poison(eng)
    steps = H.schedule_tail_one_by_one({"a": toks}, tail=40)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    rows = {("a", i): ref[i].float().numpy() for i in range(len(toks))}
    err, where = H.max_diff(got, rows)
    assert err <= (2e-4 if dtype == "float32" else 0.05) * scale, f"{err} at {where} (scale {scale})"


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["gla", "lightning"])
@pytest.mark.parametrize("dtype,wide", [("float32", False), ("bfloat16", True)])
def test_a_far_token_stays_in_the_state(tmp_path, kind, dtype, wide):
    """Decays at or next to 1: what the first tokens wrote into the state is still read hundreds of tokens later,
    through a long prompt in one step and more than a hundred tokens decoded one by one.  Changing token 2 moves
    the last logits of the plain implementation, and the engine follows it at every position."""
    Hh, D, V = (2, 64, 64) if wide else (3, 6, 10)
    if kind == "gla":
        mixer = _gla(Hh, D, V, 64.0)
    else:
        mixer = _lightning(Hh, D, V, [1.0, 0.9995, 0.999][:Hh])
    cfg = _one_layer(mixer, None, width=128 if wide else 40, side=4)
    t = planted(cfg, 5, gain=2.0)
    if kind == "gla":
        t["l0.mix.a2.b"] = torch.full_like(t["l0.mix.a2.b"], 4.0)      # sigmoid(4)^(1/64): 0.9997 a token
        t["l0.mix.a2"] = t["l0.mix.a2"] * 0.1
    from spite_amd.weights.random_init import write_random_model
    write_random_model(str(tmp_path), cfg, 5, dtype=dtype, overrides=t)
    weights = H.read_weights(str(tmp_path))
    toks = H.random_tokens(64, 420, 6)
    other = list(toks)
    other[2] = (toks[2] + 5) % 64
    ref = plain.forward(cfg, weights, toks)
    scale = float(ref.abs().max())
    assert float((plain.forward(cfg, weights, other)[-1] - ref[-1]).abs().max()) > 1e-3 * scale
    from spite_amd import Engine
    eng = Engine(str(tmp_path), dtype=dtype, page_size=32 if wide else 8, cache_tokens=512, max_requests=2, device="cuda:0")
    poison(eng)
    steps = H.schedule_tail_one_by_one({"a": toks}, tail=130)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps), 64)
    rows = {("a", i): ref[i].float().numpy() for i in range(len(toks))}
    err, where = H.max_diff(got, rows)
    assert err <= (2e-4 if dtype == "float32" else 0.05) * scale, f"{err} at {where} (scale {scale})"


@pytest.mark.gpu
def test_a_slot_used_again_starts_from_zeros(models):
    """A request that takes the slot (and the pages) of a finished one reads nothing of it: its first token's
    state is zero, whatever the slot's state rows held."""
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
    chunks are long, in true 32-bit: the plain implementation's greedy tokens."""
    cfg = CONFIGS[name]
    folder, weights = models(name, "float32")
    prompts = [H.random_tokens(cfg["vocab"], n, 40 + n) for n in (1, 19, 7)]
    eng = engine(folder, "float32", name, cache_tokens=512, max_batch_tokens=16)
    n_new = 40 if name == "small" else 12
    got = eng.generate(prompts, max_tokens=n_new, temperature=0.0)
    for p, g in zip(prompts, got):
        toks = list(p)
        for k in range(n_new):
            last = plain.forward(cfg, weights, toks)[-1]
            top = torch.topk(last, 2).values
            if float(top[0] - top[1]) < 1e-3 * float(last.abs().max()):
                break                                              # a tie at 32-bit precision: what follows may differ
            assert g[k] == plain.greedy(last), f"token {k} of a prompt of {len(p)}"
            toks.append(g[k])
        assert k >= 5


@pytest.mark.gpu
def test_decode_steps_replay_graphs(models):
    """Decode steps of one shape are captured and replayed; every replay gives the eager logits (the state
    rows move on inside the graph)."""
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
    """A configuration drawn from a seed: layer count and order, heads, sizes, chunks, bases, scaling and
    constants all vary; now and then a value is 1 or sizes are odd.  ``aligned``: sizes in multiples of 8,
    32 and 64, which the bfloat16 runs take on the matrix units in one kernel or another."""
    rng = np.random.RandomState(seed)
    pick = lambda *xs: xs[rng.randint(len(xs))]
    layers = []
    for _ in range(int(pick(1, 2, 3, 5))):
        kind = pick("gla", "lightning", "attention")
        if aligned:
            dim, vdim = int(pick(32, 64, 64, 128)), int(pick(32, 64, 64, 128))
            mlp = pick(None, _dense(int(pick(64, 128, 200))), _moe(int(pick(2, 4, 8)), int(pick(1, 2)), int(pick(32, 64)), pick(None, 32, 64)))
        else:
            dim, vdim = int(pick(2, 6, 8, 12, 20)), int(pick(2, 3, 4, 10, 16))
            mlp = pick(None, _dense(int(pick(8, 20, 32))), _moe(int(pick(1, 3, 5)), 1, int(pick(4, 12)), pick(None, 8)),
                       _moe(int(pick(3, 6)), int(pick(2, 3)), 8, pick(None, 4, 12)))
        if kind == "attention":
            kv = int(pick(1, 2, 3))
            dims = int(pick(*[x for x in (2, 4, 8, 16, 32, dim) if x <= dim and x % 2 == 0]))
            yarn = pick(None, (float(pick(1.0, 2.0, 6.0)), int(pick(16, 64, 256)), float(pick(4.0, 16.0)), float(pick(0.5, 2.0))))
            mixer = _attention(kv * int(pick(1, 2, 4)), kv, dim, vdim, float(pick(0.1, 0.25, 0.5)), pick(None, 1, 2, 7, 24, 33, 64),
                               base=float(pick(100.0, 10000.0, 500000.0)), dims=dims, yarn=yarn)
        elif kind == "gla":
            mixer = _gla(int(pick(1, 2, 3)), dim, vdim, float(pick(1.0, 4.0, 10.0)))
        else:
            heads = int(pick(1, 2, 5))
            mixer = _lightning(heads, dim, vdim, [float(pick(1.0, 0.999, 0.9, 0.6, 0.0)) for _ in range(heads)])
        layers.append(_layer(mixer, mlp))
    cfg = {"architecture": "Tebalorn", "vocab": int(pick(50, 128, 257)), "width": int(pick(64, 128, 192)) if aligned else int(pick(24, 37, 48, 64)),
           "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    if pick(True, True, False):
        cfg["embedding"] = {"scale": float(pick(1.0, 4.0, 10.0))}
    if pick(True, False):
        cfg["logit_scale"] = float(pick(0.2, 1.0, 3.0))
    if pick(True, True, False):
        cfg["token_side"] = {"dim": int(pick(8, 16, 32)) if aligned else int(pick(1, 3, 8))}
    return cfg


@pytest.mark.gpu
@pytest.mark.parametrize("seed", list(range(8)) + list(range(100, 108)))
def test_random_configurations(tmp_path, seed):
    """Whatever the configuration says: true 32-bit against the plain implementation, whole prompts and a mixed
    schedule through small pages; then bfloat16 against itself across schedules and, loosely, against the plain
    implementation."""
    cfg = random_config(seed, aligned=seed >= 100)
    page = int(np.random.RandomState(seed + 100).choice([4, 16, 32, 64]))
    weights = make_model(tmp_path / "f32", cfg, seed=seed, dtype="float32", gain=2.0, rank=int(np.random.RandomState(seed).choice([1, 3, 16])))
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
    experts = experts_of(cfg, whole, routing) if moe_layers(cfg) else None
    ref = plain_rows(cfg, weights, reqs, taken=experts)
    scale = scale_of(ref)
    close_in_16_bits(rows, ref, scale, 0.08)
    steps = H.schedule_mixed(reqs, seed=seed + 1, max_live=4)
    got = H.collect(steps, H.run_trace_inprocess(eng, steps, take=experts_for(cfg, steps, experts) if experts else None), cfg["vocab"])
    err, where = H.max_diff(got, rows)
    assert err <= 0.08 * scale, f"{err} at {where} (scale {scale}): {cfg}"


@pytest.mark.gpu
def test_replay_program(models):
    """The replay program on a model folder, as a child process: a mixed schedule in true 32-bit gives the
    plain implementation's logits."""
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
    """`spite run` on the model's folder: the greedy tokens of `Engine.generate`; and sampling with a seed through
    the framework's sampler gives the same tokens twice and other tokens than greedy somewhere."""
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
