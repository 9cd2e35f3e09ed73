"""Pumozen through the engine against the plain implementation in ``pumozen_oracle.py``:
each mechanism alone, prefill against token-by-token decoding, portions, mixed batches,
reuse of pages and state slots, far keys and page borders, the first tokens of a sequence,
long decoding, other sizes, and greedy generation through ``submit`` / ``step``.

Every case runs on the CPU (the ops' fp32 forms, the same engine, cache manager and
scheduler) and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import io
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import pumozen_oracle as O
from k8s_llm_rca_amd.engine.engine import EngineConfig, LLMEngine
from k8s_llm_rca_amd.models.pumozen import PumozenConfig, PumozenModel
from k8s_llm_rca_amd.ops import moe as M
from k8s_llm_rca_amd.ops import norm as N
from k8s_llm_rca_amd.ops import seq_ops as S

GPU = pytest.mark.gpu
BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=GPU),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=GPU)]
MFMA_BACKEND = [pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=GPU)]
DT = torch.float64
STALE = 2.0 ** 15     # what unwritten page entries hold in these tests (exact in bfloat16)


def row_errs(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def agrees(got, want, dtype, mult=1.0):
    """Logits rows against the oracle's.  fp32 (the sharp check): every row; a row whose sublayer output is nearly
    constant has its rounding noise magnified by that output's layer norm, hence a bound on the median and a wider
    one on the worst row (a wrong key, a lost state or a sink left out moves a row by 1e-2 and more).  bf16: every
    sublayer's output is normed to unit size before it is added, so each of a model's ~20 sublayers adds its own
    rounding (about 1 % of a row a few dozen channels wide) at full weight, and a router's near-tie may go the other
    way, which moves that row a lot: most rows must be close, few far off, none unrelated (two unrelated rows differ
    by about 1.4).  The bf16 runs guard the plumbing of that type; the sharp comparisons are the fp32 ones and, for
    the kernels that only bf16 has, the tests of the single mechanisms above."""
    e = row_errs(got, want)
    if dtype == torch.float32:
        return float(e.median()) < 2e-5 * mult and float(e.max()) < 4e-4 * mult
    return (float(e.median()) < 0.15 * mult and float(e.max()) < 1.1
            and int((e > 0.4 * mult).sum()) <= max(1, 0.15 * e.numel()))


def close(got, want, dtype, scale=1.0):
    """Element-wise check of an op's output against fp64."""
    got, want = got.double().cpu(), want.double().cpu()
    t = (2e-5 if dtype == torch.float32 else 2e-2) * scale
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err < t, err


# ------------------------------------------------------------------ configurations and weights
def att(heads=6, kv_heads=3, dim=8, scale=None, rot=4, base=300.0, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5 if scale is None else scale}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def dif(heads=4, kv_heads=2, dim=8, vdim=12, scale=None, diff=0.35, coef=0.4, every=7, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
         "scale": dim ** -0.5 if scale is None else scale}
    if every:
        m["q_temp"] = {"coef": coef, "every": every}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention_2", "mixer": m}


def mam(heads=6, vdim=4, state=8, groups=3, conv=4, norm_groups=2):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def dense(ff=40, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff=16, limit=0.8, experts=5, top=2, scale=1.7, shared=24, shared_limit=2.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale},
            "shared": {"ff": shared, "limit": shared_limit} if shared else None}


def config(layers, width=48, vocab=512, eps=1e-5, side=6):
    d = {"architecture": "Pumozen", "vocab": vocab, "width": width,
         "layers": [dict(mix, mlp=mlp) for mix, mlp in layers], "norm": {"eps": eps}}
    if side:
        d["token_side"] = {"dim": side}
    return d


def default_config(**kw):
    return config([(dif(), moe()), (mam(), dense()), (att(), moe(top=1, shared=0)), (dif(kv_from=0), None),
                   (att(heads=2, kv_heads=2, dim=6, rot=6, kv_from=None), dense(ff=24, limit=0.7)),
                   (mam(heads=2, vdim=8, state=5, groups=1, conv=2, norm_groups=1), moe(experts=3, top=3)),
                   (att(kv_from=2), dense())], **kw)


def weights(d, seed=0):
    """Random weights under the checkpoint's names, rounded to bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W = d["width"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def lin(o, i, mul=1.0):
        return r(o, i, std=mul * i ** -0.5)

    t = {"embed": r(d["vocab"], W)}
    side = (d.get("token_side") or {}).get("dim", 0)
    if side:
        t["side.embed"] = r(d["vocab"], side * len(d["layers"]))

    def norm(name):
        t[name], t[name + ".b"] = r(W, std=0.2, mean=1.0), r(W, std=0.1)

    def unit(p, ff):
        t[p + "gate"], t[p + "up"], t[p + "down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff)

    norm("final.norm")
    for i, L in enumerate(d["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        norm(f"l{i}.norm1")
        if L["type"] == "attention":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            t[p + "q"], t[p + "o"] = lin(H * D, W), lin(W, H * D)
            t[p + "q.norm"] = r(H * D, std=0.3, mean=1.5)
            if m.get("kv_from") is None:
                t[p + "k"], t[p + "k.norm"] = lin(G * D, W), r(G * D, std=0.3, mean=1.5)
        elif L["type"] == "attention_2":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[p + "q"], t[p + "o"], t[p + "g"] = lin(2 * H * D, W), lin(W, H * V), lin(H * V, W, 2.0)
            t[p + "q.norm"] = r(D, std=0.3, mean=1.5)
            for n_ in ("lq1", "lk1", "lq2", "lk2"):
                t[p + n_] = r(D, std=0.25)
            if m.get("kv_from") is None:
                t[p + "k"], t[p + "v"] = lin(2 * G * D, W), lin(G * V, W)
                t[p + "k.norm"] = r(D, std=0.3, mean=1.5)
        else:
            H, P, Ns, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            ch = H * P + 2 * G * Ns
            t[p + "in"] = lin(H * P + ch + H, W)
            t[p + "conv"], t[p + "conv.b"] = r(ch, taps, std=0.6), r(ch, std=0.2)
            t[p + "dt_bias"], t[p + "A_log"] = r(H, std=0.5, mean=-0.5), r(H, std=0.5, mean=-0.5)
            t[p + "D"], t[p + "norm"], t[p + "o"] = r(H, std=0.3, mean=1.0), r(H * P, std=0.2, mean=1.0), lin(W, H * P)
        f = L["mlp"]
        if f is not None:
            q = f"l{i}.mlp."
            norm(f"l{i}.norm2")
            if f["kind"] == "dense":
                unit(q, f["ff"])
            else:
                t[q + "router"] = lin(f["router"]["experts"], W, 3.0)
                for e in range(f["router"]["experts"]):
                    unit(q + f"e{e}.", f["expert"]["ff"])
                if f.get("shared"):
                    unit(q + "shared.", f["shared"]["ff"])
                    t[q + "shared.sg"] = lin(1, W, 3.0)
        if side:
            t[f"l{i}.side.gate"], t[f"l{i}.side.proj"] = lin(side, W, 2.0), lin(W, side)
            t[f"l{i}.side.norm"] = r(W, std=0.2, mean=0.6)
    return t


def engine(d, W, backend, num_blocks=24, block_size=32, slots=4, **kw):
    dev, dt = backend
    model = PumozenModel(PumozenConfig.from_json(d, "test"), dev, dt, init=False)
    model.load_tensors(W.__getitem__)
    cfg = dict(model="test", device=dev, dtype=dt, num_blocks=num_blocks, block_size=block_size, state_slots=slots,
               max_batch_tokens=1024, use_graphs=False, temperature=0.0)
    cfg.update(kw)
    eng = LLMEngine(EngineConfig(**cfg), model=model)
    for t in eng.states.t.values():       # a fresh slot must not be read: make a read loud
        t.fill_(float("nan"))
    for c in eng.kv.kc + eng.kv.vc + [t for t in eng.kv.vt if t is not None]:
        c.fill_(STALE)                    # stale pages hold finite garbage (a masked key's weight is 0)
    return eng


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def feed_all(eng, sid, tokens, cuts):
    """Feed ``tokens`` in portions ``cuts`` (the rest one by one); logits of every position."""
    out, at = [], 0
    for n in list(cuts) + [1] * len(tokens):
        if at >= len(tokens):
            break
        n = min(n, len(tokens) - at)
        out.append(eng.feed([(sid, tokens[at:at + n], list(range(n)))]))
        at += n
    return torch.cat(out)


def seg_meta(lens, pos0, slots, dev, block_tables=None):
    row0 = [0]
    for n in lens:
        row0.append(row0[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)  # noqa: E731
    row_seg = [s for s, n in enumerate(lens) for _ in range(n)]
    bt = i32(block_tables if block_tables is not None else [[0]] * len(lens))
    return S.SegMeta(len(lens), i32(row_seg), i32(row0), i32(pos0), i32(slots), bt, row0, list(pos0), list(slots),
                     n_single=0)


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=DT) * std


def in_portions(fn, total, cuts):
    out, at = [], 0
    for n in list(cuts) + [total]:
        if at >= total:
            break
        e = min(total, at + n)
        out.append(fn(at, e))
        at = e
    return torch.cat(out)


def f32(z, dev):
    return None if z is None else z.float().to(dev)


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("W", [6, 48, 300, 1024])
def test_output_norms_on_the_residual(backend, W):
    """x + LN(y), x + LN(y + sigmoid(g) y2), x + rms(y) w, each with the new rows as activations; the embedding
    rows; the per-token gate."""
    dev, dt = backend
    T, eps = 7, 1e-3
    x, y, y2 = rnd(T, W, seed=1, std=2.0), rnd(T, W, seed=2, std=5.0) + 0.7, rnd(T, W, seed=3)
    w, b, rg = rnd(W, seed=4) + 1.0, rnd(W, seed=5, std=0.3), rnd(T, 3, seed=6, std=2.0)
    X, Y, Y2, Wt, B, RG = (f32(v, dev) for v in (x, y, y2, w, b, rg))
    xin = X.clone()
    h = N.ln_residual(xin, Y, Wt, B, eps, xin, out_dtype=dt, cast=True)
    want = x + O.layer_norm(y, w, b, eps)
    close(xin, want, torch.float32)
    close(h, want, dt)
    xin = X.clone()
    h = N.ln_residual(xin, Y, Wt, B, eps, xin, y2=Y2, merge="gated", row_gate=RG[:, 1:2], out_dtype=dt, cast=True)
    want = x + O.layer_norm(y + torch.sigmoid(rg[:, 1:2]) * y2, w, b, eps)
    close(xin, want, torch.float32)
    close(h, want, dt)
    xin = X.clone()
    h = N.ln_residual(xin, Y, Wt, None, eps, xin, kind="rms", out_dtype=dt, cast=True)
    want = x + O.unit_rms(y, eps) * w
    close(xin, want, torch.float32)
    close(h, want, dt)
    xin = X.clone()
    assert N.ln_residual(xin, Y, Wt, B, eps, xin) is None               # no activations asked for
    close(xin, x + O.layer_norm(y, w, b, eps), torch.float32)
    emb = rnd(20, W, seed=13).to(torch.bfloat16)
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32, device=dev)
    x0 = torch.empty(4, W, device=dev)
    h = N.embed_rows(ids, emb.to(dev).to(dt), x0, out_dtype=dt)
    close(x0, emb.double()[ids.cpu().long()], torch.float32)
    close(h, emb.double()[ids.cpu().long()], dt)
    n = min(W, 5)
    a = rnd(4, n, seed=7, std=2.0)
    got = N.token_gate(f32(a, dev), ids, emb.to(dev).to(dt), W - n, dt)
    close(got, O.gelu_tanh(a) * emb.double()[ids.cpu().long()][:, W - n:], dt)


def slots_of(order, BS, a, e, dev):
    p = torch.arange(a, e)
    return (torch.tensor(order)[p // BS] * BS + p % BS).to(torch.int32).to(dev)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,rot", [(6, 3, 8, 4), (3, 3, 6, 6), (2, 1, 16, 0), (5, 1, 70, 32), (40, 8, 400, 64),
                                       (3, 0, 10, 4)])
def test_preparation_with_a_norm_over_the_whole_projection(backend, H, G, D, rot):
    """q and k normed over all their heads at once, THEN rotated (far from position 0); the values are the keys as
    projected; G = 0: queries only."""
    dev, dt = backend
    T, BS, eps, base = 9, 8, 1e-3, 777.0
    pos = torch.tensor([0, 1, 2, 3, 4, 5, 70001, 70002, 70003])
    x = rnd(T, H * D + G * D + 3, seed=H + D, std=2.0)                  # a column slice of something wider
    qw, kw = rnd(H * D, seed=4) + 1.5, (rnd(G * D, seed=5) + 1.5 if G else None)
    q = O.rotate((O.unit_rms(x[:, :H * D], eps) * qw).view(T, H, D), pos, rot, base)
    order = [2, 0, 1]
    sl = torch.tensor([order[i // BS] * BS + i % BS for i in range(T)], dtype=torch.int32, device=dev)
    kc = vc = vt = None
    if G:
        kc = torch.full((3, BS, G * D), STALE, device=dev, dtype=dt)
        vc = torch.full((3, BS, G * D), STALE, device=dev, dtype=dt)
        vt = torch.full((3, G * D, BS), STALE, device=dev, dtype=dt)
    got = S.attn_prep(f32(x, dev)[:, :-3], None, H, G, D, D, pos.to(torch.int32).to(dev), sl, kc, vc, dt, norm="all",
                      q_w=f32(qw, dev), k_w=f32(kw, dev), eps=eps, rot_dims=rot, rot_base=base, vt=vt, v_is_k=bool(G))
    close(got, q.reshape(T, -1), dt)
    if G:
        kr = x[:, H * D:H * D + G * D]
        k = O.rotate((O.unit_rms(kr, eps) * kw).view(T, G, D), pos, rot, base)
        close(kc.view(-1, G * D)[sl.long()], k.reshape(T, -1), dt)
        close(vc.view(-1, G * D)[sl.long()], kr, dt)
        close(vt[sl.long() // BS, :, sl.long() % BS], kr, dt)
        assert float(kc[1].float().min()) == STALE and float(vc[0, 1:].float().min()) == STALE   # nothing else written


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V,every", [(4, 2, 8, 12, 7), (3, 3, 6, 5, 1), (2, 1, 16, 8, 0), (1, 1, 70, 3, 200),
                                           (2, 0, 8, 4, 3)])
def test_preparation_of_two_score_maps(backend, H, G, D, V, every):
    """Every (head, map) of q and k normed by itself with one shared weight; the query temperature steps with
    floor((p + 1) / every); values behind the keys."""
    dev, dt = backend
    T, BS, eps, coef = 9, 8, 1e-3, 0.45
    pos = torch.tensor([0, 1, 5, 6, 7, 13, 198, 199, 70003])
    nq, nk, nv = 2 * H * D, 2 * G * D, G * V
    x = rnd(T, nq + nk + nv + 2, seed=H + D, std=2.0)
    qw, kw = rnd(D, seed=4) + 1.5, rnd(D, seed=5) + 1.5
    q = O.unit_rms(x[:, :nq].view(T, H, 2, D), eps) * qw
    if every:
        q = q * (1.0 + coef * torch.log(torch.div(pos + 1, every, rounding_mode="floor").double() + 1.0))[:, None, None, None]
    order = [1, 2, 0]
    sl = torch.tensor([order[i // BS] * BS + i % BS for i in range(T)], dtype=torch.int32, device=dev)
    kc = vc = None
    if G:
        kc = torch.full((3, BS, nk), STALE, device=dev, dtype=dt)
        vc = torch.full((3, BS, nv), STALE, device=dev, dtype=dt)
    got = S.attn_prep(f32(x, dev)[:, :nq + nk + nv], None, H, G, D, V, pos.to(torch.int32).to(dev), sl, kc, vc, dt,
                      norm="head", q_w=f32(qw, dev), k_w=f32(kw, dev) if G else None, eps=eps, maps=2,
                      q_temp=(coef, every) if every else None)
    close(got, q.reshape(T, -1), dt)
    if G:
        k = O.unit_rms(x[:, nq:nq + nk].view(T, G, 2, D), eps) * kw
        close(kc.view(-1, nk)[sl.long()], k.reshape(T, -1), dt)
        close(vc.view(-1, nv)[sl.long()], x[:, nq + nk:nq + nk + nv], dt)


def attention_case(dev, dt, H, G, D, V, n, BS, seed, maps=1, sharp=None, with_twin=False):
    """Random q / k / v for one sequence, the keys and values in shuffled pages.  ``sharp`` = (i, j): key j is
    made to stand out for query i (in every map)."""
    q, k, v = rnd(n, H, maps, D, seed=seed), rnd(n, G, maps, D, seed=seed + 1), rnd(n, G, V, seed=seed + 2)
    if sharp is not None:
        i, j = sharp
        q[i] = q[i, 0, 0]                                     # every head and map asks the same
        k[j] = 8.0 * q[i, 0, 0] / q[i, 0, 0].norm()
    q, k, v = (z.to(torch.bfloat16).double() for z in (q, k, v))
    n_pages = -(-n // BS)
    order = torch.randperm(n_pages + 2, generator=torch.Generator().manual_seed(seed)).tolist()[:n_pages]
    kc = torch.full((n_pages + 2, BS, G * maps * D), STALE, device=dev, dtype=dt)
    vc = torch.full((n_pages + 2, BS, G * V), STALE, device=dev, dtype=dt)
    sl = slots_of(order, BS, 0, n, dev).long()
    kc.view(-1, G * maps * D)[sl] = k.reshape(n, -1).to(dev).to(dt)
    vc.view(-1, G * V)[sl] = v.reshape(n, -1).to(dev).to(dt)
    vt = None
    if with_twin:                 # the values' transposed twin: the matrix-core kernel runs where it takes the sizes
        vt = torch.full((n_pages + 2, G * V, BS), STALE, device=dev, dtype=dt)
        vt[sl // BS, :, sl % BS] = v.reshape(n, -1).to(dev).to(dt)
    return q, k, v, kc, vc, [list(order)], vt


def maps_attention(q, k, v, scale, sink):
    """[n, H, M, V]: every map's causal softmax attention over its head's values, in float64."""
    n, H, Mm, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, Mm, v.shape[-1], dtype=DT)
    for h in range(H):
        g = h // (H // G)
        for m in range(Mm):
            out[:, h, m] = O.causal_weights(q[:, h, m] @ k[:, g, m].T * scale, sink=sink) @ v[:, g]
    return out


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V,maps", [(4, 2, 8, 12, 2), (3, 3, 5, 3, 2), (6, 1, 32, 16, 2), (1, 1, 64, 70, 2),
                                          (12, 4, 16, 200, 2), (6, 3, 8, 8, 1), (2, 2, 5, 5, 3)])
def test_attention_with_score_maps_over_shuffled_pages(backend, H, G, D, V, maps):
    """One map with the zero sink (the 'attention' mixer), two or three maps in fp32 (the differential one);
    whole, in portions and token by token."""
    dev, dt = backend
    n, BS, scale = 75, 16, 0.45
    q, k, v, kc, vc, bt, _ = attention_case(dev, dt, H, G, D, V, n, BS, seed=maps + H, maps=maps)
    sink = maps == 1
    want = maps_attention(q, k, v, scale, sink)
    qd = q.reshape(n, -1).to(dev).to(dt)
    sk = torch.zeros(H, device=dev) if sink else None
    for cuts in [(n,), (40, 1, 1, 2, 30), (3, 70)]:
        def run(a, e):
            sg = seg_meta([e - a], [a], [0], dev, bt)
            return S.masked_attention(qd[a:e].contiguous(), H, G, D, V, kc, vc, sg, scale, sink=sk, maps=maps,
                                      out_f32=maps > 1)
        got = in_portions(run, n, cuts)
        assert got.dtype == (torch.float32 if maps > 1 else dt)
        close(got, want.reshape(n, -1), dt)


@pytest.mark.parametrize("backend", MFMA_BACKEND)
@pytest.mark.parametrize("H,G,D,V,maps", [(4, 2, 64, 64, 2), (3, 1, 128, 64, 2), (9, 3, 64, 128, 2), (2, 2, 128, 128, 2),
                                          (1, 1, 64, 64, 2), (8, 2, 128, 128, 1), (3, 3, 64, 64, 1)])
@pytest.mark.parametrize("split", [True, False])
def test_score_maps_on_the_matrix_cores(backend, H, G, D, V, maps, split, monkeypatch):
    """The sizes the matrix-core kernel takes: tiles of 16 tokens, portions that start inside a tile's span,
    decoding token by token, with and without the split of a tile's key blocks over workgroups; two sequences."""
    dev, dt = backend
    if not split:
        monkeypatch.setattr(S, "WINDOW_SPLIT_ITEMS", 0)
    n, BS, scale = 330, 32, 0.25
    q, k, v, kc, vc, bt, vt = attention_case(dev, dt, H, G, D, V, n, BS, seed=maps + H, maps=maps, with_twin=True)
    assert S.masked_mfma_ok(H, G, D, V, dt, dev)
    sink = maps == 1
    want = maps_attention(q, k, v, scale, sink).reshape(n, -1)
    qd = q.reshape(n, -1).to(dev).to(dt)
    kw = dict(sink=torch.zeros(H, device=dev) if sink else None, maps=maps, out_f32=maps > 1, vt=vt)
    for cuts in [(n,), (40, 1, 1, 2, 30, 17), (3, 270), (319,) + (1,) * 11]:
        def run(a, e):
            return S.masked_attention(qd[a:e].contiguous(), H, G, D, V, kc, vc, seg_meta([e - a], [a], [0], dev, bt),
                                      scale, **kw)
        close(in_portions(run, n, cuts), want, dt)
    sg = seg_meta([5, n - 100], [n - 5, 100], [0, 1], dev, bt + bt)
    got = S.masked_attention(torch.cat([qd[n - 5:], qd[100:]]).contiguous(), H, G, D, V, kc, vc, sg, scale, **kw)
    close(got, torch.cat([want[n - 5:], want[100:]]), dt)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("aim", ["far", "page_last", "page_first", "self", "future"])
@pytest.mark.parametrize("maps,D,V", [(1, 16, 16), (2, 16, 8), (2, 64, 64), (1, 128, 128)])
def test_one_key_stands_out(backend, aim, maps, D, V):
    """One key draws nearly all of query i's weight: the output shows at once whether it was seen.  Query 300 as
    part of the whole prompt, of a portion, and decoded alone; keys far back, at both sides of a page border, the
    query's own, and the one just behind it (which no one may see)."""
    dev, dt = backend
    H, G, n, BS, i = 4, 2, 302, 32, 300
    j = {"far": 1, "page_last": 255, "page_first": 256, "self": 300, "future": 301}[aim]
    q, k, v, kc, vc, bt, vt = attention_case(dev, dt, H, G, D, V, n, BS, seed=3, maps=maps, sharp=(i, j),
                                             with_twin=dev == "cuda" and dt == torch.bfloat16)
    want = maps_attention(q, k, v, 1.0, sink=maps == 1)
    share = (want[i] - v[j].repeat_interleave(H // G, 0)[:, None]).abs().max()
    assert (share < 0.2) == (aim != "future")                            # the case is what its name says
    qd = q.reshape(n, -1).to(dev).to(dt)
    kw = dict(sink=torch.zeros(H, device=dev) if maps == 1 else None, maps=maps, out_f32=maps > 1, vt=vt)
    for a, e in ((0, n), (290, n), (i, i + 1)):                          # whole prompt, a portion, decoded alone
        got = S.masked_attention(qd[a:e].contiguous(), H, G, D, V, kc, vc, seg_meta([e - a], [a], [0], dev, bt), 1.0, **kw)
        close(got[i - a], want[i].reshape(-1), dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_zero_sink_takes_its_share(backend):
    """Scores far below 0: nearly all weight goes to the sink and the output vanishes; far above: the sink does not
    show.  Without a sink the first token's weight on itself is 1 whatever the score."""
    dev, dt = backend
    H, G, D, V, n = 2, 1, 8, 8, 5
    q, k, v, kc, vc, bt, _ = attention_case(dev, dt, H, G, D, V, n, 8, seed=5)
    q[:] = q[0, 0, 0]
    k[:] = q[0, 0, 0]                                                    # every q.k = |q|^2 > 0
    kc.view(-1, D)[slots_of(bt[0], 8, 0, n, dev).long()] = k.reshape(n, -1).to(dev).to(dt)
    sg = seg_meta([n], [0], [0], dev, bt)
    zero = torch.zeros(H, device=dev)
    qd = q.reshape(n, -1).to(dev).to(dt)
    low = S.masked_attention(qd, H, G, D, V, kc, vc, sg, -30.0, sink=zero).double().cpu()
    assert float(low.abs().max()) < 1e-6
    close(S.masked_attention(qd, H, G, D, V, kc, vc, sg, 0.2, sink=zero), maps_attention(q, k, v, 0.2, True).reshape(n, -1), dt)
    first = S.masked_attention(qd[:1].contiguous(), H, G, D, V, kc, vc, seg_meta([1], [0], [0], dev, bt), -30.0)
    close(first.view(H, V), v[0].repeat_interleave(H, 0), dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_joined_maps_and_grouped_norms(backend):
    """a1 - lambda a2 per head, unit norm, a constant, the sigmoid gate; and the plain forms: a weight of all heads'
    size without a gate (a norm in groups), a shared weight with a gate."""
    dev, dt = backend
    T, H, V, eps = 5, 3, 70, 1e-4
    o2, g = rnd(T, H, 2, V, seed=1, std=3.0), rnd(T, H * V + 4, seed=2)
    want = O.unit_rms(o2[:, :, 0] - 0.83 * o2[:, :, 1], eps) * 0.65 * torch.sigmoid(g[:, 4:]).view(T, H, V)
    got = S.head_norm_gate(f32(o2.reshape(T, -1), dev), f32(g, dev)[:, 4:], None, H, V, eps, dt, sub_lambda=0.83,
                           out_scale=0.65)
    close(got, want.reshape(T, -1), dt)
    o, w = rnd(T, H * V, seed=3, std=3.0), rnd(H * V, seed=4) + 1.0
    close(S.head_norm_gate(f32(o, dev), None, f32(w, dev), H, V, eps, dt),
          (O.unit_rms(o.view(T, H, V), eps) * w.view(H, V)).reshape(T, -1), dt)
    close(S.head_norm_gate(f32(o, dev), None, f32(w, dev), 1, H * V, eps, dt), O.unit_rms(o, eps) * w, dt)
    ws = rnd(V, seed=5) + 1.0
    close(S.head_norm_gate(f32(o, dev), f32(g, dev)[:, 4:], f32(ws, dev), H, V, eps, dt),
          (O.unit_rms(o.view(T, H, V), eps) * ws * torch.sigmoid(g[:, 4:]).view(T, H, V)).reshape(T, -1), dt)


def ssd_reference(x, bc, dtp, dt_bias, rate, Dk, z, H, P, G, Ns, S0=None):
    T = x.shape[0]
    dt = F.softplus(dtp + dt_bias)
    St = torch.zeros(H, Ns, P, dtype=DT) if S0 is None else S0.clone()
    y = torch.zeros(T, H, P, dtype=DT)
    xh, B, C = x.view(T, H, P), bc[:, :G * Ns].view(T, G, Ns), bc[:, G * Ns:].view(T, G, Ns)
    for i in range(T):
        for h in range(H):
            g = h // (H // G)
            St[h] = torch.exp(-rate[h] * dt[i, h]) * St[h] + dt[i, h] * torch.outer(B[i, g], xh[i, h])
            y[i, h] = St[h].T @ C[i, g] + Dk[h] * xh[i, h]
    return y.reshape(T, -1) * O.silu(z), St


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,P,G,Ns", [(6, 4, 3, 8), (2, 8, 1, 5), (3, 1, 3, 16), (1, 70, 1, 33), (4, 64, 2, 128),
                                      (2, 3, 2, 1)])
@pytest.mark.parametrize("T", [41, 333])
def test_state_space_scan_across_portions_and_slots(backend, H, P, G, Ns, T):
    """T = 333: portions of more than 128 rows run in chunks of 64 in parallel (on the device).  The inputs are
    column slices of wider matrices, as the layer hands them over."""
    dev, dt = backend
    C = H * P
    ld = 4 if Ns % 4 == 0 and C % 4 == 0 else 1       # 4: B and C rows are 16-byte aligned (the four-wide loads)
    wide = rnd(T, ld + C + 2 * G * Ns + (4 if ld == 4 else 2), seed=P).to(torch.bfloat16).double()
    zd = rnd(T, C + H + 2, seed=2).to(torch.bfloat16).double()
    x, bc, z, dtp = wide[:, ld:ld + C], wide[:, ld + C:ld + C + 2 * G * Ns], zd[:, :C], zd[:, C + 1:C + 1 + H]
    dt_bias, rate, Dk = rnd(H, seed=3) - 0.5, torch.exp(rnd(H, seed=4, std=0.5)), rnd(H, seed=5) + 1.0
    want, Sw = ssd_reference(x, bc, dtp, dt_bias, rate, Dk, z, H, P, G, Ns)
    wd, zf = wide.to(dev).to(dt), zd.to(dev).to(dt)
    dtf = f32(zd, dev)                                                   # step sizes come in fp32
    for cuts in [(T,), (1, 1, 2, 17, 3), (16, 16, 1)] if T < 100 else [(T,), (200, 133), (130, 1, 1, 201)]:
        state = torch.full((3, C, Ns), float("nan"), device=dev)

        def run(s, e):
            return S.ssd_scan(wd[s:e, ld:ld + C], wd[s:e, ld + C:ld + C + 2 * G * Ns], dtf[s:e, C + 1:C + 1 + H],
                              f32(dt_bias, dev), f32(rate, dev), f32(Dk, dev), zf[s:e, :C], H, P, G, Ns, state,
                              seg_meta([e - s], [s], [1], dev), fast_exp=dt == torch.bfloat16)
        got = in_portions(run, T, cuts)
        assert got.dtype == torch.float32
        close(got, want, torch.float32, scale=3.0 if dt == torch.float32 else 30.0)
        close(state[1].view(H, P, Ns).transpose(1, 2), Sw, torch.float32, scale=3.0 if dt == torch.float32 else 30.0)


@pytest.mark.parametrize("backend", BACKENDS)
def test_sequences_in_one_step_keep_their_own_state(backend):
    """A portion long enough for the chunk-parallel kernels beside a short one and a single token, slots that are
    not in segment order: every sequence's result and state are what it gets alone; the convolution too."""
    dev, dt = backend
    H, P, G, Ns, taps = 4, 8, 2, 6, 4
    C, ch = H * P, H * P + 2 * 2 * 6
    lens, pos0, slots = [200, 3, 1], [0, 5, 9], [2, 0, 1]
    T = sum(lens)
    xin = rnd(T, ch, seed=1)
    cw, cb = rnd(ch, taps, seed=2, std=0.5), rnd(ch, seed=3, std=0.2)
    zd = rnd(T, C + H, seed=4)
    dt_bias, rate, Dk = rnd(H, seed=5) - 0.5, torch.exp(rnd(H, seed=6, std=0.5)), rnd(H, seed=7) + 1.0

    def run(st, tail, a, e, sg):
        xbc = S.short_conv(f32(xin, dev)[a:e], f32(cw, dev), f32(cb, dev), tail, sg, act=True)
        return S.ssd_scan(xbc[:, :C], xbc[:, C:], f32(zd, dev)[a:e, C:], f32(dt_bias, dev), f32(rate, dev), f32(Dk, dev),
                          f32(zd, dev)[a:e, :C], H, P, G, Ns, st, sg)
    together = torch.full((3, C, Ns), 0.25, device=dev)                  # the continuing sequences start from some state
    tail = torch.full((3, taps - 1, ch), 0.5, device=dev)
    got = run(together, tail, 0, T, seg_meta(lens, pos0, slots, dev))
    at = 0
    for n, p0, sl in zip(lens, pos0, slots):
        alone, tl = torch.full((3, C, Ns), 0.25, device=dev), torch.full((3, taps - 1, ch), 0.5, device=dev)
        w = run(alone, tl, at, at + n, seg_meta([n], [p0], [sl], dev))
        close(got[at:at + n], w, torch.float32, scale=5.0)
        close(together[sl], alone[sl], torch.float32, scale=5.0)
        close(tail[sl], tl[sl], torch.float32)
        at += n


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("E,top,X,W", [(5, 2, 1, 48), (3, 3, 0, 20), (12, 1, 1, 64), (4, 2, 2, 7)])
def test_router_scale_and_gate_rows(backend, E, top, X, W):
    """Softmax over all experts, the top scores renormalised and scaled; rows behind the experts' are not routed."""
    dev, dt = backend
    T = 9
    h = rnd(T, W, seed=E).to(torch.bfloat16).double()
    wr = rnd(E + X, W, seed=2, std=0.5).to(torch.bfloat16).double()
    r = M.route_direct(h.to(dev).to(dt), wr.to(dev).to(dt), top, scoring="softmax", renorm=True, renorm_eps=1e-20,
                       scale=1.7, extra_rows=X)
    z = h @ wr.T
    s = torch.softmax(z[:, :E], -1)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    wt = torch.gather(s, 1, order)
    wt = wt / (wt.sum(-1, keepdim=True) + 1e-20) * 1.7
    assert torch.equal(r[1].cpu().long(), order)
    close(r[0], wt, torch.float32, scale=5.0)
    if X:
        close(r[2], z[:, E:], torch.float32, scale=5.0)
    else:
        assert len(r) == 2


@pytest.mark.parametrize("backend", BACKENDS)
def test_clamped_gated_unit(backend):
    dev, dt = backend
    gu = rnd(6, 2 * 37, seed=1, std=2.0).to(torch.bfloat16).double()
    g, u = gu[:, :37].clamp(max=0.9), gu[:, 37:].clamp(-0.9, 0.9)
    close(M.glu_clamp(gu.to(dev).to(dt), 1.702, 0.9, 1.0), g * torch.sigmoid(1.702 * g) * (u + 1.0), dt)


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("backend", BACKENDS)
def test_layers_match_after_every_layer(backend):
    dev, dt = backend
    d = default_config()
    W = weights(d, 1)
    tokens = toks(45, d["vocab"], 2)
    want = []
    O.forward(W, d, tokens, want)
    eng = engine(d, W, backend)
    sid = eng.new_sequence()
    got = []
    fw = eng.model.forward
    eng.model.forward = lambda *a, **k: fw(*a, layers_out=got, **k)
    eng.feed([(sid, tokens, [])])
    assert len(got) == len(want) == len(d["layers"])
    for i, (g, w) in enumerate(zip(got, want)):
        e = (g.double().cpu() - w).abs().max(-1).values / w.abs().max()       # per token
        if dt == torch.float32:
            assert float(e.max()) < 3e-5, (i, float(e.max()))
        else:
            assert float(e.median()) < 0.02 * (i + 1) and float(e.max()) < 0.6, (i, float(e.median()), float(e.max()))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cuts", [(), (70,), (30, 2, 2, 17, 3, 5), (69,), (1, 68)])
def test_prefill_decode_and_portions_agree_with_oracle(backend, cuts):
    """() = token by token from the first token on; (70,) = one prefill; portions down to two tokens."""
    d = default_config()
    W = weights(d, 3)
    tokens = toks(70, d["vocab"], 4)
    want = O.forward(W, d, tokens)
    eng = engine(d, W, backend)
    got = feed_all(eng, eng.new_sequence(), tokens, cuts)
    assert agrees(got, want, backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
def test_mixed_batches_equal_each_alone_and_reuse_pages_and_slots(backend):
    """Five requests of unequal length through three slots and a pool that cannot hold them all at once:
    portions of some beside single tokens of others; finished requests give pages and slots back."""
    d = default_config()
    W = weights(d, 5)
    lens = [50, 9, 33, 1, 64]
    reqs = [toks(n, d["vocab"], 10 + i) for i, n in enumerate(lens)]
    want = [O.forward(W, d, r) for r in reqs]
    eng = engine(d, W, backend, num_blocks=5, block_size=32, slots=3)
    got = [[] for _ in reqs]
    at = [0] * len(reqs)
    sid = {}
    plan = [[(0, 20), (1, 2)], [(0, 1), (1, 7), (2, 30)], [(0, 29), (2, 1)], [(2, 2), (3, 1)],       # 0, 1, 3 end
            [(4, 40)], [(4, 1), (2, 0)], [(4, 23)]]
    for step in plan:
        entries, who = [], []
        for i, n in step:
            if n == 0:
                continue
            if i not in sid:
                sid[i] = eng.new_sequence()
            entries.append((sid[i], reqs[i][at[i]:at[i] + n], list(range(n))))
            who.append((i, n))
            at[i] += n
        lg = eng.feed(entries)
        o = 0
        for i, n in who:
            got[i].append(lg[o:o + n])
            o += n
            if at[i] == lens[i]:
                eng.release_sequence(sid.pop(i))
    assert at == lens
    for i in range(len(reqs)):
        assert agrees(torch.cat(got[i]), want[i], backend[1]), i
    assert eng.kv.free_blocks == eng.kv.num_blocks and eng.states.free_slots == 3


@pytest.mark.parametrize("backend", BACKENDS)
def test_sharp_scores_over_page_borders(backend):
    """Large score scales: nearly all weight on one key, so a key lost at a page border, a sink left out or a
    map's key head mixed up shows in the logits.  Pages of 32."""
    d = config([(att(scale=6.0, rot=8), dense()), (dif(scale=5.0, every=3), None), (att(scale=7.0, kv_from=0), None),
                (dif(scale=6.0, kv_from=1, every=0), dense())])
    W = weights(d, 6)
    tokens = toks(100, d["vocab"], 7)
    want = O.forward(W, d, tokens)
    for cuts in [(100,), (31, 2, 31, 15, 2, 17), (64,)]:
        eng = engine(d, W, backend)
        assert agrees(feed_all(eng, eng.new_sequence(), tokens, cuts), want, backend[1], mult=2.0), cuts


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_portions_then_decoding(backend):
    """Portions long enough for the chunk-parallel scan, cut off a chunk's border, then single tokens."""
    d = default_config()
    W = weights(d, 17)
    tokens = toks(330, d["vocab"], 18)
    want = O.forward(W, d, tokens)
    for cuts in [(321,), (150, 171)]:
        eng = engine(d, W, backend)
        assert agrees(feed_all(eng, eng.new_sequence(), tokens, cuts), want, backend[1], mult=2.0), cuts


@pytest.mark.parametrize("backend", BACKENDS)
def test_first_tokens(backend):
    d = default_config()
    W = weights(d, 8)
    for n in (1, 2, 3):
        tokens = toks(n, d["vocab"], 20 + n)
        eng = engine(d, W, backend)
        assert agrees(feed_all(eng, eng.new_sequence(), tokens, (n,)), O.forward(W, d, tokens), backend[1], mult=2.5), n


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(backend):
    d = default_config()
    W = weights(d, 9)
    tokens = toks(150, d["vocab"], 10)
    want = O.forward(W, d, tokens)
    eng = engine(d, W, backend)
    got = feed_all(eng, eng.new_sequence(), tokens, (10,))           # 140 tokens one by one
    assert agrees(got, want, backend[1], mult=2.0)


OTHER = {
    "matrix_core_sizes": [(dif(heads=4, kv_heads=2, dim=64, vdim=64), dense()), (att(heads=4, kv_heads=2, dim=128, rot=64), None),
                          (dif(heads=4, kv_heads=2, dim=64, vdim=64, kv_from=0), None),
                          (dif(heads=3, kv_heads=1, dim=128, vdim=128, every=0), dense()),
                          (att(heads=4, kv_heads=2, dim=128, rot=64, kv_from=1), None), (att(heads=3, kv_heads=3, dim=64, rot=0), None)],
    "expert_kernel_sizes": [(dif(), moe(ff=128, experts=4, top=2, shared=128)), (mam(), moe(ff=64, experts=3, top=1, shared=0)),
                            (att(), dense(ff=256))],
    "one_head_everywhere": [(att(heads=1, kv_heads=1, dim=4, rot=2), dense(ff=8)), (dif(heads=1, kv_heads=1), moe(experts=1, top=1)),
                            (mam(heads=1, vdim=4, groups=1, norm_groups=1), None)],
    "top_one_and_top_all": [(mam(), moe(experts=4, top=1, scale=1.0)), (att(), moe(experts=4, top=4, scale=0.5, shared=0))],
    "no_shared_no_side_no_mlp": [(dif(), moe(shared=0)), (mam(), None), (att(), None)],
    "mamba_first_conv_one_groups_equal_heads": [(mam(heads=4, vdim=6, state=3, groups=4, conv=1, norm_groups=4), dense()),
                                                (mam(heads=4, vdim=6, state=128, groups=2, conv=2, norm_groups=3), None),
                                                (dif(every=0), None)],
    "no_rotation_and_whole_head": [(att(rot=0), dense()), (att(dim=8, rot=8), None), (att(dim=10, rot=2, heads=3, kv_heads=1), None)],
    "unaligned_sizes": [(dif(heads=3, kv_heads=3, dim=7, vdim=9), moe(ff=10, experts=7, top=3, shared=11)),
                        (mam(heads=3, vdim=5, state=7, groups=3, conv=6, norm_groups=5), dense(ff=13)),
                        (att(heads=5, kv_heads=1, dim=10, rot=6), None)],
    "shared_pages_of_both_kinds": [(att(), None), (dif(), None), (att(kv_from=0), dense()), (dif(kv_from=1), None),
                                   (dif(kv_from=1, every=2, diff=0.1), None), (att(kv_from=0), None)],
}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(backend, name):
    d = config(OTHER[name], width={"unaligned_sizes": 34, "matrix_core_sizes": 64, "expert_kernel_sizes": 128}.get(name, 40), eps=1e-3,
               side={"no_shared_no_side_no_mlp": 0, "unaligned_sizes": 5, "one_head_everywhere": 1}.get(name, 8))
    W = weights(d, 11)
    tokens = toks(40, d["vocab"], 12)
    want = O.forward(W, d, tokens)
    eng = engine(d, W, backend)
    assert agrees(feed_all(eng, eng.new_sequence(), tokens, (13, 2, 9)), want, backend[1], mult=2.0)


@pytest.mark.parametrize("backend", BACKENDS)
def test_greedy_generation_through_submit_and_scheduler(backend):
    """``submit`` + ``step``: the scheduler's own batching (two prompts of unequal length, then decode rows)
    must produce the oracle's greedy continuation."""
    d = default_config(vocab=8192)
    W = weights(d, 13)
    eng = engine(d, W, backend, num_blocks=16)
    prompts = [toks(37, 2000, 14), toks(6, 2000, 15)]
    outs = {}
    for i, p in enumerate(prompts):
        eng.submit(eng.new_sequence(), p, None, 6, temperature=0.0, on_done=lambda g, st, i=i: outs.__setitem__(i, g))
    eng.run_until_idle()
    for i, p in enumerate(prompts):
        seq, same = list(p), 0
        for t in outs[i][:6]:
            lg = O.forward(W, d, seq)[-1, :eng.vocab]
            if backend[1] == torch.float32:
                assert t == int(lg.argmax()), i
            else:       # bf16: the chosen token is among the best few of thousands, and mostly the best
                assert int((lg > lg[t]).sum()) < 40, i
                same += t == int(lg.argmax())
            seq.append(t)
        assert len(outs[i]) >= 6 and (backend[1] == torch.float32 or same >= 3)


def test_config_round_trip_registry_and_replay(tmp_path):
    """config.json -> configuration -> config.json; the registry picks the class by the file; a recorded
    schedule replayed through the engine gives the oracle's logits."""
    from k8s_llm_rca_amd.engine import trace as TR
    from k8s_llm_rca_amd.models import pumozen as PZ
    from k8s_llm_rca_amd.models.registry import checkpoint_arch, get_any_config, load_model
    d = default_config()
    cfg = PumozenConfig.from_json(d, "x")
    assert PumozenConfig.from_json(cfg.to_json(), "x") == cfg
    assert get_any_config("tiny-pumozen").arch == "pumozen"
    tiny = PumozenModel(get_any_config("tiny-pumozen"), "cpu", torch.float32)
    assert tiny.weight_bytes() > 0 and len(tiny.state_spec()) == 2
    W = weights(d, 21)
    path = str(tmp_path / "ckpt")
    PZ.save_checkpoint(cfg, W, path)
    assert checkpoint_arch(path) == "pumozen"
    assert isinstance(load_model(path, "cpu", torch.float32), PumozenModel)
    eng = TR.make_engine(path, torch.float32, 128, device="cpu", state_slots=2, block_size=32)
    a, b = toks(40, d["vocab"], 22), toks(21, d["vocab"], 23)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[30:31], "want": [0]}, {"id": "b", "tokens": b[:20], "want": []}],
              "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}, {"id": "a", "tokens": a[31:], "want": [8]}],
              "end": ["a", "b"]}]
    out = str(tmp_path / "out")
    log = io.StringIO()
    TR.replay(eng, io.StringIO("\n".join(json.dumps(s) for s in steps)), out, log)
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    wa, wb = O.forward(W, d, a), O.forward(W, d, b)
    g0 = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, -1))
    g2 = torch.from_numpy(np.fromfile(os.path.join(out, "2.f32"), dtype="<f4").reshape(2, -1))
    assert agrees(g0, wa[[0, 29]], torch.float32) and agrees(g2, torch.stack([wb[20], wa[39]]), torch.float32)
    assert eng.kv.free_blocks == eng.kv.num_blocks and eng.states.free_slots == 2


def test_bad_configurations_are_refused():
    for layers in ([(att(kv_from=0), None)], [(att(), None), (dif(kv_from=0), None)],
                   [(dif(), None), (dif(heads=2, kv_heads=2, kv_from=0), None)], [(mam(heads=4, groups=3), None)],
                   [(dif(), moe(experts=2, top=3))]):
        with pytest.raises(ValueError):
            PumozenModel(PumozenConfig.from_json(config(layers), "bad"), "cpu", torch.float32, init=False)


def test_trace_run_command_line(tmp_path):
    from k8s_llm_rca_amd.models import pumozen as PZ
    d = default_config()
    W = weights(d, 31)
    path = str(tmp_path / "ckpt")
    PZ.save_checkpoint(PumozenConfig.from_json(d, "x"), W, path)
    tokens = toks(12, d["vocab"], 32)
    step = json.dumps({"step": 0, "entries": [{"id": "r", "tokens": tokens, "want": [11]}], "end": ["r"]})
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64", "--device", "cpu"], input=step + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "done 0" in r.stdout, r.stderr[-2000:]
    got = torch.from_numpy(np.fromfile(str(tmp_path / "o" / "0.f32"), dtype="<f4").reshape(1, -1))
    assert agrees(got, O.forward(W, d, tokens)[-1:], torch.float32)
