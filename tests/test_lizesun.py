"""Lizesun through the engine against the plain implementation in ``lizesun_oracle.py``:
each mechanism alone, prefill against token-by-token decoding, portions, mixed batches,
reuse of pages and state slots, chunk / window edges and page borders, kept first tokens,
the first tokens of a sequence, long decoding, other sizes, and greedy generation through
``submit`` / ``step``.

Every case runs on the CPU (the ops' fp32 forms, the same engine, cache manager and
scheduler) and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import json
import math
import os
import subprocess
import sys

import pytest
import torch
import torch.nn.functional as F

import lizesun_oracle as O
from k8s_llm_rca_amd.engine.engine import EngineConfig, LLMEngine
from k8s_llm_rca_amd.models.lizesun import LizesunConfig, LizesunModel
from k8s_llm_rca_amd.ops import norm as N
from k8s_llm_rca_amd.ops import seq_ops as S

GPU = pytest.mark.gpu
BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=GPU),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=GPU)]
DT = torch.float64


def row_errs(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def agrees(got, want, dtype, mult=1.0):
    """Logits rows against the oracle's.  fp32 (the sharp check): every row.  bf16: these models are a few
    dozen channels wide, so one rounding moves a row visibly; most rows must be close, none far off."""
    e = row_errs(got, want)
    if dtype == torch.float32:
        return float(e.max()) < 5e-5 * mult
    return (float(e.median()) < 3e-2 * mult and float(e.max()) < 0.35
            and int((e > 8e-2 * mult).sum()) <= max(1, 0.1 * e.numel()))


def close(got, want, dtype, scale=1.0):
    """Element-wise check of an op's output against fp64."""
    got, want = got.double().cpu(), want.double().cpu()
    t = (2e-5 if dtype == torch.float32 else 2e-2) * scale
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err < t, err


# ------------------------------------------------------------------ configurations and weights
def att(heads=4, kv_heads=2, dim=8, vdim=12, chunk=16, scale=None, softcap=9.0, v_mix=True):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "v_mix": v_mix,
         "scale": 1.0 / math.sqrt(dim) if scale is None else scale}
    if chunk:
        m["mask"] = {"size": chunk}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m}


def par(heads=6, kv_heads=3, dim=8, vdim=4, window=11, keep=3, rot=4, base=300.0, scale=0.7, mh=3, md=8, mv=12,
        cap=6.0, ls=0.6, rs=1.3):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        left["mask"] = {"size": window, "keep_first": keep}
    if rot:
        left["rot"] = {"dims": rot, "base": base}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": mh, "dim": md, "vdim": mv, "gate_cap": cap},
                                          "left_scale": ls, "right_scale": rs}}


def dlt(heads=4, kv_heads=2, dim=8, vdim=12, conv=3, ra=5, rg=7):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                               "conv": conv, "a_rank": ra, "g_rank": rg}}


def config(layers, width=48, vocab=512, eps=1e-5, embed_scale=3.0):
    ls = [dict(mix, mlp={"kind": "dense", "ff": ff} if ff else None) for mix, ff in layers]
    return {"architecture": "Lizesun", "vocab": vocab, "width": width, "embedding": {"scale": embed_scale},
            "layers": ls, "norm": {"eps": eps}}


def default_config(**kw):
    return config([(par(), 40), (att(), 24), (dlt(), 0), (att(heads=2, kv_heads=2, dim=12, vdim=12, chunk=7), 56),
                   (par(heads=2, kv_heads=2, dim=4, vdim=6, window=5, keep=0, rot=4, mh=1, md=4, mv=4), 0),
                   (dlt(heads=2, kv_heads=2, dim=6, vdim=4, conv=2), 16)], **kw)


def weights(d, seed=0):
    """Random weights under the checkpoint's names, rounded to bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W = d["width"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def lin(o, i, mul=1.0):
        return r(o, i, std=mul * i ** -0.5)

    t = {"embed": r(d["vocab"], W, std=1.0 / d["embedding"]["scale"]), "head": lin(d["vocab"], W)}

    def norm(name):
        t[name], t[name + ".b"], t[name + ".alpha"] = r(W, std=0.2, mean=1.0), r(W, std=0.1), r((), std=0.1, mean=0.8)

    norm("final.norm")
    for i, L in enumerate(d["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        norm(f"l{i}.norm1")
        if L["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[p + "q"], t[p + "k"], t[p + "v"] = lin(H * D, W), lin(G * D, W), lin(G * V, W)
            t[p + "q.b"], t[p + "k.b"], t[p + "v.b"] = r(H * D, std=0.3), r(G * D, std=0.3), r(G * V, std=0.3)
            t[p + "q.norm"], t[p + "k.norm"] = r(D, std=0.3, mean=1.5), r(D, std=0.3, mean=1.5)
            t[p + "vmix"] = r((), std=0.1, mean=0.4)
            t[p + "g"], t[p + "o"] = lin(H, W, 2.0), lin(W, H * V)
        elif L["type"] == "parallel":
            a, b = m["left"], m["right"]
            q, s = p + "left.", p + "right."
            H, G, D, V = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            t[q + "q"], t[q + "k"], t[q + "v"] = lin(H * D, W), lin(G * D, W), lin(G * V, W)
            t[q + "sink"], t[q + "o"] = r(H, std=1.0), lin(W, H * V)
            H, D, V = b["heads"], b["dim"], b["vdim"]
            t[s + "q"], t[s + "k"], t[s + "v"] = lin(H * D, W), lin(H * D, W), lin(H * V, W)
            t[s + "g"], t[s + "o"], t[s + "norm"] = lin(H * V, W), lin(W, H * V), r(H * V, std=0.2, mean=1.0)
            t[s + "i"], t[s + "f"] = lin(H, W, 3.0), lin(H, W, 3.0)
            t[s + "i.b"], t[s + "f.b"] = r(H, std=0.5), r(H, std=0.5, mean=1.5)
        else:
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t[p + "q"], t[p + "k"], t[p + "v"] = lin(G * D, W), lin(G * D, W), lin(H * V, W)
            for n_, ch in (("q", G * D), ("k", G * D), ("v", H * V)):
                t[p + n_ + ".conv"] = r(ch, m["conv"], std=0.6)
            t[p + "b"], t[p + "A_log"], t[p + "norm"] = lin(H, W, 2.0), r(H, std=0.5, mean=-0.5), r(V, std=0.2, mean=1.0)
            t[p + "a1"], t[p + "a2"] = lin(m["a_rank"], W), lin(H * D, m["a_rank"], 2.0)
            t[p + "dt_bias"] = r(H * D, std=0.5, mean=-0.5)
            t[p + "g1"], t[p + "g2"], t[p + "o"] = lin(m["g_rank"], W), lin(H * V, m["g_rank"], 2.0), lin(W, H * V)
        if L["mlp"] is not None:
            norm(f"l{i}.norm2")
            t[f"l{i}.mlp.up"], t[f"l{i}.mlp.down"] = lin(L["mlp"]["ff"], W), lin(W, L["mlp"]["ff"], 0.5)
    return t


def engine(d, W, backend, num_blocks=24, block_size=32, slots=4, **kw):
    dev, dt = backend
    model = LizesunModel(LizesunConfig.from_json(d, "test"), dev, dt, init=False)
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


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("W", [6, 48, 300, 1024])
def test_dynamic_tanh_residual_pass_and_squared_relu(backend, W):
    dev, dt = backend
    T = 7
    x, y, y2 = rnd(T, W, seed=1, std=2.0), rnd(T, W, seed=2, std=5.0), rnd(T, W, seed=3)
    w, b = rnd(W, seed=4) + 1.0, rnd(W, seed=5, std=0.3)
    t = {"n": w, "n.b": b, "n.alpha": torch.tensor(0.37, dtype=DT)}
    f = lambda *ts: [v.float().to(dev) for v in ts]  # noqa: E731
    X, Y, Y2, Wt, B = f(x, y, y2, w, b)
    xin = X.clone()
    h = N.add_dyt(xin, Y, 1.0, None, 1.0, 0.37, Wt, B, out_dtype=dt)
    close(xin, x + y, torch.float32)
    close(h, O.dyt(x + y, t, "n"), dt)
    xin = X.clone()
    h = N.add_dyt(xin, Y, 0.6, Y2, -1.7, 0.37, Wt, B, out_dtype=dt)
    close(xin, x + 0.6 * y - 1.7 * y2, torch.float32)
    close(h, O.dyt(x + 0.6 * y - 1.7 * y2, t, "n"), dt)
    xin = X.clone()
    assert N.add_dyt(xin, Y, 1.0, Y2, 1.0) is None                      # the add alone
    close(xin, x + y + y2, torch.float32)
    xin = X.clone()
    close(N.add_dyt(xin, None, 1.0, None, 1.0, 0.37, Wt, B, out_dtype=dt), O.dyt(x, t, "n"), dt)   # the norm alone
    assert torch.equal(xin, X)
    emb = rnd(20, W, seed=13).to(torch.bfloat16)
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32, device=dev)
    x0 = torch.empty(4, W, device=dev)
    h = N.embed_scale_dyt(ids, emb.to(dev).to(dt), 5.5, x0, 0.37, Wt, B, out_dtype=dt)
    want = emb.double()[ids.cpu().long()] * 5.5
    close(x0, want, torch.float32)
    close(h, O.dyt(want, t, "n"), dt)
    u = rnd(5, W + 3, seed=6, std=3.0).to(torch.bfloat16).double()
    close(N.relu_sq(u.to(dev).to(dt)), torch.relu(u) ** 2, dt)


STALE = 2.0 ** 15     # what unwritten page entries hold in these tests (exact in bfloat16)


def paged(dev, dt, n_pages, BS, G, D, V, order):
    """Empty key / value pages and a block table that walks them in ``order``."""
    kc = torch.full((n_pages, BS, G * D), STALE, device=dev, dtype=dt)
    vc = torch.full((n_pages, BS, G * V), STALE, device=dev, dtype=dt)
    return kc, vc, [list(order)]


def slots_of(order, BS, a, e, dev):
    p = torch.arange(a, e)
    return (torch.tensor(order)[p // BS] * BS + p % BS).to(torch.int32).to(dev)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V,rot,norm,wts", [(4, 2, 8, 12, 4, True, False), (3, 3, 6, 5, 6, True, True),
                                                  (2, 1, 16, 8, 0, True, True), (5, 1, 70, 3, 32, False, False),
                                                  (1, 1, 4, 130, 2, True, False), (40, 8, 400, 3, 64, True, True)])
def test_attention_preparation(backend, H, G, D, V, rot, norm, wts):
    """Bias, rotation far from position 0, unit norm with and without a weight, value mixing, paged write."""
    dev, dt = backend
    T, BS, eps, base, lam = 9, 8, 1e-3, 777.0, 0.3
    pos = torch.tensor([0, 1, 2, 3, 4, 5, 70001, 70002, 70003])
    x = rnd(T, H * D + G * D + G * V + 3, seed=H + D, std=2.0)              # a column slice of something wider
    bias = rnd(H * D + G * D + G * V, seed=3)
    qw, kw = (rnd(D, seed=4) + 1.5, rnd(D, seed=5) + 1.5) if wts else (None, None)
    vo = rnd(T, G * V, seed=6)
    xb = x[:, :-3] + bias
    q = O.rotate_half(xb[:, :H * D].view(T, H, D), pos, rot, base)
    k = O.rotate_half(xb[:, H * D:H * D + G * D].view(T, G, D), pos, rot, base)
    if norm:
        q, k = O.unit_rms(q, eps), O.unit_rms(k, eps)
        if wts:
            q, k = q * qw, k * kw
    v = xb[:, H * D + G * D:]
    order = [2, 0, 1]
    kc, vc, _ = paged(dev, dt, 3, BS, G, D, V, order)
    vt = torch.full((3, G * V, BS), STALE, device=dev, dtype=dt)
    sl = torch.tensor([order[i // BS] * BS + i % BS for i in range(T)], dtype=torch.int32, device=dev)
    f32 = lambda z: None if z is None else z.float().to(dev)  # noqa: E731
    keep = torch.empty(T, G * V, device=dev)
    got = S.attn_prep(f32(x)[:, :-3], f32(bias), H, G, D, V, pos.to(torch.int32).to(dev), sl, kc, vc, dt, norm=norm,
                      q_w=f32(qw), k_w=f32(kw), eps=eps, rot_dims=rot, rot_base=base, lam=lam, v_other=f32(vo),
                      v_keep=keep, vt=vt)
    close(got, q.reshape(T, -1), dt)
    close(keep, v, torch.float32)
    close(kc.view(-1, G * D)[sl.long()], k.reshape(T, -1), dt)
    vm = (1 - lam) * v + lam * vo
    close(vc.view(-1, G * V)[sl.long()], vm, dt)
    close(vt[sl.long() // BS, :, sl.long() % BS], vm, dt)
    assert float(kc[1].float().min()) == STALE and float(vc[0, 1:].float().min()) == STALE   # nothing else was written


def attention_case(dev, dt, H, G, D, V, n, BS, seed, sharp=None, with_twin=False):
    """Random q / k / v for one sequence, the keys and values in shuffled pages.  ``sharp`` = (i, j): key j is
    made to stand out for query i."""
    q, k, v = rnd(n, H, D, seed=seed), rnd(n, G, D, seed=seed + 1), rnd(n, G, V, seed=seed + 2)
    if sharp is not None:
        i, j = sharp
        q[i] = q[i, 0]                                        # every head asks the same
        k[j] = 8.0 * q[i, 0] / q[i, 0].norm()
    q, k, v = (z.to(torch.bfloat16).double() for z in (q, k, v))
    n_pages = -(-n // BS)
    order = torch.randperm(n_pages + 2, generator=torch.Generator().manual_seed(seed)).tolist()[:n_pages]
    kc, vc, bt = paged(dev, dt, n_pages + 2, BS, G, D, V, order)
    sl = slots_of(order, BS, 0, n, dev).long()
    kc.view(-1, G * D)[sl] = k.reshape(n, -1).to(dev).to(dt)
    vc.view(-1, G * V)[sl] = v.reshape(n, -1).to(dev).to(dt)
    if with_twin:                 # the values' transposed twin: the matrix-core kernel runs where it takes the sizes
        vt = torch.full((n_pages + 2, G * V, BS), STALE, device=dev, dtype=dt)
        vt[sl // BS, :, sl % BS] = v.reshape(n, -1).to(dev).to(dt)
        return q, k, v, kc, vc, bt, vt
    return q, k, v, kc, vc, bt


MASKS = [dict(chunk=16), dict(chunk=7, softcap=2.5), dict(window=11, keep_first=3), dict(window=1, keep_first=0),
         dict(window=5, keep_first=40), dict(), dict(window=64, keep_first=2, chunk=24), dict(chunk=1)]


def visible(chunk=0, window=0, keep_first=0, **_):
    return lambda i, j: (not chunk or i // chunk == j // chunk) and (not window or i - j < window or j < keep_first)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V", [(4, 2, 8, 12), (3, 3, 5, 3), (6, 1, 32, 16), (1, 1, 64, 70), (24, 4, 16, 200)])
@pytest.mark.parametrize("mask", range(len(MASKS)))
def test_masked_attention_paged(backend, H, G, D, V, mask):
    dev, dt = backend
    mk = MASKS[mask]
    n, BS, scale = 75, 16, 0.45
    q, k, v, kc, vc, bt = attention_case(dev, dt, H, G, D, V, n, BS, seed=mask + H)
    sink = rnd(H, seed=9) if mask % 2 else None
    gate = rnd(n, H + 2, seed=10) if mask % 3 else None
    want = O.masked_softmax_attention(q, k, v, scale, visible(**mk), softcap=mk.get("softcap", 0.0), sink=sink)
    if gate is not None:
        want = want * torch.sigmoid(gate[:, 1:H + 1])[:, :, None]
    kw = dict(softcap=mk.get("softcap", 0.0), chunk=mk.get("chunk", 0), window=mk.get("window", 0),
              keep_first=mk.get("keep_first", 0), sink=None if sink is None else sink.float().to(dev))
    gd = None if gate is None else gate.float().to(dev)
    qd = q.reshape(n, -1).to(dev).to(dt)
    for cuts in [(n,), (40, 1, 1, 2, 30), (3, 70)]:
        def run(a, e):
            sg = seg_meta([e - a], [a], [0], dev, bt)
            return S.masked_attention(qd[a:e].contiguous(), H, G, D, V, kc, vc, sg, scale,
                                      gate=None if gd is None else gd[a:e, 1:], **kw)
        close(in_portions(run, n, cuts), want.reshape(n, -1), dt)


# query 100 and the key that stands out, just inside / outside every edge
EDGES = {"chunk_in": (dict(chunk=26), 78), "chunk_out": (dict(chunk=26), 77),
         "window_in": (dict(window=30, keep_first=4), 71), "window_out": (dict(window=30, keep_first=4), 70),
         "first_in": (dict(window=30, keep_first=4), 3), "first_out": (dict(window=30, keep_first=4), 4),
         "far": (dict(), 1)}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("aim", ["chunk_in", "chunk_out", "window_in", "window_out", "first_in", "first_out", "far"])
def test_one_key_stands_out_at_every_edge(backend, aim):
    """One key draws nearly all of query i's weight: the output shows at once whether the mask let it in.
    Query 100 as part of a portion and decoded alone; the page border lies at 96."""
    dev, dt = backend
    H, G, D, V, n, BS, i = 4, 2, 16, 8, 101, 32, 100
    mk, j = EDGES[aim]
    q, k, v, kc, vc, bt = attention_case(dev, dt, H, G, D, V, n, BS, seed=3, sharp=(i, j))
    want = O.masked_softmax_attention(q, k, v, 1.0, visible(**mk))
    share = (want[i] - v[j].repeat_interleave(H // G, 0)).abs().max()
    assert (share < 0.2) == aim.endswith("in") or aim == "far" and share < 0.2     # the case is what its name says
    qd = q.reshape(n, -1).to(dev).to(dt)
    kw = dict(chunk=mk.get("chunk", 0), window=mk.get("window", 0), keep_first=mk.get("keep_first", 0))
    for a in (0, 90, i):                                               # whole prompt, a portion, decoded alone
        got = S.masked_attention(qd[a:].contiguous(), H, G, D, V, kc, vc, seg_meta([n - a], [a], [0], dev, bt), 1.0, **kw)
        close(got[-1], want[i].reshape(-1), dt)


MFMA_BACKEND = [pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=GPU)]


@pytest.mark.parametrize("backend", MFMA_BACKEND)
@pytest.mark.parametrize("H,G,D,V", [(4, 2, 64, 64), (3, 1, 128, 64), (18, 2, 64, 128), (2, 2, 128, 128), (1, 1, 64, 64)])
@pytest.mark.parametrize("mask", range(len(MASKS)))
@pytest.mark.parametrize("split", [True, False])
def test_masked_attention_on_the_matrix_cores(backend, H, G, D, V, mask, split, monkeypatch):
    """The sizes the matrix-core kernel takes: tiles of 16 tokens, portions that start inside a tile's
    span, a chunk border inside a tile, decoding token by token; with and without the split of a tile's key
    blocks over workgroups that steps of few rows get."""
    dev, dt = backend
    if not split:
        monkeypatch.setattr(S, "WINDOW_SPLIT_ITEMS", 0)
    mk = MASKS[mask]
    n, BS, scale = 150, 32, 0.25
    q, k, v, kc, vc, bt, vt = attention_case(dev, dt, H, G, D, V, n, BS, seed=mask + H, with_twin=True)
    assert S.masked_mfma_ok(H, G, D, V, dt, dev)
    sink = rnd(H, seed=9) if mask % 2 else None
    gate = rnd(n, H + 2, seed=10) if mask % 3 else None
    want = O.masked_softmax_attention(q, k, v, scale, visible(**mk), softcap=mk.get("softcap", 0.0), sink=sink)
    if gate is not None:
        want = want * torch.sigmoid(gate[:, 1:H + 1])[:, :, None]
    kw = dict(softcap=mk.get("softcap", 0.0), chunk=mk.get("chunk", 0), window=mk.get("window", 0),
              keep_first=mk.get("keep_first", 0), sink=None if sink is None else sink.float().to(dev))
    gd = None if gate is None else gate.float().to(dev)
    qd = q.reshape(n, -1).to(dev).to(dt)
    for cuts in [(n,), (40, 1, 1, 2, 30, 17), (3, 70), (139,) + (1,) * 11]:
        def run(a, e):
            sg = seg_meta([e - a], [a], [0], dev, bt)
            return S.masked_attention(qd[a:e].contiguous(), H, G, D, V, kc, vc, sg, scale,
                                      gate=None if gd is None else gd[a:e, 1:], vt=vt, **kw)
        close(in_portions(run, n, cuts), want.reshape(n, -1), dt)
    # two sequences in one step share nothing: the second one's rows read its own pages
    sg = seg_meta([5, n - 100], [n - 5, 100], [0, 1], dev, bt + bt)
    got = S.masked_attention(torch.cat([qd[n - 5:], qd[100:]]).contiguous(), H, G, D, V, kc, vc, sg, scale,
                             gate=None if gd is None else torch.cat([gd[n - 5:], gd[100:]])[:, 1:], vt=vt, **kw)
    close(got, torch.cat([want[n - 5:], want[100:]]).reshape(n - 95, -1), dt)


@pytest.mark.parametrize("backend", MFMA_BACKEND)
@pytest.mark.parametrize("mk", [dict(), dict(window=2100, keep_first=70), dict(chunk=2112, softcap=3.0)])
def test_masked_attention_many_blocks(backend, mk):
    """More than 64 key blocks per tile (the block table is refilled), as a whole prompt and for the last
    tokens alone (many parts).  The expected values are a dense softmax in float64."""
    dev, dt = backend
    H, G, D, V, n, BS, scale = 2, 1, 64, 64, 2200, 64, 0.2
    q, k, v, kc, vc, bt, vt = attention_case(dev, dt, H, G, D, V, n, BS, seed=7, with_twin=True)
    sc = torch.einsum("ihd,jd->hij", q, k[:, 0]) * scale
    if mk.get("softcap"):
        sc = mk["softcap"] * torch.tanh(sc / mk["softcap"])
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    vis = j <= i
    if mk.get("chunk"):
        vis &= (i // mk["chunk"]) == (j // mk["chunk"])
    if mk.get("window"):
        vis &= ((i - j) < mk["window"]) | (j < mk["keep_first"])
    want = torch.einsum("hij,jv->ihv", torch.softmax(sc.masked_fill(~vis, float("-inf")), -1), v[:, 0]).reshape(n, -1)
    qd = q.reshape(n, -1).to(dev).to(dt)
    kw = dict(softcap=mk.get("softcap", 0.0), chunk=mk.get("chunk", 0), window=mk.get("window", 0),
              keep_first=mk.get("keep_first", 0))
    got = S.masked_attention(qd, H, G, D, V, kc, vc, seg_meta([n], [0], [0], dev, bt), scale, vt=vt, **kw)
    close(got, want, dt)
    for a in (n - 1, n - 3, n - 40):
        got = S.masked_attention(qd[a:].contiguous(), H, G, D, V, kc, vc, seg_meta([n - a], [a], [0], dev, bt), scale,
                                 vt=vt, **kw)
        close(got, want[a:], dt)


@pytest.mark.parametrize("backend", MFMA_BACKEND)
@pytest.mark.parametrize("aim", ["chunk_in", "chunk_out", "window_in", "window_out", "first_in", "first_out", "far"])
def test_one_key_stands_out_on_the_matrix_cores(backend, aim):
    dev, dt = backend
    H, G, D, V, n, BS, i = 4, 2, 64, 64, 101, 32, 100
    mk, j = EDGES[aim]
    q, k, v, kc, vc, bt, vt = attention_case(dev, dt, H, G, D, V, n, BS, seed=3, sharp=(i, j), with_twin=True)
    want = O.masked_softmax_attention(q, k, v, 1.0, visible(**mk))
    qd = q.reshape(n, -1).to(dev).to(dt)
    kw = dict(chunk=mk.get("chunk", 0), window=mk.get("window", 0), keep_first=mk.get("keep_first", 0))
    for a in (0, 90, i):
        got = S.masked_attention(qd[a:].contiguous(), H, G, D, V, kc, vc, seg_meta([n - a], [a], [0], dev, bt), 1.0,
                                 vt=vt, **kw)
        close(got[-1], want[i].reshape(-1), dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_sink_takes_its_share(backend):
    dev, dt = backend
    H, G, D, V, n = 2, 1, 8, 4, 5
    q, k, v, kc, vc, bt = attention_case(dev, dt, H, G, D, V, n, 8, seed=5)
    sink = torch.tensor([30.0, -30.0], dtype=DT)                       # head 0: nearly all weight; head 1: none
    got = S.masked_attention(q.reshape(n, -1).to(dev).to(dt), H, G, D, V, kc, vc, seg_meta([n], [0], [0], dev, bt), 0.3,
                             sink=sink.float().to(dev)).view(n, H, V).double().cpu()
    assert float(got[:, 0].abs().max()) < 1e-6
    close(got[:, 1], O.masked_softmax_attention(q, k, v, 0.3, lambda i, j: True)[:, 1], dt)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V", [(4, 2, 8, 12), (2, 2, 6, 4), (3, 1, 33, 70), (1, 1, 128, 64), (2, 1, 200, 5)])
@pytest.mark.parametrize("T", [41, 333])
def test_gated_delta_across_portions_and_slots(backend, H, G, D, V, T):
    """T = 333: portions of more than 128 rows run in chunks of 64 in parallel (on the device)."""
    dev, dt = backend
    x = rnd(T, 2 * G * D + H * V, seed=D).to(torch.bfloat16).double()
    a, beta = rnd(T, H * D, seed=2), rnd(T, H + 3, seed=3, std=2.0)
    rate, bias = torch.exp(rnd(H, seed=4, std=0.5)), rnd(H * D, seed=5) - 0.5
    q = x[:, :G * D].view(T, G, D)
    k = x[:, G * D:2 * G * D].view(T, G, D)
    v = x[:, 2 * G * D:].view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    g = torch.exp(-rate[None, :, None] * F.softplus(a + bias).view(T, H, D))
    bt = torch.sigmoid(beta[:, 2:2 + H])
    Sm = torch.zeros(H, D, V, dtype=DT)
    want = torch.zeros(T, H, V, dtype=DT)
    for i in range(T):
        for h in range(H):
            kk, qq = k[i, h // (H // G)], q[i, h // (H // G)]
            Sh = g[i, h][:, None] * Sm[h]
            Sh = Sh + kk[:, None] * (bt[i, h] * (v[i, h] - Sh.T @ kk))[None, :]
            Sm[h] = Sh
            want[i, h] = Sh.T @ qq
    f32 = lambda z: z.float().to(dev)  # noqa: E731
    xd, bd = x.to(dev).to(dt), f32(beta)
    for cuts in [(T,), (1, 1, 2, 17, 3), (16, 16, 1)] if T < 100 else [(T,), (200, 133), (130, 1, 1, 201)]:
        state = torch.full((3, H, D, V), float("nan"), device=dev)

        def run(s, e):
            return S.gated_delta(xd[s:e].contiguous(), H, G, D, V, f32(a[s:e]), f32(rate), f32(bias), bd[s:e, 2:], state,
                                 seg_meta([e - s], [s], [1], dev))
        close(in_portions(run, T, cuts), want.reshape(T, -1), dt, scale=2.0)
        close(state[1], Sm, torch.float32, scale=2.0 if dt == torch.float32 else 1e3)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,D,V", [(3, 8, 12), (1, 4, 4), (2, 33, 70), (2, 128, 64), (1, 200, 130)])
@pytest.mark.parametrize("T", [41, 333])
def test_matrix_memory_across_portions_and_slots(backend, H, D, V, T):
    """T = 333: portions of more than 128 rows run in chunks of 64 in parallel (on the device)."""
    dev, dt = backend
    cap = 5.0
    x = rnd(T, 2 * H * D + 2 * H * V + 2 * H, seed=D)
    x[:, -2 * H:] *= 4.0                                                # gates that reach the cap
    gb = rnd(2 * H, seed=2)
    HD, HV = H * D, H * V
    t = {"q": torch.eye(x.shape[1], dtype=DT)[:HD], "k": torch.eye(x.shape[1], dtype=DT)[HD:2 * HD],
         "v": torch.eye(x.shape[1], dtype=DT)[2 * HD:2 * HD + HV], "g": torch.zeros(HV, x.shape[1], dtype=DT),
         "i": torch.eye(x.shape[1], dtype=DT)[2 * HD + 2 * HV:2 * HD + 2 * HV + H],
         "f": torch.eye(x.shape[1], dtype=DT)[2 * HD + 2 * HV + H:], "i.b": gb[:H], "f.b": gb[H:],
         "norm": torch.ones(HV, dtype=DT), "o": torch.eye(HV, dtype=DT)}
    # the oracle's mixer with identity projections: its output is unit_rms(o) / 2 per head
    want = O.matrix_memory(x, t, "", {"heads": H, "dim": D, "vdim": V, "gate_cap": cap}, 1e-5)
    f32 = lambda z: z.float().to(dev)  # noqa: E731
    xd, ones, zero = f32(x), torch.ones(HV, device=dev), torch.zeros(T, HV, device=dev)
    for k, cuts in enumerate([(T,), (1, 1, 2, 17, 3), (16, 16, 1)] if T < 100 else [(T,), (200, 133), (130, 1, 1, 201)]):
        st = [torch.full((3,) + s, float("nan"), device=dev) for s in ((H, D, V), (H, D), (H,))]

        def run(s, e):
            sg = seg_meta([e - s], [s], [2], dev)
            if k % 2:        # the scale applied by the op itself, or handed on to the norm
                o, mul = S.matrix_memory(xd[s:e], H, D, V, f32(gb), cap, *st, sg), None
            else:
                o, mul = S.matrix_memory(xd[s:e], H, D, V, f32(gb), cap, *st, sg, defer_scale=True)
            return S.head_norm_gate(o, zero[s:e], ones, H, V, 1e-5, torch.float32, mul=mul)
        close(in_portions(run, T, cuts), want, torch.float32, scale=3.0 if T < 100 else 6.0)


@pytest.mark.parametrize("backend", BACKENDS)
def test_head_norm_gate_weight_shapes(backend):
    dev, dt = backend
    T, H, V = 5, 3, 70
    o, g = rnd(T, H * V, seed=1, std=3.0), rnd(T, H * V + 4, seed=2)
    for w in (rnd(V, seed=3) + 1.0, rnd(H * V, seed=4) + 1.0):
        want = O.unit_rms(o.view(T, H, V), 1e-4) * w.view(-1, V) * torch.sigmoid(g[:, 4:]).view(T, H, V)
        got = S.head_norm_gate(o.float().to(dev), g.float().to(dev)[:, 4:], w.float().to(dev), H, V, 1e-4, dt)
        close(got, want.reshape(T, -1), dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_two_sequences_in_one_step_keep_their_own_state(backend):
    """Recurrences of two sequences interleaved over two steps, with slots that are not in segment order."""
    dev, dt = backend
    H, D, V, cap = 2, 8, 6, 4.0
    xa, xb = rnd(9, 2 * H * (D + V) + 2 * H, seed=1), rnd(6, 2 * H * (D + V) + 2 * H, seed=2)
    gb = rnd(2 * H, seed=3)
    f32 = lambda z: z.float().to(dev)  # noqa: E731

    def alone(x):
        st = [torch.full((2,) + s, float("nan"), device=dev) for s in ((H, D, V), (H, D), (H,))]
        return S.matrix_memory(f32(x), H, D, V, f32(gb), cap, *st, seg_meta([x.shape[0]], [0], [1], dev))
    st = [torch.full((4,) + s, float("nan"), device=dev) for s in ((H, D, V), (H, D), (H,))]
    o1 = S.matrix_memory(f32(torch.cat([xa[:5], xb[:1]])), H, D, V, f32(gb), cap, *st, seg_meta([5, 1], [0, 0], [3, 0], dev))
    o2 = S.matrix_memory(f32(torch.cat([xb[1:], xa[5:]])), H, D, V, f32(gb), cap, *st, seg_meta([5, 4], [1, 5], [0, 3], dev))
    close(torch.cat([o1[:5], o2[5:]]), alone(xa), torch.float32)
    close(torch.cat([o1[5:], o2[:5]]), alone(xb), torch.float32)


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_and_short_portions_in_one_step(backend):
    """A portion long enough for the chunk-parallel kernels beside a short one and a single token: every
    sequence's result is what it gets alone."""
    dev, dt = backend
    H, G, D, V = 2, 1, 16, 24
    lens, pos0, slots = [200, 3, 1], [0, 5, 9], [2, 0, 1]
    T = sum(lens)
    x = rnd(T, 2 * G * D + H * V, seed=1).to(torch.bfloat16).double()
    a, beta = rnd(T, H * D, seed=2), rnd(T, H, seed=3)
    rate, bias = torch.exp(rnd(H, seed=4, std=0.5)), rnd(H * D, seed=5) - 0.5
    xm, gb = rnd(T, 2 * H * (D + V) + 2 * H, seed=6), rnd(2 * H, seed=7)
    f32 = lambda z: z.float().to(dev)  # noqa: E731

    def states(fill):
        return [torch.full((3,) + s, fill, device=dev) for s in ((H, D, V), (H, D, V), (H, D), (H,))]

    def run(st, xs, as_, bs, xms, sg):
        o1 = S.gated_delta(xs.to(dev).to(dt).contiguous(), H, G, D, V, f32(as_), f32(rate), f32(bias), f32(bs), st[0], sg)
        o2 = S.matrix_memory(f32(xms), H, D, V, f32(gb), 4.0, st[1], st[2], st[3], sg)
        return o1, o2
    together = states(0.25)                    # the two continuing sequences start from some state
    o1, o2 = run(together, x, a, beta, xm, seg_meta(lens, pos0, slots, dev))
    at = 0
    for n, p0, sl in zip(lens, pos0, slots):
        alone = states(0.25)
        w1, w2 = run(alone, x[at:at + n], a[at:at + n], beta[at:at + n], xm[at:at + n], seg_meta([n], [p0], [sl], dev))
        close(o1[at:at + n], w1, torch.float32, scale=5.0)
        close(o2[at:at + n], w2, torch.float32, scale=5.0)
        for u, v in zip(together, alone):
            close(u[sl], v[sl], torch.float32, scale=5.0)
        at += n


# ------------------------------------------------------------------ whole models
@pytest.mark.parametrize("backend", BACKENDS)
def test_layers_match_after_every_layer(backend):
    dev, dt = backend
    d = default_config()
    W = weights(d, 1)
    tokens = toks(45, d["vocab"], 2)
    want = []
    O.forward(d, W, tokens, want)
    eng = engine(d, W, backend)
    sid = eng.new_sequence()
    got = []
    fw = eng.model.forward
    eng.model.forward = lambda *a, **k: fw(*a, layers_out=got, **k)
    eng.feed([(sid, tokens, [])])
    assert len(got) == len(want) == len(d["layers"])
    for i, (g, w) in enumerate(zip(got, want)):
        e = float((g.double().cpu() - w).abs().max() / w.abs().max())
        assert e < (3e-5 if dt == torch.float32 else 1e-1), (i, e)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cuts", [(), (70,), (30, 2, 2, 17, 3, 5), (69,), (1, 68)])
def test_prefill_decode_and_portions_agree_with_oracle(backend, cuts):
    """() = token by token from the first token on; (70,) = one prefill; portions down to two tokens."""
    d = default_config()
    W = weights(d, 3)
    tokens = toks(70, d["vocab"], 4)
    want = O.forward(d, W, tokens)
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
    want = [O.forward(d, W, r) for r in reqs]
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


@pytest.mark.parametrize("backend", BACKENDS)
def test_edges_and_page_borders_with_sharp_scores(backend):
    """Large score scales: nearly all weight on one key, so a chunk, a window or the kept first tokens off by
    one show in the logits.  Edges at 24 / 48 (chunks), i - 20 (window), 5 (kept) and pages of 32."""
    d = config([(att(chunk=24, scale=6.0, softcap=50.0), 24), (par(window=20, keep=5, scale=9.0, rot=8), 0),
                (att(chunk=24, scale=6.0, softcap=0.0), 16)])
    W = weights(d, 6)
    tokens = toks(100, d["vocab"], 7)
    want = O.forward(d, W, tokens)
    for cuts in [(100,), (23, 2, 24, 15, 2, 30), (47,)]:
        eng = engine(d, W, backend)
        assert agrees(feed_all(eng, eng.new_sequence(), tokens, cuts), want, backend[1], mult=2.0), cuts


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_portions_then_decoding(backend):
    """Portions long enough for the chunk-parallel recurrences, cut off a chunk's border, then single tokens."""
    d = default_config()
    W = weights(d, 17)
    tokens = toks(330, d["vocab"], 18)
    want = O.forward(d, W, tokens)
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
        assert agrees(feed_all(eng, eng.new_sequence(), tokens, (n,)), O.forward(d, W, tokens), backend[1], mult=2.5), n


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_past_windows_and_chunks(backend):
    d = default_config()
    W = weights(d, 9)
    tokens = toks(150, d["vocab"], 10)
    want = O.forward(d, W, tokens)
    eng = engine(d, W, backend)
    got = feed_all(eng, eng.new_sequence(), tokens, (10,))           # 140 tokens one by one
    assert agrees(got, want, backend[1], mult=2.0)


OTHER = {
    "matrix_core_sizes": [(att(heads=4, kv_heads=2, dim=64, vdim=64, chunk=24), 32),
                          (par(heads=2, kv_heads=1, dim=128, vdim=64, window=20, keep=5, rot=64, mh=2, md=64, mv=64), 0),
                          (dlt(heads=2, kv_heads=1, dim=64, vdim=128), 16), (att(heads=4, kv_heads=2, dim=64, vdim=64, chunk=24), 0)],
    "one_head_everywhere": [(att(heads=1, kv_heads=1, dim=4, vdim=4), 8), (par(heads=1, kv_heads=1, mh=1), 8),
                            (dlt(heads=1, kv_heads=1), 8)],
    "delta_first_grouped_no_conv": [(dlt(heads=6, kv_heads=2, dim=5, vdim=3, conv=1, ra=1, rg=1), 0), (att(v_mix=False), 8)],
    "three_value_mixers": [(att(), 0), (att(heads=2, kv_heads=2, dim=4, vdim=12), 8), (par(), 0), (att(chunk=3), 8)],
    "no_masks_no_cap_no_rotation": [(att(chunk=0, softcap=0.0), 8), (par(window=0, keep=0, rot=0), 8)],
    "rotation_over_the_whole_head": [(par(dim=8, rot=8, keep=0, window=4), 8), (par(dim=6, rot=2, keep=9, window=2), 0)],
    "wide_taps_unaligned": [(dlt(heads=3, kv_heads=3, dim=7, vdim=9, conv=6), 10), (par(dim=10, vdim=7, rot=6, mh=2, md=5, mv=7), 0)],
    "no_feed_forward_at_all": [(att(), 0), (dlt(), 0)],
}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(backend, name):
    d = config(OTHER[name], width={"wide_taps_unaligned": 34, "matrix_core_sizes": 64}.get(name, 40), eps=1e-3,
               embed_scale=1.0)
    W = weights(d, 11)
    tokens = toks(40, d["vocab"], 12)
    want = O.forward(d, W, tokens)
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
        seq = list(p)
        for t in outs[i][:6]:
            lg = O.forward(d, W, seq)[-1, :eng.vocab]
            if backend[1] == torch.float32:
                assert t == int(lg.argmax()), i
            else:       # bf16: a near-tie may go the other way; the chosen token must be (nearly) the best
                assert float(lg.max() - lg[t]) < 0.1 * float(lg.std()), i
            seq.append(t)
        assert len(outs[i]) >= 6


def test_config_round_trip_registry_and_replay(tmp_path):
    """config.json -> configuration -> config.json; the registry picks the class by the file; a recorded
    schedule replayed through the engine gives the oracle's logits; tensors give the low-rank sizes."""
    from k8s_llm_rca_amd.engine import trace as TR
    from k8s_llm_rca_amd.models import lizesun as LZ
    from k8s_llm_rca_amd.models.registry import checkpoint_arch, get_any_config, load_model
    d = default_config()
    cfg = LizesunConfig.from_json(d, "x")
    assert LizesunConfig.from_json(cfg.to_json(), "x") == cfg
    assert get_any_config("tiny-lizesun").arch == "lizesun"
    W = weights(d, 21)
    d2 = json.loads(json.dumps(d))
    for L in d2["layers"]:                                    # a checkpoint's config.json does not name the ranks
        L["mixer"].pop("a_rank", None)
        L["mixer"].pop("g_rank", None)
    path = str(tmp_path / "ckpt")
    LZ.save_checkpoint(cfg, W, path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(d2, f)
    assert checkpoint_arch(path) == "lizesun"
    assert isinstance(load_model(path, "cpu", torch.float32), LizesunModel)
    eng = TR.make_engine(path, torch.float32, 128, device="cpu", state_slots=2, block_size=32)
    a, b = toks(40, d["vocab"], 22), toks(21, d["vocab"], 23)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[30:31], "want": [0]}, {"id": "b", "tokens": b[:20], "want": []}],
              "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}, {"id": "a", "tokens": a[31:], "want": [8]}],
              "end": ["a", "b"]}]
    import io
    out = str(tmp_path / "out")
    log = io.StringIO()
    TR.replay(eng, io.StringIO("\n".join(json.dumps(s) for s in steps)), out, log)
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    import numpy as np
    wa, wb = O.forward(d, W, a), O.forward(d, W, b)
    g0 = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, -1))
    g2 = torch.from_numpy(np.fromfile(os.path.join(out, "2.f32"), dtype="<f4").reshape(2, -1))
    assert agrees(g0, wa[[0, 29]], torch.float32) and agrees(g2, torch.stack([wb[20], wa[39]]), torch.float32)
    assert eng.kv.free_blocks == eng.kv.num_blocks and eng.states.free_slots == 2


def test_trace_run_command_line(tmp_path):
    from k8s_llm_rca_amd.models import lizesun as LZ
    d = default_config()
    W = weights(d, 31)
    path = str(tmp_path / "ckpt")
    LZ.save_checkpoint(LizesunConfig.from_json(d, "x"), W, path)
    tokens = toks(12, d["vocab"], 32)
    step = json.dumps({"step": 0, "entries": [{"id": "r", "tokens": tokens, "want": [11]}], "end": ["r"]})
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64", "--device", "cpu"], input=step + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "done 0" in r.stdout, r.stderr[-2000:]
    import numpy as np
    got = torch.from_numpy(np.fromfile(str(tmp_path / "o" / "0.f32"), dtype="<f4").reshape(1, -1))
    assert agrees(got, O.forward(d, W, tokens)[-1:], torch.float32)
