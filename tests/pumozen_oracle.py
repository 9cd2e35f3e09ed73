"""Pumozen, slowly: every mechanism of the design as one plain function over a whole sequence, in
float64, with no cache, no state and no batching.  Tests compare the engine with it; it shares no
code with the package.

``t`` maps tensor names of the safetensors file to tensors, ``cfg`` is config.json as a dict.
"""
import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def rotate(x, pos, dims, base):
    """x [T, heads, D]: entry i pairs with i + dims / 2 on the first ``dims`` entries of every head."""
    if not dims:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = pos.to(F64)[:, None] * f[None]
    co, si = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * co - v * si, v * co + u * si, x[..., dims:]], -1)


def causal_weights(s, sink):
    """s [T, T] scores -> weights over j <= i; ``sink``: one more term exp(0) in the denominator."""
    T = s.shape[0]
    vis = torch.ones(T, T).tril().bool()
    s = s.masked_fill(~vis, -math.inf)
    m = s.amax(-1, keepdim=True)
    if sink:
        m = m.clamp_min(0.0)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink:
        den = den + torch.exp(-m)
    return e / den


def attention(t, p, m, h, eps, kv=None):
    """The 'attention' mixer: values are the keys as projected; norm over the whole projection, then
    rotation; a sink of score 0 in the softmax.  Returns (output, (k, v)) with k, v as a cache holds them."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(T)
    rot = m.get("rot") or {}
    q = h @ t[p + "q"].to(F64).T
    q = unit_rms(q, eps) * t[p + "q.norm"].to(F64)
    q = rotate(q.view(T, H, D), pos, rot.get("dims", 0), rot.get("base", 10000.0))
    if kv is None:
        kr = h @ t[p + "k"].to(F64).T
        v = kr.view(T, G, D)
        k = unit_rms(kr, eps) * t[p + "k.norm"].to(F64)
        k = rotate(k.view(T, G, D), pos, rot.get("dims", 0), rot.get("base", 10000.0))
    else:
        k, v = kv
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        w = causal_weights(q[:, hh] @ k[:, g].T * m["scale"], sink=True)
        out[:, hh] = w @ v[:, g]
    return out.reshape(T, -1) @ t[p + "o"].to(F64).T, (k, v)


def attention_2(t, p, m, h, eps, kv=None):
    """The differential mixer: two softmax maps per head over the same values, joined with one lambda,
    a unit norm per head, a sigmoid output gate.  Returns (output, (k, v))."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ t[p + "q"].to(F64).T).view(T, H, 2, D)
    q = unit_rms(q, eps) * t[p + "q.norm"].to(F64)
    qt = m.get("q_temp")
    if qt:
        temp = 1.0 + qt["coef"] * torch.log(torch.div(pos + 1, qt["every"], rounding_mode="floor").to(F64) + 1.0)
        q = q * temp[:, None, None, None]
    if kv is None:
        k = (h @ t[p + "k"].to(F64).T).view(T, G, 2, D)
        k = unit_rms(k, eps) * t[p + "k.norm"].to(F64)
        v = (h @ t[p + "v"].to(F64).T).view(T, G, V)
    else:
        k, v = kv
    lam = (math.exp(float((t[p + "lq1"].to(F64) * t[p + "lk1"].to(F64)).sum()))
           - math.exp(float((t[p + "lq2"].to(F64) * t[p + "lk2"].to(F64)).sum())) + m["diff"])
    out = torch.zeros(T, H, V, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        a = [causal_weights(q[:, hh, j] @ k[:, g, j].T * m["scale"], sink=False) @ v[:, g] for j in range(2)]
        out[:, hh] = unit_rms(a[0] - lam * a[1], eps) * (1.0 - m["diff"])
    out = out.reshape(T, -1) * torch.sigmoid(h @ t[p + "g"].to(F64).T)
    return out @ t[p + "o"].to(F64).T, (k, v)


def mamba2(t, p, m, h, eps):
    """State-space duality layer, token by token."""
    T = h.shape[0]
    Hn, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = Hn * P
    zx = h @ t[p + "in"].to(F64).T
    z, xbc, dt = zx[:, :inner], zx[:, inner:2 * inner + 2 * G * N], zx[:, 2 * inner + 2 * G * N:]
    cw, cb = t[p + "conv"].to(F64), t[p + "conv.b"].to(F64)
    pad = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F64), xbc])
    conv = cb.expand(T, -1).clone()
    for j in range(taps):
        conv = conv + cw[:, j] * pad[j:j + T]
    xbc = silu(conv)
    x = xbc[:, :inner].view(T, Hn, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + t[p + "dt_bias"].to(F64))
    rate = torch.exp(t[p + "A_log"].to(F64))
    Dk = t[p + "D"].to(F64)
    y = torch.zeros(T, Hn, P, dtype=F64)
    S = torch.zeros(Hn, N, P, dtype=F64)
    for i in range(T):
        for hh in range(Hn):
            g = hh // (Hn // G)
            S[hh] = torch.exp(-rate[hh] * dt[i, hh]) * S[hh] + dt[i, hh] * torch.outer(B[i, g], x[i, hh])
            y[i, hh] = S[hh].T @ C[i, g] + Dk[hh] * x[i, hh]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * t[p + "norm"].to(F64)
    return y @ t[p + "o"].to(F64).T


def gated_unit(t, p, h, limit):
    g = (h @ t[p + "gate"].to(F64).T).clamp(max=limit)
    u = (h @ t[p + "up"].to(F64).T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ t[p + "down"].to(F64).T


def feed_forward(t, p, f, h):
    if f["kind"] == "dense":
        return gated_unit(t, p, h, f["limit"])
    r = f["router"]
    s = torch.softmax(h @ t[p + "router"].to(F64).T, -1)
    top = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :r["top"]]
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        w = s[i, top[i]]
        w = w / (w.sum() + 1e-20) * r.get("scale", 1.0)
        for e, we in zip(top[i].tolist(), w):
            out[i] += we * gated_unit(t, f"{p}e{e}.", h[i:i + 1], f["expert"]["limit"])[0]
    sh = f.get("shared")
    if sh:
        out = out + gated_unit(t, p + "shared.", h, sh["limit"]) * torch.sigmoid(h @ t[p + "shared.sg"].to(F64).T)
    return out


def token_side(t, cfg, i, ids, x, eps):
    dim = cfg["token_side"]["dim"]
    e = t["side.embed"].to(F64)[ids][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ t[f"l{i}.side.gate"].to(F64).T) * e
    y = g @ t[f"l{i}.side.proj"].to(F64).T
    return x + unit_rms(y, eps) * t[f"l{i}.side.norm"].to(F64)


def forward(t, cfg, ids, layers_out=None):
    """Logits [T, vocab] of one whole sequence ``ids`` (a list of ints)."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x = t["embed"].to(F64)[ids]
    cached = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        if L["type"] == "mamba2":
            y = mamba2(t, p, m, x, eps)
        else:
            fn = attention if L["type"] == "attention" else attention_2
            y, kv = fn(t, p, m, x, eps, cached[m["kv_from"]] if m.get("kv_from") is not None else None)
            cached[i] = kv
        x = x + layer_norm(y, t[f"l{i}.norm1"].to(F64), t[f"l{i}.norm1.b"].to(F64), eps)
        if L.get("mlp") is not None:
            y = feed_forward(t, f"l{i}.mlp.", L["mlp"], x)
            x = x + layer_norm(y, t[f"l{i}.norm2"].to(F64), t[f"l{i}.norm2.b"].to(F64), eps)
        if cfg.get("token_side"):
            x = token_side(t, cfg, i, ids, x, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, t["final.norm"].to(F64), t["final.norm.b"].to(F64), eps)
    return x @ t["embed"].to(F64).T
