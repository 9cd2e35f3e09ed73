"""A plain, slow implementation of the Lizesun decoder: float64, one whole sequence at a time,
token by token where there is a recurrence, no cache, no batching.  One function per
mechanism; nothing here is shared with the package.

``cfg`` is the config.json dictionary, ``t`` maps tensor names to float64 tensors.
"""
import torch

F64 = torch.float64


def dyt(x, t, name):
    """Dynamic Tanh: tanh(alpha x) * w + b (no statistics of x)."""
    return torch.tanh(t[name + ".alpha"] * x) * t[name] + t[name + ".b"]


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def relu_sq_ff(h, t, p):
    return (torch.relu(h @ t[p + "up"].T) ** 2) @ t[p + "down"].T


def rotate_half(x, pos, dims, base):
    """x [n, heads, dim]: entry i of the first ``dims`` is paired with entry i + dims / 2."""
    if not dims:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = pos.to(F64)[:, None] * f[None]
    c, s = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def masked_softmax_attention(q, k, v, scale, visible, softcap=0.0, sink=None):
    """q [n, H, D], k [n, G, D], v [n, G, V]; ``visible(i, j)`` for j <= i.  A sink adds exp(sink_h)
    to head h's denominator (no key, no value)."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[-1], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(n):
            js = torch.tensor([j for j in range(i + 1) if visible(i, j)])
            s = (k[js, g] @ q[i, h]) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            m = s.max()
            if sink is not None:
                m = torch.maximum(m, sink[h])
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e[:, None] * v[js, g]).sum(0) / den
    return out


def chunked_attention(h, t, p, m, eps, v_first):
    """The 'attention' mixer.  Returns (output, this layer's values before mixing or None)."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T + t[p + "q.b"]).view(n, H, D)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).view(n, G, D)
    v = (h @ t[p + "v"].T + t[p + "v.b"]).view(n, G, V)
    q = unit_rms(q, eps) * t[p + "q.norm"]
    k = unit_rms(k, eps) * t[p + "k.norm"]
    mine = None
    if m.get("v_mix"):
        if v_first is None:
            mine = v
        else:
            lam = t[p + "vmix"]
            v = (1.0 - lam) * v + lam * v_first
    c = int((m.get("mask") or {}).get("size", 0))        # no mask: plain causal
    o = masked_softmax_attention(q, k, v, float(m["scale"]), lambda i, j: not c or i // c == j // c,
                                 softcap=float(m.get("softcap") or 0.0))
    o = o * torch.sigmoid(h @ t[p + "g"].T)[:, :, None]
    return o.reshape(n, H * V) @ t[p + "o"].T, mine


def window_sink_attention(h, t, p, m, eps):
    """The left half of the 'parallel' mixer."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}       # no rot: no rotation
    q = rotate_half((h @ t[p + "q"].T).view(n, H, D), pos, int(rot["dims"]), float(rot["base"]))
    k = rotate_half((h @ t[p + "k"].T).view(n, G, D), pos, int(rot["dims"]), float(rot["base"]))
    v = (h @ t[p + "v"].T).view(n, G, V)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    mask = m.get("mask") or {}
    w, kf = int(mask.get("size", 0)), int(mask.get("keep_first", 0))
    o = masked_softmax_attention(q, k, v, float(m["scale"]), lambda i, j: not w or i - j < w or j < kf,
                                 sink=t[p + "sink"])
    return o.reshape(n, H * V) @ t[p + "o"].T


def matrix_memory(h, t, p, m, eps):
    """The right half of the 'parallel' mixer: a matrix memory with exponential gates kept stable by a
    running maximum that starts at 0."""
    n = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ t[p + "q"].T).view(n, H, D) * D ** -0.5
    k = (h @ t[p + "k"].T).view(n, H, D)
    v = (h @ t[p + "v"].T).view(n, H, V)
    ig = cap * torch.tanh((h @ t[p + "i"].T + t[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ t[p + "f"].T + t[p + "f.b"]) / cap))
    S = torch.zeros(H, D, V, dtype=F64)
    nn = torch.zeros(H, D, dtype=F64)
    mm = torch.zeros(H, dtype=F64)
    out = torch.zeros(n, H, V, dtype=F64)
    for i in range(n):
        m_new = torch.maximum(fg[i] + mm, ig[i])
        a, b = torch.exp(fg[i] + mm - m_new), torch.exp(ig[i] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[i][:, :, None] * v[i][:, None, :]
        nn = a[:, None] * nn + b[:, None] * k[i]
        mm = m_new
        num = torch.einsum("hdv,hd->hv", S, q[i])
        den = torch.maximum((nn * q[i]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
        out[i] = num / den[:, None]
    o = unit_rms(out, eps).reshape(n, H * V) * t[p + "norm"] * torch.sigmoid(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def causal_conv_silu(x, w):
    """x [n, C], w [C, taps] (last column = the current token), zeros before the start, then SiLU."""
    n, taps = x.shape[0], w.shape[1]
    ext = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=F64), x])
    y = sum(w[:, j] * ext[j:j + n] for j in range(taps))
    return y * torch.sigmoid(y)


def channel_delta(h, t, p, m, eps):
    """Gated delta rule with one decay per head and key channel."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ t[p + "q"].T, t[p + "q.conv"]).view(n, G, D)
    k = causal_conv_silu(h @ t[p + "k"].T, t[p + "k.conv"]).view(n, G, D)
    v = causal_conv_silu(h @ t[p + "v"].T, t[p + "v.conv"]).view(n, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ t[p + "b"].T)
    lo = (h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "dt_bias"]
    g = torch.exp(-torch.exp(t[p + "A_log"])[None, :, None] * torch.nn.functional.softplus(lo).view(n, H, D))
    S = torch.zeros(H, D, V, dtype=F64)
    out = torch.zeros(n, H, V, dtype=F64)
    for i in range(n):
        for hh in range(H):
            kk, qq = k[i, hh // (H // G)], q[i, hh // (H // G)]
            Sh = g[i, hh][:, None] * S[hh]
            u = beta[i, hh] * (v[i, hh] - Sh.T @ kk)
            Sh = Sh + kk[:, None] * u[None, :]
            S[hh] = Sh
            out[i, hh] = Sh.T @ qq
    gate = torch.sigmoid((h @ t[p + "g1"].T) @ t[p + "g2"].T).view(n, H, V)
    o = unit_rms(out, eps) * t[p + "norm"] * gate
    return o.reshape(n, H * V) @ t[p + "o"].T


def forward(cfg, t, tokens, layers_out=None):
    """Logits [n, vocab] (float64) of one sequence; ``layers_out`` receives the residual after every layer."""
    t = {k: v.to(F64) for k, v in t.items()}
    eps = float(cfg["norm"]["eps"])
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    v_first = None
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = dyt(x, t, p + "norm1")
        if L["type"] == "attention":
            y, mine = chunked_attention(h, t, p + "mix.", m, eps, v_first)
            if mine is not None:
                v_first = mine
        elif L["type"] == "parallel":
            y = (float(m["left_scale"]) * window_sink_attention(h, t, p + "mix.left.", m["left"], eps)
                 + float(m["right_scale"]) * matrix_memory(h, t, p + "mix.right.", m["right"], eps))
        elif L["type"] == "channel_delta":
            y = channel_delta(h, t, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + y
        if L.get("mlp") is not None:
            x = x + relu_sq_ff(dyt(x, t, p + "norm2"), t, p + "mlp.")
        if layers_out is not None:
            layers_out.append(x.clone())
    return dyt(x, t, "final.norm") @ t["head"].T
