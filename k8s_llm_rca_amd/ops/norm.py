"""Fused residual-add + RMSNorm (B2) and SwiGLU (B8)."""
from __future__ import annotations

from typing import Optional

import torch

from ._lib import check, lib, ptr, stream_ptr, use_hip


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``y = rmsnorm(x + residual) * w``; when ``residual`` is given it is updated in place to ``x + residual``."""
    T, H = x.shape
    if out is None:
        out = torch.empty((T, H), dtype=x.dtype, device=x.device)
    if use_hip(x):
        assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and H % 8 == 0
        assert x.stride(1) == 1 and out.is_contiguous() and weight.is_contiguous() and H <= 16384
        if residual is not None:
            assert residual.is_contiguous() and residual.shape == (T, H)
        check(lib().k8s_rmsnorm(ptr(x), ptr(residual), ptr(weight), ptr(out), T, H, x.stride(0), out.stride(0),
                                float(eps), stream_ptr(x)), "rmsnorm")
        return out
    xf = x.float()
    if residual is not None:
        xf = xf + residual.float()
        residual.copy_(xf.to(residual.dtype))
        xf = residual.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    out.copy_((xf * torch.rsqrt(var + eps) * weight.float()).to(out.dtype))
    return out


def splitk_addnorm(part: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``rmsnorm(bf16(part.sum(0)) + residual) * w`` with ``residual`` updated in
    place: the reduction of a split-K GEMM's fp32 partials ``part``
    ``[splits, T, H]`` fused into the residual add + RMSNorm that consumes it
    (the native layer executor's epilogue for split-K o / down projections)."""
    S, T, H = part.shape
    if out is None:
        out = torch.empty((T, H), dtype=residual.dtype, device=residual.device)
    if use_hip(residual):
        assert part.dtype == torch.float32 and part.is_contiguous() and residual.is_contiguous()
        assert residual.shape == (T, H) and out.is_contiguous() and weight.dtype == torch.bfloat16
        check(lib().k8s_splitk_addnorm(ptr(part), S, ptr(residual), ptr(weight), ptr(out), T, H, out.stride(0),
                                       float(eps), stream_ptr(residual)), "splitk_addnorm")
        return out
    acc = part[0].clone()
    for s in range(1, S):
        acc += part[s]
    return rmsnorm(acc.to(residual.dtype), weight, eps, residual=residual, out=out)


def silu_mul(gu: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    T, I2 = gu.shape
    inter = I2 // 2
    if out is None:
        out = torch.empty((T, inter), dtype=gu.dtype, device=gu.device)
    if use_hip(gu):
        assert gu.is_contiguous() and out.is_contiguous() and inter % 8 == 0 and gu.dtype == torch.bfloat16
        check(lib().k8s_silu_mul(ptr(gu), ptr(out), T, inter, stream_ptr(gu)), "silu_mul")
        return out
    g, u = gu.float().split(inter, dim=-1)
    out.copy_((torch.nn.functional.silu(g) * u).to(out.dtype))
    return out


def nonfinite_flag(x: torch.Tensor, flag: torch.Tensor) -> None:
    """Debug: ``flag[0] = 1`` (int32, device) when ``x`` holds a NaN / inf;
    never clears it.  CPU tensors: the same test in PyTorch."""
    if use_hip(x):
        xc = x.contiguous()
        check(lib().k8s_nonfinite_flag(ptr(xc), xc.numel(), ptr(flag), stream_ptr(x)), "nonfinite_flag")
        return
    if not torch.isfinite(x).all():
        flag[0] = 1


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """PolyNorm activation of fp32 rows: ``a N(z) + b N(z^2) + c N(z^3) + e`` with ``coef = (a, b, c, e)``,
    powers element by element and ``N(v) = v / sqrt(mean(v^2) + eps)`` over the row."""
    T, F = z.shape
    out = torch.empty(T, F, dtype=out_dtype, device=z.device)
    if use_hip(z):
        assert z.dtype == torch.float32 and z.is_contiguous() and coef.dtype == out_dtype and coef.numel() == 4
        check(lib().k8s_polynorm(ptr(z), ptr(coef), ptr(out), T, F, float(eps), 0 if out_dtype == torch.bfloat16 else 1,
                                 stream_ptr(z)), "polynorm")
        return out
    a, b, c, e = [float(v) for v in coef.float()]

    def unit(v):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)

    out.copy_((a * unit(z) + b * unit(z * z) + c * unit(z * z * z) + e).to(out_dtype))
    return out


# ------------------------------------------------------------------ layer norms around an fp32 residual
# (csrc/kernels/norm_mix.hip).  The residual stream, the sublayer outputs and every small
# parameter (norm weights and biases, depth coefficients) are fp32; ``out_dtype`` is the
# activation type that the next GEMM reads.
def _odt(t: torch.dtype) -> int:
    if t == torch.bfloat16:
        return 0
    if t == torch.float32:
        return 1
    raise TypeError(f"activations must be bfloat16 or float32, not {t}")


def _ln(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w + b


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """``(x - mean) / sqrt(var + eps) * w + b`` of fp32 rows (two passes: the variance is the mean of the
    squared deviations)."""
    T, W = x.shape
    out = torch.empty(T, W, dtype=out_dtype, device=x.device)
    if use_hip(x):
        assert x.dtype == torch.float32 and x.is_contiguous() and w.dtype == b.dtype == torch.float32
        check(lib().k8s_layernorm(ptr(x), ptr(w), ptr(b), ptr(out), T, W, float(eps), _odt(out_dtype),
                                  stream_ptr(x)), "layernorm")
        return out
    out.copy_(_ln(x, w, b, eps).to(out_dtype))
    return out


def embed_layernorm(ids: torch.Tensor, embed: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float,
                    x_out: torch.Tensor, nw: Optional[torch.Tensor] = None, nb: Optional[torch.Tensor] = None,
                    out_dtype=None) -> Optional[torch.Tensor]:
    """``x_out = LN(embed[ids]; w, b)`` (fp32); with ``nw, nb`` also returns ``LN(x_out; nw, nb)`` as
    activations (the first layer's input norm, same pass)."""
    T, W = ids.shape[0], embed.shape[1]
    h = torch.empty(T, W, dtype=out_dtype, device=embed.device) if nw is not None else None
    if use_hip(embed):
        assert x_out.dtype == torch.float32 and x_out.is_contiguous() and x_out.shape == (T, W)
        assert embed.is_contiguous() and ids.dtype == torch.int32
        check(lib().k8s_embed_ln(ptr(ids), ptr(embed), _odt(embed.dtype), ptr(w), ptr(b), ptr(x_out), ptr(nw),
                                 ptr(nb), ptr(h), _odt(out_dtype) if h is not None else 1, T, W, float(eps),
                                 stream_ptr(embed)), "embed_ln")
        return h
    x_out.copy_(_ln(embed[ids.long()].float(), w, b, eps))
    if h is not None:
        h.copy_(_ln(x_out, nw, nb, eps).to(out_dtype))
    return h


def ln_residual(src: torch.Tensor, y: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], eps: float,
                dst: torch.Tensor, y2: Optional[torch.Tensor] = None, merge: Optional[str] = None,
                mw: Optional[tuple] = None, nw: Optional[torch.Tensor] = None, nb: Optional[torch.Tensor] = None,
                out_dtype=None, kind: str = "layer", row_gate: Optional[torch.Tensor] = None,
                cast: bool = False) -> Optional[torch.Tensor]:
    """``dst = src + LN(u; w, b)`` on fp32 rows (``dst`` may be ``src``), where ``u`` is the sublayer
    output ``y``, or two outputs joined: ``merge="sum"``: ``y + y2``; ``merge="rms"``:
    ``(unit_rms(y) mw[0] + unit_rms(y2) mw[1]) / 2``; ``merge="gated"``: ``y + sigmoid(row_gate) y2`` with one gate
    logit per row (``row_gate`` [T] or a column [T, 1] of a wider fp32 matrix).  ``kind="rms"``: the norm is
    ``u / sqrt(mean(u^2) + eps) * w`` instead (``b`` None).  With ``nw, nb`` also returns ``LN(dst; nw, nb)`` as
    activations (the next sublayer's input norm, same pass); with ``cast`` the new rows themselves as
    activations (the next sublayer reads the residual as it is)."""
    T, W = src.shape
    assert not (cast and nw is not None)
    h = torch.empty(T, W, dtype=out_dtype, device=src.device) if (nw is not None or cast) else None
    mode = {None: 0, "rms": 1, "sum": 2, "gated": 3}[merge if y2 is not None else None]
    knd = {"layer": 0, "rms": 1}[kind]
    if use_hip(src):
        for t in (src, y, dst) + ((y2,) if y2 is not None else ()):
            assert t.dtype == torch.float32 and t.is_contiguous() and t.shape == (T, W)
        wl, wr = mw if mode == 1 else (None, None)
        rgs = 0
        if mode == 3:
            assert row_gate.dtype == torch.float32 and row_gate.shape[0] == T and row_gate.numel() == T
            rgs = row_gate.stride(0)
        check(lib().k8s_ln_residual(ptr(src), ptr(y), ptr(y2), mode, ptr(wl), ptr(wr), ptr(w), ptr(b), ptr(dst),
                                    ptr(nw), ptr(nb), ptr(h), _odt(out_dtype) if h is not None else 1, T, W,
                                    float(eps), stream_ptr(src), knd, ptr(row_gate) if mode == 3 else 0, rgs),
              "ln_residual")
        return h
    if mode == 1:
        def unit(v):
            return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        u = 0.5 * (unit(y) * mw[0] + unit(y2) * mw[1])
    elif mode == 2:
        u = y + y2
    elif mode == 3:
        u = y + torch.sigmoid(row_gate.reshape(T, 1)) * y2
    else:
        u = y
    if knd == 1:
        dst.copy_(src + u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w)
    else:
        dst.copy_(src + _ln(u, w, b, eps))
    if nw is not None:
        h.copy_(_ln(dst, nw, nb, eps).to(out_dtype))
    elif cast:
        h.copy_(dst.to(out_dtype))
    return h


def embed_rows(ids: torch.Tensor, embed: torch.Tensor, x_out: torch.Tensor, out_dtype=None) -> Optional[torch.Tensor]:
    """``x_out = embed[ids]`` (fp32); with ``out_dtype`` also returns the rows as activations of that type."""
    T, W = ids.shape[0], embed.shape[1]
    h = torch.empty(T, W, dtype=out_dtype, device=embed.device) if out_dtype is not None else None
    if use_hip(embed):
        assert x_out.dtype == torch.float32 and x_out.is_contiguous() and x_out.shape == (T, W)
        assert embed.is_contiguous() and ids.dtype == torch.int32
        check(lib().k8s_embed_rows(ptr(ids), ptr(embed), _odt(embed.dtype), ptr(x_out), ptr(h),
                                   _odt(out_dtype) if h is not None else 1, T, W, stream_ptr(embed)), "embed_rows")
        return h
    x_out.copy_(embed[ids.long()].float())
    if h is not None:
        h.copy_(x_out.to(out_dtype))
    return h


def token_gate(a: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int, out_dtype) -> torch.Tensor:
    """``gelu_tanh(a) * table[ids, col0 : col0 + n]`` for fp32 ``a`` [T, n] as activations: a per-token input looked up
    by token id and gated by a projection of the hidden row (``gelu_tanh(z) = z / 2 (1 + tanh(sqrt(2 / pi)
    (z + 0.044715 z^3)))``)."""
    T, n = a.shape
    out = torch.empty(T, n, dtype=out_dtype, device=a.device)
    if use_hip(a):
        assert a.dtype == torch.float32 and a.is_contiguous() and table.is_contiguous() and ids.dtype == torch.int32
        check(lib().k8s_token_gate(ptr(a), ptr(ids), ptr(table), _odt(table.dtype), table.shape[1], int(col0),
                                   ptr(out), _odt(out_dtype), T, n, stream_ptr(a)), "token_gate")
        return out
    g = torch.nn.functional.gelu(a, approximate="tanh")
    out.copy_((g * table[ids.long(), col0:col0 + n].float()).to(out_dtype))
    return out


def depth_mix_ln(stack: torch.Tensor, n: int, coef: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float,
                 out_dtype, a_out: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None):
    """Weighted sum over depth: ``a = sum_{j < n} coef[j] * stack[j]`` (``stack`` [>= n, T, W] fp32 holds the
    embedding output and every layer's result) and its layer norm ``LN(a; w, b)`` as activations, one
    pass.  ``rows`` (int64 / int32 indices): only those rows, in that order.  Returns (a, h)."""
    _, T, W = stack.shape
    R = T if rows is None else rows.shape[0]
    if a_out is None:
        a_out = torch.empty(R, W, dtype=torch.float32, device=stack.device)
    h = torch.empty(R, W, dtype=out_dtype, device=stack.device)
    if use_hip(stack):
        assert stack.dtype == torch.float32 and stack.is_contiguous() and coef.dtype == torch.float32
        assert a_out.is_contiguous() and a_out.shape == (R, W) and n <= coef.shape[0] and n <= stack.shape[0]
        ri = None if rows is None else rows.to(torch.int32)
        check(lib().k8s_depth_mix_ln(ptr(stack), T, n, ptr(coef), ptr(ri), R, ptr(a_out), ptr(w), ptr(b), ptr(h),
                                     _odt(out_dtype), W, float(eps), stream_ptr(stack)), "depth_mix_ln")
        return a_out, h
    a = torch.zeros(T, W)
    for j in range(n):
        a += coef[j] * stack[j]
    if rows is not None:
        a = a[rows.long()]
    a_out.copy_(a)
    h.copy_(_ln(a_out, w, b, eps).to(out_dtype))
    return a_out, h


def softcap_(logits: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
    """In place on fp32 logits: ``cap * tanh(scale * z / cap)`` (``cap`` <= 0: only the scale)."""
    if use_hip(logits):
        assert logits.dtype == torch.float32 and logits.is_contiguous()
        check(lib().k8s_softcap(ptr(logits), logits.numel(), float(scale), float(cap), stream_ptr(logits)), "softcap")
        return logits
    logits.mul_(scale)
    if cap > 0:
        logits.copy_(cap * torch.tanh(logits / cap))
    return logits


# ------------------------------------------------------------------ Dynamic Tanh norm around an fp32 residual
# (csrc/kernels/dyt_ops.hip).  ``dyt(x) = tanh(alpha x) * w + b`` per element: no mean, no variance, so
# nothing couples a row's entries and the residual add, the norm and the cast are one elementwise pass.
def embed_scale_dyt(ids: torch.Tensor, embed: torch.Tensor, scale: float, x_out: torch.Tensor, alpha: float,
                    w: Optional[torch.Tensor], b: Optional[torch.Tensor], out_dtype) -> Optional[torch.Tensor]:
    """``x_out = embed[ids] * scale`` (fp32); with ``w, b`` also returns ``dyt(x_out)`` as activations."""
    T, W = ids.shape[0], embed.shape[1]
    h = torch.empty(T, W, dtype=out_dtype, device=embed.device) if w is not None else None
    if use_hip(embed):
        assert x_out.dtype == torch.float32 and x_out.is_contiguous() and x_out.shape == (T, W)
        assert embed.is_contiguous() and ids.dtype == torch.int32
        check(lib().k8s_embed_scale_dyt(ptr(ids), ptr(embed), _odt(embed.dtype), float(scale), ptr(x_out),
                                        float(alpha), ptr(w), ptr(b), ptr(h), _odt(out_dtype) if h is not None else 1,
                                        T, W, stream_ptr(embed)), "embed_scale_dyt")
        return h
    x_out.copy_(embed[ids.long()].float() * scale)
    if h is not None:
        h.copy_((torch.tanh(alpha * x_out) * w + b).to(out_dtype))
    return h


def add_dyt(x: torch.Tensor, y: Optional[torch.Tensor], sy: float = 1.0, y2: Optional[torch.Tensor] = None,
            sy2: float = 1.0, alpha: float = 1.0, w: Optional[torch.Tensor] = None, b: Optional[torch.Tensor] = None,
            out_dtype=None) -> Optional[torch.Tensor]:
    """In place on the fp32 residual: ``x += sy * y (+ sy2 * y2)`` (``y`` None: nothing is added); with
    ``w, b`` also returns ``tanh(alpha x) * w + b`` of the new rows as activations (the next sublayer's
    input norm, same pass)."""
    T, W = x.shape
    h = torch.empty(T, W, dtype=out_dtype, device=x.device) if w is not None else None
    if use_hip(x):
        for t in (x, y, y2):
            assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.shape == (T, W))
        assert y is not None or y2 is None
        if y is None and h is None:
            return None
        check(lib().k8s_add_dyt(ptr(x), ptr(y), float(sy), ptr(y2), float(sy2), float(alpha), ptr(w), ptr(b), ptr(h),
                                _odt(out_dtype) if h is not None else 1, T, W, stream_ptr(x)), "add_dyt")
        return h
    if y is not None:
        x.add_(sy * y if y2 is None else sy * y + sy2 * y2)
    if h is not None:
        h.copy_((torch.tanh(alpha * x) * w + b).to(out_dtype))
    return h


def relu_sq(u: torch.Tensor) -> torch.Tensor:
    """``max(u, 0)^2`` per element, in fp32, as ``u``'s type."""
    if use_hip(u):
        assert u.is_contiguous()
        out = torch.empty_like(u)
        check(lib().k8s_relu_sq(ptr(u), ptr(out), u.numel(), _odt(u.dtype), stream_ptr(u)), "relu_sq")
        return out
    return torch.relu(u.float()).pow(2).to(u.dtype)
