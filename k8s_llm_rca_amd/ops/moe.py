"""MoE routing ops (B11/B12): top-k router, expert permutation, weighted combine."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ._lib import check, lib, ptr, scratch, stream_ptr, use_hip


def route_topk(logits: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """softmax -> top-k -> renormalise.  Returns (weights fp32 [T,k], ids int32 [T,k])."""
    T, E = logits.shape
    if use_hip(logits):
        assert logits.dtype == torch.bfloat16 and logits.is_contiguous()
        w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
        ids = torch.empty(T, k, dtype=torch.int32, device=logits.device)
        check(lib().k8s_moe_route(ptr(logits), T, E, k, ptr(w), ptr(ids), stream_ptr(logits)), "moe_route")
        return w, ids
    p = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(p, k, dim=-1)
    return w / w.sum(-1, keepdim=True), ids.int()


def align(ids: torch.Tensor, E: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sort the T*k (token, slot) pairs by expert.  Returns (order, inv, offsets[E+1]) int32."""
    flat = ids.reshape(-1).contiguous()
    n = flat.numel()
    if use_hip(flat):
        order = torch.empty(n, dtype=torch.int32, device=flat.device)
        inv = torch.empty(n, dtype=torch.int32, device=flat.device)
        offsets = torch.empty(E + 1, dtype=torch.int32, device=flat.device)
        check(lib().k8s_moe_align(ptr(flat), n, E, 0, ptr(order), ptr(inv), ptr(offsets), stream_ptr(flat)),
              "moe_align")
        return order, inv, offsets
    order = torch.argsort(flat.long(), stable=True).int()
    inv = torch.empty_like(order)
    inv[order.long()] = torch.arange(n, dtype=torch.int32)
    counts = torch.bincount(flat.long(), minlength=E)
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(counts, 0).int()
    return order, inv, offsets


def combine(y_perm: torch.Tensor, inv: torch.Tensor, w: torch.Tensor, T: int, k: int) -> torch.Tensor:
    """out[t] = sum_j w[t,j] * y_perm[inv[t*k+j]]."""
    H = y_perm.shape[1]
    out = torch.empty(T, H, dtype=y_perm.dtype, device=y_perm.device)
    if use_hip(y_perm):
        assert y_perm.is_contiguous() and w.dtype == torch.float32
        check(lib().k8s_moe_combine(ptr(y_perm), ptr(inv), ptr(w), T, k, H, ptr(out), stream_ptr(y_perm)),
              "moe_combine")
        return out
    g = y_perm.float()[inv.long()].view(T, k, H)
    out.copy_((g * w.view(T, k, 1)).sum(1).to(out.dtype))
    return out


def grouped_gemm(a: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, fuse_silu: bool = False,
                 out: Optional[torch.Tensor] = None, splits: int = 1, glds: int = 0) -> torch.Tensor:
    """B13: rows offsets[e]..offsets[e+1] of ``a`` times ``w[e]^T`` for every
    expert in one launch (``w`` [E, N, K]).  ``fuse_silu``: ``a`` is the
    gate_up output [rows, 2K] and the activation silu(gate) * up is formed on
    the fly.  ``splits`` > 1 splits K over workgroups (fp32 partials + a
    reduce; see grouped_gemm.hip).  ``glds`` = 10 + NB runs the LDS-DMA strip
    kernel with NB stages instead (64-row tiles: decode batches).  Offsets stay
    on the device (no host sync)."""
    E, N, K = w.shape
    rows = a.shape[0]
    if out is None:
        out = torch.empty(rows, N, dtype=a.dtype, device=a.device)
    if rows == 0:
        return out
    if glds and use_hip(a) and a.dtype == torch.bfloat16 and not fuse_silu and N % 64 == 0 and K % (64 * splits) == 0:
        # the LDS-DMA strip kernel (csrc/kernels/gemm_stream.hip grouped_glds_kernel)
        assert a.dtype == torch.bfloat16 and w.is_contiguous() and a.stride(1) == 1 and out.is_contiguous()
        max_tiles = (rows + 63) // 64 + E
        part = _split_scratch(a.device, splits * rows * N) if splits > 1 else None
        check(lib().k8s_grouped_glds(ptr(a), a.stride(0), ptr(w), ptr(out), out.stride(0), ptr(offsets), E, N, K,
                                     max_tiles, glds, splits, ptr(part), rows, stream_ptr(a)), "grouped_glds")
        return out
    if use_hip(a) and a.dtype == torch.bfloat16 and N % 128 == 0 and K % (64 * splits) == 0:
        assert a.dtype == torch.bfloat16 and w.is_contiguous() and a.stride(1) == 1 and out.is_contiguous()
        assert a.shape[1] == (2 * K if fuse_silu else K)
        max_tiles = (rows + 63) // 64 + E
        part = _split_scratch(a.device, splits * rows * N) if splits > 1 else None
        check(lib().k8s_grouped_gemm(ptr(a), a.stride(0), ptr(w), ptr(out), out.stride(0), ptr(offsets), E, N, K,
                                     max_tiles, int(fuse_silu), splits, ptr(part), rows, stream_ptr(a)),
              "grouped_gemm")
        return out
    if use_hip(a) and not fuse_silu and a.dtype == w.dtype and a.dtype in (torch.bfloat16, torch.float32):
        # any shape, bf16 or fp32, offsets read on the device (csrc/kernels/ffn_ops.hip)
        assert w.is_contiguous() and a.is_contiguous() and out.is_contiguous() and a.shape[1] == K
        check(lib().k8s_grouped_any(ptr(a), ptr(w), ptr(offsets), ptr(out), rows, E, N, K,
                                    0 if a.dtype == torch.bfloat16 else 1, stream_ptr(a)), "grouped_any")
        return out
    offs = offsets.tolist()
    for e in range(E):
        lo, hi = offs[e], offs[e + 1]
        if hi <= lo:
            continue
        x = a[lo:hi].float()
        if fuse_silu:
            x = torch.nn.functional.silu(x[:, :K]) * x[:, K:]
        out[lo:hi] = (x @ w[e].float().t()).to(out.dtype)
    return out


def grouped_big_ok(rows: int, N: int, K: int, silu: bool) -> bool:
    """What the grouped form of csrc/kernels/gemm_big.hip accepts."""
    return rows > 0 and K % 128 == 0 and N % (128 if silu else 256) == 0


def grouped_big(x: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor, silu: bool = False,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """B13 at prefill sizes on the 8-phase MFMA GEMM (csrc/kernels/gemm_big.hip,
    grouped form): rows offsets[e]..offsets[e+1] of ``x`` times ``w[e]^T`` in one
    launch with the offsets read on the device (no host sync, capturable).
    ``silu``: ``w`` [E, 2I, K] is the gate_up weight (gate rows first) and the
    result is the SwiGLU activation [rows, I] -- gate_up is never written."""
    from .linear import BIG_PIPE
    E, Nw, K = w.shape
    N = Nw // 2 if silu else Nw
    rows = x.shape[0]
    if out is None:
        out = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    if rows == 0:
        return out
    assert x.dtype == torch.bfloat16 and w.is_contiguous() and x.stride(1) == 1 and x.shape[1] == K
    assert offsets.dtype == torch.int32 and offsets.is_cuda and grouped_big_ok(rows, N, K, silu)
    check(lib().k8s_gemm_big_grouped(ptr(x), x.stride(0), ptr(w), ptr(out), out.stride(0), ptr(offsets), E, rows, N,
                                     K, int(silu), BIG_PIPE, stream_ptr(x)), "gemm_big_grouped")
    return out


_scratch = {}


def _split_scratch(dev: torch.device, n: int) -> torch.Tensor:
    t = _scratch.get(dev)
    if t is None or t.numel() < n:
        if t is not None:  # never freed: graphs captured earlier replay at its address (ops/linear.py _scratch)
            from . import linear as LIN
            LIN._retired_scratch.append(t)
        t = scratch(max(n, 1 << 20), torch.float32, dev)
        _scratch[dev] = t
    return t


def reserve_split_scratch(dev: torch.device, max_rows: int, N: int, splits: int) -> None:
    """Allocate the split-K partial buffer before any HIP-graph capture."""
    _split_scratch(dev, max_rows * N * splits)


# ------------------------------------------------------------------ routers and gated units beside Mixtral's
def _dt(t: torch.dtype) -> int:
    return 0 if t == torch.bfloat16 else 1


def route_direct(h: torch.Tensor, w_router: torch.Tensor, k: int, scoring: str = "sigmoid",
                 renorm: bool = False, choice_bias: Optional[torch.Tensor] = None,
                 renorm_eps: float = 0.0, scale: float = 1.0, extra_rows: int = 0):
    """Router straight from the hidden rows: fp32 logits ``h @ w_router.T``, scores by ``scoring``
    ("sigmoid" or "softmax"), the ``k`` largest (ties: lowest index), renormalised only with
    ``renorm`` (divided by their sum + ``renorm_eps``), then times ``scale``.  With ``choice_bias`` (fp32 [E])
    the experts are chosen by score + bias while the weights are the plain scores.
    Returns (weights fp32 [T, k], ids int32 [T, k]).  With ``extra_rows`` = X the last X rows of ``w_router``
    are not experts: their fp32 logits are returned as a third result [T, X] (gates that read the same rows)."""
    T, W = h.shape
    X = int(extra_rows)
    E = w_router.shape[0] - X
    if use_hip(h):
        assert h.is_contiguous() and w_router.is_contiguous() and h.dtype == w_router.dtype
        w = torch.empty(T, k, dtype=torch.float32, device=h.device)
        ids = torch.empty(T, k, dtype=torch.int32, device=h.device)
        extra = torch.empty(T, X, dtype=torch.float32, device=h.device) if X else None
        check(lib().k8s_router(ptr(h), ptr(w_router), T, W, E, k, 0 if scoring == "sigmoid" else 1, int(renorm),
                               ptr(w), ptr(ids), _dt(h.dtype), stream_ptr(h), ptr(choice_bias), float(renorm_eps),
                               X, ptr(extra), float(scale)), "router")
        return (w, ids, extra) if X else (w, ids)
    z = h.float() @ w_router.float().t()
    extra = z[:, E:].contiguous()
    z = z[:, :E]
    s = torch.sigmoid(z) if scoring == "sigmoid" else torch.softmax(z, -1)
    # stable descending sort: equal scores keep the lower expert first
    c = s if choice_bias is None else s + choice_bias.float()
    order = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :k]
    w = torch.gather(s, 1, order)
    if renorm:
        w = w / (w.sum(-1, keepdim=True) + renorm_eps)
    if scale != 1.0:
        w = w * scale
    return (w, order.int(), extra) if X else (w, order.int())


def gather_rows(h: torch.Tensor, order: torch.Tensor, k: int, w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of ``h`` in expert order (``order`` from :func:`align`), each scaled by its routing weight
    ``w`` [T, k] when the weight multiplies the expert's input."""
    n, W = order.numel(), h.shape[1]
    if use_hip(h):
        assert h.is_contiguous() and (w is None or (w.dtype == torch.float32 and w.is_contiguous()))
        xp = torch.empty(n, W, dtype=h.dtype, device=h.device)
        check(lib().k8s_moe_gather(ptr(h), ptr(order), ptr(w), ptr(xp), n, W, k, _dt(h.dtype), stream_ptr(h)),
              "moe_gather")
        return xp
    xp = h.float()[(order // k).long()]
    if w is not None:
        xp = xp * w.reshape(-1)[order.long()][:, None]
    return xp.to(h.dtype)


def glu_clamp(gu: torch.Tensor, alpha: float, limit: float, up_shift: float = 1.0) -> torch.Tensor:
    """Clamped gated unit on ``gu`` [rows, 2F] = (gate | up): ``g = min(gate, limit)``,
    ``u = clamp(up, -limit, limit)``, result ``g * sigmoid(alpha g) * (u + up_shift)``."""
    rows, F2 = gu.shape
    F = F2 // 2
    if use_hip(gu):
        assert gu.is_contiguous()
        out = torch.empty(rows, F, dtype=gu.dtype, device=gu.device)
        check(lib().k8s_glu_clamp(ptr(gu), ptr(out), rows, F, float(alpha), float(limit), float(up_shift),
                                  _dt(gu.dtype), stream_ptr(gu)), "glu_clamp")
        return out
    g = gu[:, :F].float().clamp(max=limit)
    u = gu[:, F:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + up_shift)).to(gu.dtype)


def combine_f32(y_perm: torch.Tensor, inv: torch.Tensor, T: int, k: int,
                w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 ``out[t] = sum_j (w[t, j] or 1) * y_perm[inv[t k + j]]``."""
    W = y_perm.shape[1]
    if use_hip(y_perm):
        assert y_perm.is_contiguous()
        out = torch.empty(T, W, dtype=torch.float32, device=y_perm.device)
        check(lib().k8s_moe_combine_f32(ptr(y_perm), ptr(inv), ptr(w), ptr(out), T, W, k, _dt(y_perm.dtype),
                                        stream_ptr(y_perm)), "moe_combine_f32")
        return out
    g = y_perm.float()[inv.long()].view(T, k, W)
    if w is not None:
        g = g * w.view(T, k, 1)
    return g.sum(1)


BIG_MIN_ROWS = 2048   # above: the prefill-size grouped GEMM (gemm_big.hip), as the Mixtral block picks it


def grouped_auto(a: torch.Tensor, w: torch.Tensor, offsets: torch.Tensor) -> torch.Tensor:
    """``grouped_gemm`` with the kernel chosen by size: the grouped form of the prefill GEMM for
    many rows, the weight-streaming grouped kernel for decode-size batches, the any-shape kernel
    (or fp32) otherwise.  None of them reads the offsets on the host."""
    E, N, K = w.shape
    if (use_hip(a) and a.dtype == torch.bfloat16 and a.shape[0] > BIG_MIN_ROWS
            and grouped_big_ok(a.shape[0], N, K, False)):
        return grouped_big(a, w, offsets)
    return grouped_gemm(a, w, offsets)
