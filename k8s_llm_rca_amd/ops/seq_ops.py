"""Ops of layers that carry per-sequence state besides the paged cache:
sinusoidal positions, the short causal convolution in front of a sublayer, the
minGRU recurrence, the post-sublayer norm of an fp32 residual, attention over a
paged latent cache (``csrc/kernels/seq_ops.hip``, ``latent_attn.hip``), window
attention and recurrent mixers (``mixer_ops.hip``, ``window_attn.hip``), masked
softmax attention behind a q / k preparation pass and matrix-state recurrences
(``masked_attn.hip``, ``matrix_mem.hip``).

A step's rows come in SEGMENTS (:class:`SegMeta`): consecutive rows of one
sequence -- a decode token or a portion of a prompt.  Device tensors run the HIP
kernels; CPU tensors the fp32 PyTorch forms below (the engine's CPU backend).
The residual stream, norms, recurrence and softmax are fp32 in both; ``dt`` is
the activation / weight type (bf16 or fp32).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np

import torch

from ._lib import check, lib, ptr, scratch, stream_ptr, use_hip

DECODE_PART = 256   # keys per partition of a decode row (split-KV); borders depend on the key index only


@dataclass
class SegMeta:
    n_seg: int
    row_seg: torch.Tensor      # [T] int32: segment of every row
    seg_row0: torch.Tensor     # [n_seg + 1] int32 row offsets
    seg_pos0: torch.Tensor     # [n_seg] int32 position of the segment's first token
    seg_slot: torch.Tensor     # [n_seg] int32 state slot of the segment's sequence
    block_tables: torch.Tensor  # [n_seg, maxb] int32 cache pages
    row0_host: List[int]
    pos0_host: List[int]
    slot_host: List[int]
    # rows [0, n_single) take the decode kernels (single tokens, short portions); the rest are prompt portions
    n_single: int = 0
    _items: Dict[int, tuple] = field(default_factory=dict)

    def attn_items(self, tokens_per_item: int) -> tuple:
        """Work items of the MFMA attention kernels, made once per step and item size:
        (decode items [n, 4] int32 on the device, prompt items, most keys a decode row sees).
        An item is (segment, first row, tokens, position of the first row's token); a segment's prompt
        items are padded with empty ones to a multiple of four."""
        got = self._items.get(tokens_per_item)
        if got is not None:
            return got
        dec, pre, kmax = [], [], 0
        for s in range(self.n_seg):
            a, b, p0 = self.row0_host[s], self.row0_host[s + 1], self.pos0_host[s]
            if a < self.n_single:
                dec += [(s, r, 1, p0 + r - a) for r in range(a, b)]
                kmax = max(kmax, p0 + b - a)
            else:
                pre += [(s, r, min(tokens_per_item, b - r), p0 + r - a) for r in range(a, b, tokens_per_item)]
                pre += [(s, a, 0, p0)] * (-len(pre) % 4)   # a workgroup's four waves share one segment's keys
        host = torch.from_numpy(np.asarray(dec + pre, dtype=np.int32).reshape(-1, 4))
        dev = self.row_seg.device
        if dev.type == "cuda":
            host = host.pin_memory()
        both = host.to(dev, non_blocking=True)
        got = (both[:len(dec)], both[len(dec):], kmax)
        self._items[tokens_per_item] = got
        return got


    def tile_items(self, tokens_per_item: int) -> torch.Tensor:
        """Every segment cut into tiles of at most ``tokens_per_item`` consecutive tokens ([n, 4] int32 on
        the device: segment, first row, tokens, position of the first token), made once per step."""
        key = ("tiles", tokens_per_item)
        got = self._items.get(key)
        if got is None:
            it = [(s, r, min(tokens_per_item, self.row0_host[s + 1] - r), self.pos0_host[s] + r - self.row0_host[s])
                  for s in range(self.n_seg) for r in range(self.row0_host[s], self.row0_host[s + 1], tokens_per_item)]
            host = torch.from_numpy(np.asarray(it, dtype=np.int32).reshape(-1, 4))
            if self.row_seg.device.type == "cuda":
                host = host.pin_memory()
            got = self._items[key] = host.to(self.row_seg.device, non_blocking=True)
        return got

    def chunk_ranges(self, rows: int, min_rows: int) -> Optional[tuple]:
        """Segments cut into chunks of at most ``rows`` rows, for recurrences that run the chunks in
        parallel: (chunks [n, 4] int32: segment, first row, rows, 0; seg_chunk0 [n_seg + 1] int32), both on
        the device; None when no segment has more than ``min_rows`` rows (the sequential kernel runs)."""
        key = ("ranges", rows, min_rows)
        if key in self._items:
            return self._items[key]
        out = None
        if max(b - a for a, b in zip(self.row0_host[:-1], self.row0_host[1:])) > min_rows:
            ch, c0 = [], [0]
            for s in range(self.n_seg):
                a, b = self.row0_host[s], self.row0_host[s + 1]
                ch += [(s, r, min(rows, b - r), 0) for r in range(a, b, rows)]
                c0.append(len(ch))
            host = torch.from_numpy(np.asarray([v for c in ch for v in c] + c0, dtype=np.int32))
            if self.row_seg.device.type == "cuda":
                host = host.pin_memory()
            dev = host.to(self.row_seg.device, non_blocking=True)
            out = (dev[:4 * len(ch)].view(-1, 4), dev[4 * len(ch):])
        self._items[key] = out
        return out

    def scan_chunks(self, rows: int) -> Optional[torch.Tensor]:
        """Chunks of at most ``rows`` rows for the time-parallel recurrence ([n, 4] int32 on the device:
        segment, first row, rows, index of the segment's first chunk); None when no segment is longer
        than two chunks (the sequential kernel runs)."""
        key = -rows
        if key in self._items:
            return self._items[key]
        out = None
        if max(b - a for a, b in zip(self.row0_host[:-1], self.row0_host[1:])) > 2 * rows:
            ch = []
            for s in range(self.n_seg):
                a, b, first = self.row0_host[s], self.row0_host[s + 1], len(ch)
                ch += [(s, r, min(rows, b - r), first) for r in range(a, b, rows)]
            host = torch.from_numpy(np.asarray(ch, dtype=np.int32))
            if self.row_seg.device.type == "cuda":
                host = host.pin_memory()
            out = host.to(self.row_seg.device, non_blocking=True)
        self._items[key] = out
        return out


SCAN_CHUNK = 64     # rows per chunk of the time-parallel minGRU
SSM_CHUNK = 64      # rows per chunk of the time-parallel selective scan and retention
SEQ_FILL_LANES = 1 << 18   # sequential lanes (segments x channels) from which the chunk-parallel form stops paying


def _dt(t: torch.dtype) -> int:
    if t == torch.bfloat16:
        return 0
    if t == torch.float32:
        return 1
    raise TypeError(f"activations must be bfloat16 or float32, not {t}")


def embed_sinpos(ids: torch.Tensor, pos: torch.Tensor, embed: torch.Tensor, base: float = 10000.0) -> torch.Tensor:
    """fp32 ``embed[ids] + sinusoid(pos)``: entry 2i = sin(p base^(-2i/W)), entry 2i+1 its cosine."""
    T, W = ids.shape[0], embed.shape[1]
    if use_hip(embed):
        x = torch.empty(T, W, dtype=torch.float32, device=embed.device)
        check(lib().k8s_embed_sinpos(ptr(ids), ptr(pos), ptr(embed), ptr(x), T, W, float(base), _dt(embed.dtype),
                                     stream_ptr(embed)), "embed_sinpos")
        return x
    i2 = (torch.arange(W, dtype=torch.float64) // 2) * 2
    ang = pos.double()[:, None] * torch.exp(-i2 / W * torch.log(torch.tensor(float(base), dtype=torch.float64)))[None]
    pe = torch.where((torch.arange(W) % 2 == 1)[None], ang.cos(), ang.sin()).float()
    return embed[ids.long()].float() + pe


def canon_conv(x: torch.Tensor, w: torch.Tensor, tail: torch.Tensor, seg: SegMeta, out_dtype) -> torch.Tensor:
    """``h = x + conv(x)``: per channel ``conv(x)_t = sum_j w[:, j] x_(t - taps + 1 + j)`` over each sequence
    (zeros before its start).  ``tail`` [slots, taps - 1, W] fp32 holds every sequence's last inputs and is
    advanced by this step's rows."""
    T, W = x.shape
    taps = w.shape[1]
    h = torch.empty(T, W, dtype=out_dtype, device=x.device)
    if use_hip(x):
        assert x.dtype == torch.float32 and x.is_contiguous() and w.is_contiguous() and tail.is_contiguous()
        assert tail.shape[1:] == (taps - 1, W) and w.dtype == out_dtype and taps <= 16
        check(lib().k8s_canon_conv(ptr(x), ptr(w), ptr(tail), ptr(seg.row_seg), ptr(seg.seg_row0), ptr(seg.seg_pos0),
                                   ptr(seg.seg_slot), ptr(h), T, seg.n_seg, W, taps, _dt(out_dtype), stream_ptr(x)),
              "canon_conv")
        return h
    wf = w.float()
    nt = taps - 1
    for s in range(seg.n_seg):
        a, b, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        prev = tail[sl] if p0 > 0 else torch.zeros(nt, W)
        ext = torch.cat([prev, x[a:b]])                     # inputs pos0 - nt .. pos0 + n - 1
        acc = x[a:b].clone()
        for j in range(taps):
            acc += wf[:, j] * ext[j:j + (b - a)]
        h[a:b] = acc.to(out_dtype)
        if nt:
            tail[sl] = ext[-nt:]
    return h


def mingru_scan(zug: torch.Tensor, bz: torch.Tensor, bu: torch.Tensor, state: torch.Tensor, seg: SegMeta,
                out_dtype) -> torch.Tensor:
    """minGRU over every segment: ``zug`` [T, 3C] fp32 = (z | u | g) projections without biases;
    ``S <- (1 - z) S + z cand`` with ``z = sigmoid(.)``, ``cand = u + 1/2`` for ``u >= 0`` else ``sigmoid(u)``;
    returns ``S * silu(g)``.  ``state`` [slots, C] fp32 is read (past position 0) and advanced."""
    T, C3 = zug.shape
    C = C3 // 3
    y = torch.empty(T, C, dtype=out_dtype, device=zug.device)
    if use_hip(zug):
        assert zug.dtype == torch.float32 and zug.is_contiguous() and state.is_contiguous() and bz.dtype == out_dtype
        chunks = seg.scan_chunks(SCAN_CHUNK)
        if chunks is not None:   # long prompt portions: parallel over time as well as channels
            ab = scratch(chunks.shape[0] * 2 * C, torch.float32, zug.device)
            s0 = scratch(seg.n_seg * C, torch.float32, zug.device)
            check(lib().k8s_mingru_chunked(ptr(zug), ptr(bz), ptr(bu), ptr(state), ptr(chunks), chunks.shape[0],
                                           ptr(seg.seg_row0), ptr(seg.seg_pos0), ptr(seg.seg_slot), ptr(ab), ptr(s0),
                                           ptr(y), C, _dt(out_dtype), stream_ptr(zug)), "mingru_chunked")
            return y
        check(lib().k8s_mingru_scan(ptr(zug), ptr(bz), ptr(bu), ptr(state), ptr(seg.seg_row0), ptr(seg.seg_pos0),
                                    ptr(seg.seg_slot), ptr(y), seg.n_seg, C, _dt(out_dtype), stream_ptr(zug)),
              "mingru_scan")
        return y
    z = torch.sigmoid(zug[:, :C] + bz.float())
    u = zug[:, C:2 * C] + bu.float()
    g = zug[:, 2 * C:]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    for s in range(seg.n_seg):
        a, b, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        S = state[sl].clone() if p0 > 0 else torch.zeros(C)
        for r in range(a, b):
            S = (1 - z[r]) * S + z[r] * cand[r]
            y[r] = (S * torch.nn.functional.silu(g[r])).to(out_dtype)
        state[sl] = S
    return y


def postnorm_(x: torch.Tensor, y: Optional[torch.Tensor], w: torch.Tensor, alpha: float, eps: float) -> torch.Tensor:
    """In place on the fp32 residual: ``x <- unit_rms(alpha x + y) * (1 + w)`` (``y`` None: no sublayer output)."""
    T, W = x.shape
    if use_hip(x):
        assert x.dtype == torch.float32 and x.is_contiguous()
        assert y is None or (y.is_contiguous() and y.shape == x.shape)
        check(lib().k8s_postnorm(ptr(x), ptr(y), 1 if y is None else _dt(y.dtype), ptr(w), _dt(w.dtype), None, T, W,
                                 float(alpha), float(eps), stream_ptr(x)), "postnorm")
        return x
    v = alpha * x + (y.float() if y is not None else 0.0)
    x.copy_(v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w.float()))
    return x


def unit_norm_out(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``unit_rms(x) * (1 + w)`` of fp32 rows as activations of ``w``'s type (``x`` is left as it is)."""
    T, W = x.shape
    out = torch.empty(T, W, dtype=w.dtype, device=x.device)
    if use_hip(x):
        assert x.dtype == torch.float32 and x.is_contiguous()
        check(lib().k8s_postnorm(ptr(x), None, 1, ptr(w), _dt(w.dtype), ptr(out), T, W, 1.0, float(eps),
                                 stream_ptr(x)), "unit_norm_out")
        return out
    out.copy_((x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w.float())).to(w.dtype))
    return out


def latent_norm(dn: torch.Tensor, wq: torch.Tensor, wkv: Optional[torch.Tensor], slots: torch.Tensor,
                cache: Optional[torch.Tensor], q_rank: int, kv_rank: int, eps: float, out_dtype,
                cache_t: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of the joint down projection ``dn`` [T, >= q_rank + kv_rank] fp32: the query latent is
    RMS-normed (plain weight) and returned; the key-value latent (``wkv`` given) is RMS-normed and
    written to the paged latent ``cache`` [pages, BS, kv_rank] at ``slots`` (page * BS + offset), and
    to its transposed twin ``cache_t`` [pages, kv_rank, BS] when given (the MFMA kernels' PV operand)."""
    T = dn.shape[0]
    cq = torch.empty(T, q_rank, dtype=out_dtype, device=dn.device)
    kr = kv_rank if wkv is not None else 0
    if use_hip(dn):
        assert dn.dtype == torch.float32 and dn.stride(1) == 1 and wq.dtype == out_dtype
        assert cache is None or (cache.is_contiguous() and cache.dtype == out_dtype and cache.shape[-1] == kv_rank)
        ct = cache_t if kr else None
        assert ct is None or (ct.is_contiguous() and ct.dtype == out_dtype and ct.shape[1] == kv_rank)
        check(lib().k8s_latent_norm(ptr(dn), dn.stride(0), ptr(wq), ptr(wkv), ptr(slots), ptr(cq), ptr(cache),
                                    ptr(ct), cache.shape[1] if kr else 1, T, q_rank, kr, float(eps),
                                    _dt(out_dtype), stream_ptr(dn)), "latent_norm")
        return cq
    q = dn[:, :q_rank]
    cq.copy_((q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * wq.float()).to(out_dtype))
    if kr:
        c = dn[:, q_rank:q_rank + kr]
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * wkv.float()
        ok = slots >= 0
        cache.view(-1, kr)[slots[ok].long()] = c[ok].to(cache.dtype)
        if cache_t is not None:
            BS = cache.shape[1]
            sl = slots[ok].long()
            cache_t[sl // BS, :, sl % BS] = c[ok].to(cache_t.dtype)
    return cq


def mfma_tiles(R: int, dtype, device) -> int:
    """Query tiles per wave the MFMA attention kernels run prompt portions with for latent rank ``R``
    (0: they do not take this rank or type -- the vector-pipe kernel runs instead)."""
    if dtype != torch.bfloat16 or torch.device(device).type != "cuda":
        return 0
    return int(lib().k8s_latent_attn_mfma_ok(int(R)))


def latent_attention_mfma(qa: torch.Tensor, cache: torch.Tensor, cache_t: torch.Tensor, gate: torch.Tensor,
                          seg: SegMeta, positions: torch.Tensor, scale: float) -> torch.Tensor:
    """:func:`latent_attention` on the matrix cores: bf16 absorbed queries ``qa`` [T, H, R], the latent
    pages and their transposed twins.  Decode rows (the step's first ``seg.n_single``) are split over
    partitions of ``DECODE_PART`` keys and merged; prompt portions run one wave per group of tokens."""
    T, H, R = qa.shape
    BS = cache.shape[1]
    tiles = mfma_tiles(R, qa.dtype, qa.device)
    assert tiles and qa.is_contiguous() and cache.is_contiguous() and cache_t.is_contiguous() and BS % 32 == 0
    assert gate.dtype == torch.float32 and gate.stride(1) == 1 and seg.block_tables.is_contiguous()
    out = torch.empty(T, H, R, dtype=torch.bfloat16, device=qa.device)
    tpi = tiles * (16 // min(H, 16))
    dec, pre, kmax = seg.attn_items(tpi)
    L, st = lib(), stream_ptr(qa)
    bt, maxb = seg.block_tables, seg.block_tables.shape[1]
    if dec.shape[0]:
        n_parts = -(-kmax // DECODE_PART)
        nd = seg.n_single
        part_o = scratch(nd * H * n_parts * R, torch.float32, qa.device)
        part_ml = scratch(nd * H * n_parts * 2, torch.float32, qa.device)
        check(L.k8s_latent_attn_mfma(ptr(qa), ptr(cache), ptr(cache_t), ptr(bt), maxb, ptr(dec), dec.shape[0],
                                     ptr(gate), gate.stride(0), ptr(out), ptr(part_o), ptr(part_ml), n_parts,
                                     DECODE_PART, ptr(positions), nd, H, R, BS, float(scale), 1, 1, st),
              "latent_attn_mfma (decode)")
    if pre.shape[0]:
        check(L.k8s_latent_attn_mfma(ptr(qa), ptr(cache), ptr(cache_t), ptr(bt), maxb, ptr(pre), pre.shape[0],
                                     ptr(gate), gate.stride(0), ptr(out), None, None, 1, DECODE_PART, None, 0,
                                     H, R, BS, float(scale), 0, tiles, st), "latent_attn_mfma (prefill)")
    return out


def latent_attention(qa: torch.Tensor, cache: torch.Tensor, gate: torch.Tensor, seg: SegMeta, scale: float,
                     out_dtype) -> torch.Tensor:
    """Causal attention of absorbed queries ``qa`` [T, H, R] fp32 over the paged latents ``cache``
    [pages, BS, R]: ``p = softmax(scale * qa . c_j)`` over the keys up to the row's own position,
    output ``sigmoid(gate[t, h]) * sum_j p_j c_j`` [T, H, R] (``gate`` fp32, row stride free)."""
    T, H, R = qa.shape
    BS = cache.shape[1]
    out = torch.empty(T, H, R, dtype=out_dtype, device=qa.device)
    if use_hip(qa):
        assert qa.dtype == torch.float32 and qa.is_contiguous() and cache.is_contiguous() and cache.dtype == out_dtype
        assert gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.shape[1] >= H
        assert seg.block_tables.is_contiguous()
        check(lib().k8s_latent_attn_rows(ptr(qa), ptr(cache), ptr(seg.block_tables), seg.block_tables.shape[1],
                                         ptr(seg.row_seg), ptr(seg.seg_row0), ptr(seg.seg_pos0), ptr(gate),
                                         gate.stride(0), ptr(out), 0, T, H, R, BS, float(scale), _dt(out_dtype),
                                         stream_ptr(qa)), "latent_attn_rows")
        return out
    flat = cache.view(-1, R)
    for s in range(seg.n_seg):
        a, b, p0 = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s]
        n_ctx = p0 + b - a
        pages = seg.block_tables[s].long()
        kp = torch.arange(n_ctx)
        c = flat[pages[kp // BS] * BS + kp % BS].float()                      # [ctx, R]
        sc = torch.einsum("thr,jr->thj", qa[a:b], c) * scale
        vis = kp[None, :] <= (p0 + torch.arange(b - a))[:, None]
        sc = sc.masked_fill(~vis[:, None, :], float("-inf"))
        o = torch.einsum("thj,jr->thr", torch.softmax(sc, -1), c)
        out[a:b] = (o * torch.sigmoid(gate[a:b, :H])[:, :, None]).to(out_dtype)
    return out


# ------------------------------------------------------------------ recurrent mixers and window attention
# (csrc/kernels/mixer_ops.hip, window_attn.hip).  Small parameters (convolution taps, biases, decays,
# A, D, the distance bias and the head-mixing matrix) are fp32 tensors.
@dataclass
class SegStepInputs:
    """One step in the segment layout (:class:`SegMeta`)."""
    input_ids: torch.Tensor        # [T] int32
    positions: torch.Tensor        # [T] int32
    slots: torch.Tensor            # [T] int32 cache slot (page * BS + offset) of every row
    seg: SegMeta
    logits_idx: torch.Tensor       # [n] int64 rows whose logits are needed


def short_conv(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], tail: torch.Tensor, seg: SegMeta,
               act: bool = True) -> torch.Tensor:
    """Causal per-channel convolution with bias and SiLU: ``out_t = act(b + sum_j w[:, j] x_(t - taps + 1 + j))``
    over each sequence (the last column of ``w`` [C, taps] is the current token's; zeros before the
    start).  ``x`` [T, C] may be a column slice of a wider matrix.  ``tail`` [slots, taps - 1, C] fp32
    holds every sequence's last inputs and is advanced by this step's rows."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.empty(T, C, dtype=x.dtype, device=x.device)
    if use_hip(x):
        assert x.stride(1) == 1 and w.dtype == torch.float32 and w.is_contiguous() and tail.is_contiguous()
        assert tail.shape[1:] == (taps - 1, C) and 1 <= taps <= 16 and (b is None or b.dtype == torch.float32)
        d = _dt(x.dtype)
        items = seg.tile_items(WINDOW_TILE)      # rows in tiles of one segment: metadata once per tile
        check(lib().k8s_short_conv(ptr(x), x.stride(0), d, ptr(w), ptr(b), ptr(tail), ptr(seg.row_seg),
                                   ptr(seg.seg_row0), ptr(seg.seg_pos0), ptr(seg.seg_slot), ptr(out), T, seg.n_seg, C,
                                   taps, int(act), d, stream_ptr(x), ptr(items), items.shape[0]), "short_conv")
        return out
    nt = taps - 1
    xf = x.float()
    for s in range(seg.n_seg):
        a, e, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        prev = tail[sl] if p0 > 0 else torch.zeros(nt, C)
        ext = torch.cat([prev, xf[a:e]])
        acc = torch.zeros(e - a, C) if b is None else b.expand(e - a, C).clone()
        for j in range(taps):
            acc += w[:, j] * ext[j:j + (e - a)]
        out[a:e] = (torch.nn.functional.silu(acc) if act else acc).to(x.dtype)
        if nt:
            tail[sl] = ext[-nt:]
    return out


def selective_scan(xc: torch.Tensor, dtp: torch.Tensor, dt_bias: torch.Tensor, dbc: torch.Tensor, R: int,
                   A: torch.Tensor, D: torch.Tensor, z: torch.Tensor, state: torch.Tensor, seg: SegMeta) -> torch.Tensor:
    """Diagonal selective state-space recurrence per channel c and state n, fp32:
    ``dt = softplus(dtp + dt_bias)``; ``S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n``;
    ``y_c = (sum_n S[c, n] C_n + D_c x_c) * silu(z_c)``.  ``dbc`` [T, >= R + 2N] fp32 holds B at column R
    and C at column R + N; ``dtp`` [T, C] fp32; ``xc`` [T, C] and ``z`` (a column slice) activations.
    ``state`` [slots, C, N] fp32 is read (past position 0) and advanced."""
    T, C = xc.shape
    N = A.shape[1]
    y = torch.empty(T, C, dtype=xc.dtype, device=xc.device)
    if use_hip(xc):
        assert xc.is_contiguous() and dtp.dtype == torch.float32 and dtp.is_contiguous() and dtp.shape == (T, C)
        assert dbc.dtype == torch.float32 and dbc.stride(1) == 1 and dbc.shape[1] >= R + 2 * N
        assert z.stride(1) == 1 and z.dtype == xc.dtype and state.is_contiguous() and state.shape[1:] == (C, N)
        assert A.dtype == D.dtype == dt_bias.dtype == torch.float32 and A.is_contiguous()
        # long portions: chunks run in parallel (a pass from zero states, a carry over the chunks, the
        # chunks again from their start states); short ones token by token
        # (with many sequences the token-by-token kernel already fills the chip, at half the exponentials)
        cr = seg.chunk_ranges(SSM_CHUNK, 2 * SSM_CHUNK) if seg.n_seg * C < SEQ_FILL_LANES else None
        chunks, c0, cs, csd, nch = None, None, None, None, 0
        if cr is not None:
            chunks, c0 = cr
            nch = chunks.shape[0]
            cs = scratch(nch * C * N, torch.float32, xc.device)
            csd = scratch(nch * C, torch.float32, xc.device)
        check(lib().k8s_selective_scan(ptr(xc), _dt(xc.dtype), ptr(dtp), ptr(dt_bias), ptr(dbc), dbc.stride(0), R,
                                       ptr(A), ptr(D), ptr(z), z.stride(0), ptr(state), ptr(seg.seg_row0),
                                       ptr(seg.seg_pos0), ptr(seg.seg_slot), ptr(y), seg.n_seg, C, N, T,
                                       stream_ptr(xc), ptr(chunks), nch, ptr(c0), ptr(cs), ptr(csd)), "selective_scan")
        return y
    dt = torch.nn.functional.softplus(dtp + dt_bias)
    xf, zf = xc.float(), z.float()
    Bm, Cm = dbc[:, R:R + N], dbc[:, R + N:R + 2 * N]
    for s in range(seg.n_seg):
        a, e, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        S = state[sl].clone() if p0 > 0 else torch.zeros(C, N)
        for r in range(a, e):
            S = torch.exp(dt[r][:, None] * A) * S + (dt[r] * xf[r])[:, None] * Bm[r][None, :]
            y[r] = ((S @ Cm[r] + D * xf[r]) * torch.nn.functional.silu(zf[r])).to(xc.dtype)
        state[sl] = S
    return y


def ssd_scan(x: torch.Tensor, bc: torch.Tensor, dtp: torch.Tensor, dt_bias: torch.Tensor, rate: torch.Tensor,
             D: torch.Tensor, z: torch.Tensor, H: int, P: int, G: int, N: int, state: torch.Tensor, seg: SegMeta,
             fast_exp: bool = False) -> torch.Tensor:
    """State-space recurrence with one decay per head and token (state-space duality), fp32.  Head h of ``H`` owns
    the channels ``h P .. h P + P - 1`` of ``x`` [T, H P] and reads B / C group ``h // (H // G)`` of ``bc`` [T, 2 G N]
    = (B [G, N] | C [G, N]):  ``dt = softplus(dtp[:, h] + dt_bias[h])``;  ``S <- exp(-rate[h] dt) S + dt B x^T``
    (``S`` [N, P] per head);  ``y = (S^T C + D[h] x) * silu(z)``.  ``x``, ``bc``, ``z`` are activations of one type and
    may be column slices; ``dtp`` [T, H] fp32 (row stride free).  ``state`` [slots, H P, N] fp32 is read (past
    position 0) and advanced.  Returns y [T, H P] fp32.  ``fast_exp``: the hardware exponentials (relative error
    about 1e-6) instead of ``expf`` / ``log1pf``."""
    T, C = x.shape
    y = torch.empty(T, C, dtype=torch.float32, device=x.device)
    if use_hip(x):
        assert C == H * P and H % G == 0 and 1 <= N <= 128 and bc.shape[1] == 2 * G * N
        assert x.stride(1) == bc.stride(1) == z.stride(1) == dtp.stride(1) == 1 and x.dtype == bc.dtype == z.dtype
        assert dtp.dtype == torch.float32 and dtp.shape[1] == H and z.shape[1] == C
        assert dt_bias.dtype == rate.dtype == D.dtype == torch.float32 and dt_bias.numel() == rate.numel() == D.numel() == H
        assert state.is_contiguous() and state.shape[1:] == (C, N)
        # long portions: chunks in parallel (end states from zero + the sum of step sizes, a carry over the
        # chunks, the chunks again from their start states); short ones, and steps whose sequences x channels
        # already fill the chip, token by token
        cr = seg.chunk_ranges(SSM_CHUNK, 2 * SSM_CHUNK) if seg.n_seg * C < SEQ_FILL_LANES else None
        chunks, c0, cs, csd, nch = None, None, None, None, 0
        if cr is not None:
            chunks, c0 = cr
            nch = chunks.shape[0]
            cs = scratch(nch * C * N, torch.float32, x.device)
            csd = scratch(nch * C, torch.float32, x.device)
        check(lib().k8s_ssd_scan(ptr(x), x.stride(0), ptr(bc), bc.stride(0), _dt(x.dtype), ptr(dtp), dtp.stride(0),
                                 ptr(dt_bias), ptr(rate), ptr(D), ptr(z), z.stride(0), ptr(state), ptr(seg.seg_row0),
                                 ptr(seg.seg_pos0), ptr(seg.seg_slot), ptr(y), seg.n_seg, H, P, G, N, T,
                                 int(fast_exp), stream_ptr(x), ptr(chunks), nch, ptr(c0), ptr(cs), ptr(csd)),
              "ssd_scan")
        return y
    dt = torch.nn.functional.softplus(dtp.float() + dt_bias)                 # [T, H]
    dec = torch.exp(-rate * dt)
    xf, zf = x.float().view(T, H, P), z.float()
    rep = H // G
    Bm = bc[:, :G * N].float().view(T, G, N).repeat_interleave(rep, 1)      # [T, H, N]
    Cm = bc[:, G * N:].float().view(T, G, N).repeat_interleave(rep, 1)
    for s in range(seg.n_seg):
        a, e, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        S = state[sl].view(H, P, N).clone() if p0 > 0 else torch.zeros(H, P, N)
        for r in range(a, e):
            S = dec[r][:, None, None] * S + (dt[r][:, None] * xf[r])[:, :, None] * Bm[r][:, None, :]
            o = torch.einsum("hpn,hn->hp", S, Cm[r]) + D[:, None] * xf[r]
            y[r] = o.reshape(-1) * torch.nn.functional.silu(zf[r])
        state[sl] = S.reshape(C, N)
    return y


def retention(qkvg: torch.Tensor, H: int, D: int, V: int, decay: torch.Tensor, rot_dims: int, rot_base: float,
              state: torch.Tensor, seg: SegMeta, positions: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """Retention per head, fp32: rows of ``qkvg`` [T, 2HD + 2HV] fp32 = (q | k | v | g).  q and k are
    rotated on their first ``rot_dims`` entries (entry i paired with i + rot_dims / 2, angle
    ``pos * rot_base^(-2i / rot_dims)``), k is scaled by ``D^(-1/2)``; ``S <- decay_h S + k v^T``;
    ``o = S^T q``; the result is ``o / rms(o) * silu(g)`` [T, H * V].  ``state`` [slots, H, D, V] fp32.
    On the device q and k are rotated IN PLACE in ``qkvg``."""
    T = qkvg.shape[0]
    out = torch.empty(T, H * V, dtype=out_dtype, device=qkvg.device)
    if use_hip(qkvg):
        assert qkvg.dtype == torch.float32 and qkvg.stride(1) == 1 and qkvg.shape[1] == 2 * H * (D + V)
        assert state.is_contiguous() and state.shape[1:] == (H, D, V) and decay.dtype == torch.float32
        oraw = scratch(T * H * V, torch.float32, qkvg.device)
        # long portions: chunks in parallel (end states from zero, a carry over the chunks, the chunks
        # again from their start states); short ones token by token
        cr = seg.chunk_ranges(SSM_CHUNK, 2 * SSM_CHUNK) if seg.n_seg * H * V * 8 < SEQ_FILL_LANES else None
        chunks, c0, cs, nch = None, None, None, 0
        if cr is not None:
            chunks, c0 = cr
            nch = chunks.shape[0]
            cs = scratch(nch * H * D * V, torch.float32, qkvg.device)
        check(lib().k8s_retention(ptr(qkvg), qkvg.stride(0), ptr(positions), ptr(decay), ptr(state), ptr(seg.seg_row0),
                                  ptr(seg.seg_pos0), ptr(seg.seg_slot), ptr(out), seg.n_seg, H, D, V, rot_dims,
                                  float(rot_base), float(eps), _dt(out_dtype), stream_ptr(qkvg), T, ptr(oraw),
                                  ptr(chunks), nch, ptr(c0), ptr(cs)), "retention")
        return out
    half = rot_dims // 2
    f = torch.exp(-(2.0 * torch.arange(half, dtype=torch.float64) / max(rot_dims, 1)) * math.log(rot_base))
    ang = positions.double()[:, None] * f[None]
    co, si = ang.cos().float()[:, None, :], ang.sin().float()[:, None, :]

    def rot(x):
        u, v = x[..., :half], x[..., half:rot_dims]
        return torch.cat([u * co - v * si, v * co + u * si, x[..., rot_dims:]], -1)

    q = rot(qkvg[:, :H * D].view(T, H, D))
    k = rot(qkvg[:, H * D:2 * H * D].view(T, H, D)) * D ** -0.5
    v = qkvg[:, 2 * H * D:2 * H * D + H * V].view(T, H, V)
    g = qkvg[:, 2 * H * D + H * V:].view(T, H, V)
    for s in range(seg.n_seg):
        a, e, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        S = state[sl].clone() if p0 > 0 else torch.zeros(H, D, V)
        for r in range(a, e):
            S = decay[:, None, None] * S + k[r][:, :, None] * v[r][:, None, :]
            o = torch.einsum("hdv,hd->hv", S, q[r])
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * torch.nn.functional.silu(g[r])
            out[r] = o.reshape(-1).to(out_dtype)
        state[sl] = S
    return out


def window_mfma_ok(H: int, G: int, D: int, V: int, dtype, device) -> bool:
    """Whether the matrix-core window attention kernel takes these sizes (bf16 on the device only;
    the vector-pipe kernel runs everything else)."""
    if dtype != torch.bfloat16 or torch.device(device).type != "cuda":
        return False
    return bool(lib().k8s_window_attn_mfma_ok(int(H), int(G), int(D), int(V)))


WINDOW_TILE = 16    # query tokens per work item of the matrix-core window attention kernel
WINDOW_PART = 128   # keys per part when a step of few rows is split over the keys too
WINDOW_SPLIT_ITEMS = 32


def window_kv_write(qkv: torch.Tensor, k_off: int, kc: torch.Tensor, vc: torch.Tensor, slots: torch.Tensor,
                    vt: Optional[torch.Tensor] = None) -> None:
    """The key and value columns of the joint projection's rows (k at ``k_off``, v behind it) go to the
    pages ``kc`` [pages, BS, G D] / ``vc`` [pages, BS, G V] at ``slots`` (page * BS + offset), the values
    also to the transposed twin ``vt`` [pages, G V, BS] when given (the matrix-core kernel's PV operand)."""
    T = qkv.shape[0]
    nk, nv = kc.shape[-1], vc.shape[-1]
    BS = kc.shape[1]
    if use_hip(qkv):
        assert qkv.stride(1) == 1 and kc.is_contiguous() and vc.is_contiguous() and kc.dtype == vc.dtype == qkv.dtype
        assert qkv.shape[1] >= k_off + nk + nv
        assert vt is None or (vt.is_contiguous() and vt.dtype == qkv.dtype and vt.shape[1:] == (nv, BS))
        check(lib().k8s_window_kv_write(ptr(qkv), qkv.stride(0), k_off, nk, nv, ptr(slots), ptr(kc), ptr(vc), T,
                                        _dt(qkv.dtype), stream_ptr(qkv), ptr(vt), BS), "window_kv_write")
        return
    ok = slots >= 0
    sl = slots[ok].long()
    kc.view(-1, nk)[sl] = qkv[ok, k_off:k_off + nk]
    vc.view(-1, nv)[sl] = qkv[ok, k_off + nk:k_off + nk + nv]
    if vt is not None:
        vt[sl // BS, :, sl % BS] = qkv[ok, k_off + nk:k_off + nk + nv]


def window_attention(qkv: torch.Tensor, H: int, G: int, D: int, V: int, kc: torch.Tensor, vc: torch.Tensor,
                     r1: torch.Tensor, r2: torch.Tensor, talk: torch.Tensor, window: int, scale: float,
                     seg: SegMeta, vt: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Sliding-window attention of the rows' queries (the first H D columns of ``qkv``) over the paged
    keys and values, which already hold this step's rows: position i sees j with ``0 <= i - j < window``;
    ``s = scale q.k - r1[h] ln(1 + r2[h] (i - j))``; ``p_j = exp(s_j) / (1 + sum exp(s))`` (a sink of score 0
    without a value); the heads' weights are mixed, ``w_h = sum_g talk[h, g] p_g``, and head h applies
    its mixed weights to the values of key / value head ``h // (H // G)``.  Returns [T, H V].
    With the transposed value pages ``vt`` (bf16, sizes of :func:`window_mfma_ok`) the matrix-core
    kernel runs: tiles of ``WINDOW_TILE`` tokens, the weights rounded to bf16 for the value product."""
    T = qkv.shape[0]
    BS = kc.shape[1]
    out = torch.empty(T, H * V, dtype=qkv.dtype, device=qkv.device)
    if use_hip(qkv):
        assert qkv.stride(1) == 1 and kc.is_contiguous() and vc.is_contiguous() and kc.dtype == vc.dtype == qkv.dtype
        assert kc.shape[-1] == G * D and vc.shape[-1] == G * V and seg.block_tables.is_contiguous()
        assert r1.dtype == r2.dtype == talk.dtype == torch.float32 and talk.is_contiguous() and H % G == 0
        if vt is not None and window_mfma_ok(H, G, D, V, qkv.dtype, qkv.device) and qkv.stride(0) % 8 == 0:
            assert vt.is_contiguous() and vt.shape[1:] == (G * V, BS) and BS % 32 == 0
            items = seg.tile_items(WINDOW_TILE)
            n_items = items.shape[0]
            # steps of few rows (decoding): the keys are split over workgroups as well -- parts of
            # WINDOW_PART keys counted from each tile's first key block, merged in part order
            n_parts, pml, po = 1, None, None
            if n_items <= WINDOW_SPLIT_ITEMS:
                kmax = max(p + b - a for p, a, b in zip(seg.pos0_host, seg.row0_host[:-1], seg.row0_host[1:]))
                span = min(int(window) + WINDOW_TILE + 30, -(-kmax // 32) * 32)
                n_parts = -(-span // WINDOW_PART)
                if n_parts > 1:
                    pml = scratch(n_items * n_parts * H * 32, torch.float32, qkv.device)
                    po = scratch(n_items * n_parts * 16 * H * V, torch.float32, qkv.device)
            check(lib().k8s_window_attn_mfma(ptr(qkv), qkv.stride(0), ptr(kc), ptr(vt), ptr(seg.block_tables),
                                             seg.block_tables.shape[1], ptr(items), n_items, ptr(r1), ptr(r2),
                                             ptr(talk), ptr(out), H, G, D, V, BS, int(window), float(scale),
                                             stream_ptr(qkv), WINDOW_PART, n_parts, ptr(pml), ptr(po)),
                  "window_attn_mfma")
            return out
        check(lib().k8s_window_attn_rows(ptr(qkv), qkv.stride(0), ptr(kc), ptr(vc), ptr(seg.block_tables),
                                         seg.block_tables.shape[1], ptr(seg.row_seg), ptr(seg.seg_row0),
                                         ptr(seg.seg_pos0), ptr(r1), ptr(r2), ptr(talk), ptr(out), T, H, G, D, V, BS,
                                         int(window), float(scale), _dt(qkv.dtype), stream_ptr(qkv)),
              "window_attn_rows")
        return out
    kf, vf = kc.view(-1, G, D), vc.view(-1, G, V)
    rep = H // G
    for s in range(seg.n_seg):
        a, e, p0 = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s]
        n, n_ctx = e - a, p0 + e - a
        lo = max(0, p0 - window + 1)
        kp = torch.arange(lo, n_ctx)
        rows = seg.block_tables[s].long()[kp // BS] * BS + kp % BS
        k = kf[rows].float().repeat_interleave(rep, 1)             # [ctx, H, D]
        v = vf[rows].float().repeat_interleave(rep, 1)             # [ctx, H, V]
        q = qkv[a:e, :H * D].float().view(n, H, D)
        dist = (p0 + torch.arange(n))[:, None] - kp[None, :]       # [n, ctx]
        sc = torch.einsum("thd,jhd->thj", q, k) * scale
        sc = sc - r1[None, :, None] * torch.log1p(r2[None, :, None] * dist.clamp_min(0).float()[:, None, :])
        vis = (dist >= 0) & (dist < window)
        sc = sc.masked_fill(~vis[:, None, :], float("-inf"))
        m = sc.amax(-1, keepdim=True).clamp_min(0.0)
        ex = torch.exp(sc - m)
        p = ex / (torch.exp(-m) + ex.sum(-1, keepdim=True))
        pm = torch.einsum("hg,tgj->thj", talk, p)
        out[a:e] = torch.einsum("thj,jhv->thv", pm, v).reshape(n, H * V).to(qkv.dtype)
    return out


# ------------------------------------------------------------------ masked softmax attention with a prepared q / k,
# and matrix-state recurrences (csrc/kernels/masked_attn.hip, matrix_mem.hip)
def attn_prep(qkv: torch.Tensor, bias: Optional[torch.Tensor], H: int, G: int, D: int, V: int,
              positions: torch.Tensor, slots: torch.Tensor, kc: Optional[torch.Tensor], vc: Optional[torch.Tensor],
              out_dtype, norm=False, q_w: Optional[torch.Tensor] = None, k_w: Optional[torch.Tensor] = None,
              eps: float = 0.0, rot_dims: int = 0, rot_base: float = 10000.0, lam: float = 0.0,
              v_other: Optional[torch.Tensor] = None, v_keep: Optional[torch.Tensor] = None,
              vt: Optional[torch.Tensor] = None, maps: int = 1, v_is_k: bool = False,
              q_temp: Optional[Tuple[float, int]] = None) -> torch.Tensor:
    """Between the joint projection and attention, one pass over the fp32 rows of ``qkv`` [T, H M D + G M D + G V]
    = (q | k | v) with ``M = maps`` score maps per head (q and k laid out [head][map][D]):  add ``bias`` (fp32, same
    width, optional);  rotate q and k on their first ``rot_dims`` entries per head (entry i paired with
    i + rot_dims / 2, angle ``pos * rot_base^(-2 i / rot_dims)``);  with ``norm`` (True or "head") divide every q and k
    head by its root mean square (``eps`` inside the root) and multiply by ``q_w`` / ``k_w`` [D] where given -- behind
    the rotation;  with ``norm="all"`` divide q, and k, by the root mean square of the WHOLE projection and multiply by
    ``q_w`` [H M D] / ``k_w`` [G M D] -- in front of the rotation;  with ``q_temp = (coef, every)`` multiply q by
    ``1 + coef ln(floor((pos + 1) / every) + 1)``;  ``v_keep`` [T, G V] fp32 receives the values as projected;  with
    ``v_other`` the values become ``(1 - lam) v + lam v_other``.  ``v_is_k``: there are no value columns, the values
    are the keys as projected (before norm and rotation; V = M D).  k and v go to the pages ``kc`` [pages, BS, G M D] /
    ``vc`` [pages, BS, G V] at ``slots`` (and v to the transposed twin ``vt`` when given); q is returned [T, H M D] as
    activations.  ``G = 0``: only queries (a layer that reads another layer's pages)."""
    T = qkv.shape[0]
    HQ, GK = H * maps, G * maps
    NQ, NK, NV = HQ * D, GK * D, G * V
    mode = {False: 0, None: 0, True: 1, "head": 1, "all": 2}[norm]
    v_col = NQ if v_is_k else NQ + NK
    assert not v_is_k or NV == NK
    q_out = torch.empty(T, NQ, dtype=out_dtype, device=qkv.device)
    BS = kc.shape[1] if kc is not None else 1
    tq_coef, tq_every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 0)
    if use_hip(qkv):
        assert qkv.dtype == torch.float32 and qkv.stride(1) == 1 and qkv.shape[1] == v_col + NV
        if G:
            assert kc.is_contiguous() and vc.is_contiguous() and kc.dtype == vc.dtype == out_dtype
            assert kc.shape[-1] == NK and vc.shape[-1] == NV
        assert rot_dims % 2 == 0 and 0 <= rot_dims <= D
        for t, n in ((bias, v_col + NV), (q_w, NQ if mode == 2 else D), (k_w, NK if mode == 2 else D)):
            assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n)
        for t in (v_other, v_keep):
            assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.shape == (T, NV))
        assert vt is None or (vt.is_contiguous() and vt.dtype == out_dtype and vt.shape[1:] == (NV, BS))
        check(lib().k8s_attn_prep(ptr(qkv), qkv.stride(0), ptr(bias), HQ, GK, D, NV, ptr(positions), ptr(slots),
                                  ptr(kc), ptr(vc), ptr(vt), BS, ptr(q_out), _dt(out_dtype), mode, ptr(q_w),
                                  ptr(k_w), float(eps), int(rot_dims), float(rot_base), float(lam), ptr(v_other),
                                  ptr(v_keep), T, stream_ptr(qkv), v_col, tq_coef, tq_every), "attn_prep")
        return q_out
    x = qkv + bias if bias is not None else qkv
    q, k, v = x[:, :NQ], x[:, NQ:NQ + NK], x[:, v_col:v_col + NV]
    if mode == 2:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * (q_w if q_w is not None else 1.0)
        if NK:
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * (k_w if k_w is not None else 1.0)
    q, k = q.reshape(T, HQ, D), k.reshape(T, GK, D)
    if rot_dims:
        half = rot_dims // 2
        f = torch.exp(-(2.0 * torch.arange(half, dtype=torch.float64) / rot_dims) * math.log(rot_base))
        ang = positions.double()[:, None] * f[None]
        co, si = ang.cos().float()[:, None, :], ang.sin().float()[:, None, :]

        def rot(z):
            a, b = z[..., :half], z[..., half:rot_dims]
            return torch.cat([a * co - b * si, b * co + a * si, z[..., rot_dims:]], -1)

        q, k = rot(q), rot(k)
    if mode == 1:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
        if q_w is not None:
            q = q * q_w
        if k_w is not None:
            k = k * k_w
    if tq_every:
        temp = 1.0 + tq_coef * torch.log(torch.div(positions + 1, tq_every, rounding_mode="floor").float() + 1.0)
        q = q * temp[:, None, None]
    if v_keep is not None:
        v_keep.copy_(v)
    if v_other is not None:
        v = (1.0 - lam) * v + lam * v_other
    if G:
        ok = slots >= 0
        sl = slots[ok].long()
        kc.view(-1, NK)[sl] = k.reshape(T, NK)[ok].to(kc.dtype)
        vc.view(-1, NV)[sl] = v[ok].to(vc.dtype)
        if vt is not None:
            vt[sl // BS, :, sl % BS] = v[ok].to(vt.dtype)
    q_out.copy_(q.reshape(T, NQ).to(out_dtype))
    return q_out


def masked_attention(q: torch.Tensor, H: int, G: int, D: int, V: int, kc: torch.Tensor, vc: torch.Tensor,
                     seg: SegMeta, scale: float, softcap: float = 0.0, chunk: int = 0, window: int = 0,
                     keep_first: int = 0, sink: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                     vt: Optional[torch.Tensor] = None, maps: int = 1, out_f32: bool = False) -> torch.Tensor:
    """Softmax attention of the rows' queries ``q`` [T, H D] over the paged keys and values (which already
    hold this step's rows), query head h reading key / value head ``h // (H // G)``.  Position i sees j <= i
    with, for ``chunk`` > 0, ``i // chunk == j // chunk`` and, for ``window`` > 0, ``i - j < window or j < keep_first``
    (positions count from the sequence's start).  ``s = scale q.k``, then ``softcap * tanh(s / softcap)`` for
    ``softcap`` > 0.  ``sink`` [H] fp32 adds ``exp(sink_h)`` to head h's denominator (no key, no value).  ``gate``
    [T, >= H] fp32 (row stride free): head h's output is multiplied by ``sigmoid(gate[t, h])``.
    Returns [T, H V].  With the transposed value pages ``vt`` (bf16, sizes of :func:`masked_mfma_ok`) the
    matrix-core kernel runs.
    ``maps`` = M > 1: every head has M score maps -- ``q`` is [T, H M D] and the key pages [.., G M D], both laid out
    [head][map][D]; map m of head h scores against key head ``(h // (H // G)) M + m``, has a softmax of its own and
    applies it to value head ``h // (H // G)``; the result is [T, H M V], every map's by itself (``sink`` and ``gate``
    then count H M).  ``out_f32``: the result in fp32 whatever the activation type."""
    T = q.shape[0]
    BS = kc.shape[1]
    HQ = H * maps
    out = torch.empty(T, HQ * V, dtype=torch.float32 if out_f32 else q.dtype, device=q.device)
    if use_hip(q):
        assert q.is_contiguous() and q.shape[1] == HQ * D and kc.is_contiguous() and vc.is_contiguous()
        assert kc.dtype == vc.dtype == q.dtype and kc.shape[-1] == G * maps * D and vc.shape[-1] == G * V and H % G == 0
        assert seg.block_tables.is_contiguous() and chunk >= 0 and window >= 0 and keep_first >= 0
        assert sink is None or (sink.dtype == torch.float32 and sink.shape[0] == HQ)
        assert gate is None or (gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.shape[1] >= HQ)
        gs = gate.stride(0) if gate is not None else 0
        if vt is not None and masked_mfma_ok(H, G, D, V, q.dtype, q.device):
            assert vt.is_contiguous() and vt.shape[1:] == (G * V, BS) and BS % 32 == 0
            items = seg.tile_items(WINDOW_TILE)
            n_items = items.shape[0]
            # steps of few rows (decoding): a tile's key blocks are split over workgroups as well -- parts of
            # MASK_PART_BLOCKS blocks of the tile's own block list (at most MASK_MAX_PARTS parts), then a merge
            n_parts, pb, pml, po = 1, MASK_PART_BLOCKS, None, None
            if n_items <= WINDOW_SPLIT_ITEMS:
                kmax = max(p + b - a for p, a, b in zip(seg.pos0_host, seg.row0_host[:-1], seg.row0_host[1:]))
                nblk = -(-kmax // 32) + 1                  # an upper bound of any tile's blocks
                if window > 0:     # a tile's span: the window, its 16 tokens, a block's alignment; + the kept blocks
                    nblk = min(nblk, (int(window) + 45) // 32 + 1 + -(-int(keep_first) // 32))
                if chunk > 0:
                    nblk = min(nblk, (int(chunk) + 45) // 32 + 1)
                pb = max(MASK_PART_BLOCKS, -(-nblk // MASK_MAX_PARTS))
                n_parts = -(-nblk // pb)
                if n_parts > 1:
                    pml = scratch(n_items * n_parts * HQ * 32, torch.float32, q.device)
                    po = scratch(n_items * n_parts * 16 * HQ * V, torch.float32, q.device)
            check(lib().k8s_masked_attn_mfma(ptr(q), ptr(kc), ptr(vt), ptr(seg.block_tables),
                                             seg.block_tables.shape[1], ptr(items), n_items, ptr(sink),
                                             ptr(gate), gs, ptr(out), H, G, D, V, BS, int(chunk), int(window),
                                             int(keep_first), float(scale), float(softcap), stream_ptr(q), pb, n_parts,
                                             ptr(pml), ptr(po), int(maps), int(out_f32)), "masked_attn_mfma")
            return out
        check(lib().k8s_masked_attn_rows(ptr(q), ptr(kc), ptr(vc), ptr(seg.block_tables), seg.block_tables.shape[1],
                                         ptr(seg.row_seg), ptr(seg.seg_row0), ptr(seg.seg_pos0), ptr(sink), ptr(gate),
                                         gs, ptr(out), T, H, G, D, V, BS, int(chunk), int(window), int(keep_first),
                                         float(scale), float(softcap), _dt(q.dtype), stream_ptr(q), int(maps),
                                         int(out_f32)), "masked_attn_rows")
        return out
    kf, vf = kc.view(-1, G, maps, D), vc.view(-1, G, V)
    rep = H // G
    for s in range(seg.n_seg):
        a, e, p0 = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s]
        n, n_ctx = e - a, p0 + e - a
        kp = torch.arange(n_ctx)
        rows = seg.block_tables[s].long()[kp // BS] * BS + kp % BS
        k = kf[rows].float().repeat_interleave(rep, 1).reshape(n_ctx, HQ, D)                  # [ctx, H M, D]
        v = vf[rows].float().repeat_interleave(rep, 1).repeat_interleave(maps, 1)             # [ctx, H M, V]
        qi = (p0 + torch.arange(n))[:, None]
        vis = kp[None, :] <= qi
        if chunk > 0:
            vis &= (qi // chunk) == (kp[None, :] // chunk)
        if window > 0:
            vis &= ((qi - kp[None, :]) < window) | (kp[None, :] < keep_first)
        sc = torch.einsum("thd,jhd->thj", q[a:e].float().view(n, HQ, D), k) * scale
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        sc = sc.masked_fill(~vis[:, None, :], float("-inf"))
        m = sc.amax(-1, keepdim=True)
        if sink is not None:
            m = torch.maximum(m, sink[None, :, None])
        ex = torch.exp(sc - m)
        den = ex.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[None, :, None] - m)
        o = torch.einsum("thj,jhv->thv", ex / den, v)
        if gate is not None:
            o = o * torch.sigmoid(gate[a:e, :HQ])[:, :, None]
        out[a:e] = o.reshape(n, HQ * V).to(out.dtype)
    return out


MASK_PART_BLOCKS = 4    # 32-key blocks per part when a step of few rows is split over the keys too
MASK_MAX_PARTS = 32


def masked_mfma_ok(H: int, G: int, D: int, V: int, dtype, device) -> bool:
    """Whether the matrix-core form of :func:`masked_attention` takes these sizes (bf16 on the device only)."""
    if dtype != torch.bfloat16 or torch.device(device).type != "cuda":
        return False
    fn = getattr(lib(), "k8s_masked_attn_mfma_ok", None)
    return bool(fn(int(H), int(G), int(D), int(V))) if fn is not None else False


def head_norm_gate(o: torch.Tensor, gate: Optional[torch.Tensor], w: Optional[torch.Tensor], H: int, V: int, eps: float,
                   out_dtype, mul: Optional[torch.Tensor] = None, sub_lambda: Optional[float] = None,
                   out_scale: float = 1.0) -> torch.Tensor:
    """``u / rms(u over each head's V) * w * sigmoid(gate) * out_scale`` of fp32 rows ``o`` [T, H V], ``u = o * mul`` with
    ``mul`` [T, H] where given; ``w`` [V] (shared by the heads) or [H V] or None; ``gate`` [T, H V] fp32 (row stride
    free) or None.  With ``sub_lambda`` the rows hold two results per head, [T, H, 2, V], and
    ``u = o[:, :, 0] - sub_lambda * o[:, :, 1]`` (two score maps over the same values, joined)."""
    T = o.shape[0]
    out = torch.empty(T, H * V, dtype=out_dtype, device=o.device)
    sub = sub_lambda is not None
    if use_hip(o):
        assert o.dtype == torch.float32 and o.is_contiguous() and o.shape[1] == H * V * (2 if sub else 1)
        assert gate is None or (gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.shape[1] >= H * V)
        assert w is None or (w.dtype == torch.float32 and w.numel() in (V, H * V))
        assert mul is None or (mul.dtype == torch.float32 and mul.is_contiguous() and mul.numel() == T * H)
        check(lib().k8s_head_norm_gate(ptr(o), ptr(gate), gate.stride(0) if gate is not None else 0, ptr(w),
                                       V if w is not None and w.numel() == H * V else 0,
                                       ptr(out), T, H, V, float(eps), _dt(out_dtype), stream_ptr(o), ptr(mul),
                                       int(sub), float(sub_lambda or 0.0), float(out_scale)), "head_norm_gate")
        return out
    if sub:
        oh = o.view(T, H, 2, V)
        oh = oh[:, :, 0] - sub_lambda * oh[:, :, 1]
    else:
        oh = o.view(T, H, V)
    if mul is not None:
        oh = oh * mul.view(T, H, 1)
    oh = oh * torch.rsqrt(oh.pow(2).mean(-1, keepdim=True) + eps) * out_scale
    if w is not None:
        oh = oh * (w.view(H, V) if w.numel() == H * V else w.view(1, V))
    if gate is not None:
        oh = oh * torch.sigmoid(gate[:, :H * V]).view(T, H, V)
    out.copy_(oh.reshape(T, H * V).to(out_dtype))
    return out


MAT_CHUNK = 64      # rows per chunk of the chunk-parallel matrix-state recurrences
MAT_FILL_GROUPS = 1024   # workgroups (segments x heads x 64-column blocks) from which token by token fills the chip


def _mat_chunks(seg: SegMeta, H: int, V: int):
    """The chunk ranges of a step for the matrix-state recurrences, or None where they run token by token:
    no long portion, or enough sequences that the sequential form fills the chip at less than half the work."""
    if seg.n_seg * H * -(-V // 64) >= MAT_FILL_GROUPS:
        return None
    return seg.chunk_ranges(MAT_CHUNK, 2 * MAT_CHUNK)
UNIT_EPS = 1e-6     # q and k of the delta rule: x / sqrt(sum(x^2) + UNIT_EPS)


def gated_delta(qkv: torch.Tensor, H: int, G: int, D: int, V: int, a: torch.Tensor, rate: torch.Tensor,
                dt_bias: torch.Tensor, beta: torch.Tensor, state: torch.Tensor, seg: SegMeta) -> torch.Tensor:
    """Gated delta rule per head, fp32.  Rows of ``qkv`` [T, 2 G D + H V] = (q | k | v) activations; head h
    reads q / k head ``h // (H // G)``; q and k become unit vectors (``UNIT_EPS``), q times ``D^(-1/2)``.
    Decay per head and key channel ``g = exp(-rate_h softplus(a + dt_bias))`` from ``a`` [T, H D] fp32;
    ``beta`` [T, >= H] fp32 before its sigmoid (row stride free).  Per token
    ``S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q`` with ``S`` [D, V].
    ``state`` [slots, H, D, V] fp32 is read (past position 0) and advanced.  Returns o [T, H V] fp32."""
    T = qkv.shape[0]
    out = torch.empty(T, H * V, dtype=torch.float32, device=qkv.device)
    if use_hip(qkv):
        assert qkv.is_contiguous() and qkv.shape[1] == 2 * G * D + H * V and H % G == 0
        assert a.dtype == torch.float32 and a.is_contiguous() and a.shape == (T, H * D)
        assert beta.dtype == torch.float32 and beta.stride(1) == 1 and beta.shape[1] >= H
        assert rate.dtype == dt_bias.dtype == torch.float32 and rate.numel() == H and dt_bias.numel() == H * D
        assert state.is_contiguous() and state.shape[1:] == (H, D, V)
        # long portions: chunks in parallel (end states and step-matrix products from zero / identity, a carry
        # over the chunks, the chunks again from their start states); short ones token by token
        cr = _mat_chunks(seg, H, V)
        chunks, c0, cs, cx, nch = None, None, None, None, 0
        if cr is not None:
            chunks, c0 = cr
            nch = chunks.shape[0]
            cs = scratch(nch * H * D * V, torch.float32, qkv.device)
            cx = scratch(nch * H * D * D, torch.float32, qkv.device)
        check(lib().k8s_gated_delta(ptr(qkv), _dt(qkv.dtype), ptr(a), ptr(rate), ptr(dt_bias), ptr(beta),
                                    beta.stride(0), ptr(state), ptr(seg.seg_row0), ptr(seg.seg_pos0),
                                    ptr(seg.seg_slot), ptr(out), seg.n_seg, T, H, G, D, V, float(UNIT_EPS),
                                    stream_ptr(qkv), ptr(chunks), nch, ptr(c0), ptr(cs), ptr(cx)), "gated_delta")
        return out
    x = qkv.float()
    q = x[:, :G * D].view(T, G, D)
    k = x[:, G * D:2 * G * D].view(T, G, D)
    v = x[:, 2 * G * D:].view(T, H, V)
    q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + UNIT_EPS) * D ** -0.5
    k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + UNIT_EPS)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)      # [T, H, D]
    g = torch.exp(-rate.view(1, H, 1) * torch.nn.functional.softplus(a + dt_bias.view(1, -1)).view(T, H, D))
    bt = torch.sigmoid(beta[:, :H])
    for s in range(seg.n_seg):
        r0, r1, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        S = state[sl].clone() if p0 > 0 else torch.zeros(H, D, V)
        for r in range(r0, r1):
            S = g[r][:, :, None] * S
            u = bt[r][:, None] * (v[r] - torch.einsum("hdv,hd->hv", S, k[r]))
            S = S + k[r][:, :, None] * u[:, None, :]
            out[r] = torch.einsum("hdv,hd->hv", S, q[r]).reshape(-1)
        state[sl] = S
    return out


DEN_EPS = 1e-6      # matrix memory: o = S^T q / (max(|n.q|, exp(-m)) + DEN_EPS)


def matrix_memory(x: torch.Tensor, H: int, D: int, V: int, gate_bias: torch.Tensor, cap: float,
                  state: torch.Tensor, nstate: torch.Tensor, mstate: torch.Tensor, seg: SegMeta,
                  defer_scale: bool = False):
    """Matrix memory with exponential gates per head, fp32.  Rows of ``x`` [T, 2 H D + 2 H V + 2 H] fp32 =
    (q | k | v | . | i | f): q is scaled by ``D^(-1/2)``; the log gates are ``i = cap tanh((i + b_i) / cap)`` and
    ``f = logsigmoid(cap tanh((f + b_f) / cap))`` with ``gate_bias`` [2 H] = (b_i | b_f).  With the running maximum
    ``m`` (0 at the start of a sequence):  ``m' = max(f + m, i)``;  ``S <- e^(f + m - m') S + e^(i - m') k v^T``;  n likewise
    with k alone;  ``o = S^T q / (max(|n.q|, e^(-m')) + DEN_EPS)``.  ``state`` [slots, H, D, V], ``nstate`` [slots, H, D],
    ``mstate`` [slots, H] fp32 are read (past position 0) and advanced.  Returns o [T, H V] fp32; with
    ``defer_scale`` (o', mul) with ``o = o' * mul[:, :, None]``, ``mul`` [T, H], for :func:`head_norm_gate` to apply."""
    T = x.shape[0]
    out = torch.empty(T, H * V, dtype=torch.float32, device=x.device)
    if use_hip(x):
        assert x.dtype == torch.float32 and x.stride(1) == 1 and x.shape[1] == 2 * H * (D + V) + 2 * H
        assert gate_bias.dtype == torch.float32 and gate_bias.numel() == 2 * H
        assert state.is_contiguous() and state.shape[1:] == (H, D, V) and nstate.is_contiguous()
        assert nstate.shape[1:] == (H, D) and mstate.is_contiguous() and mstate.shape[1:] == (H,)
        ab = scratch(T * H * 3, torch.float32, x.device)
        nq = scratch(T * H, torch.float32, x.device)
        mul = scratch((T, H), torch.float32, x.device)
        # long portions: chunks in parallel (end states from zero, a carry over the chunks, the chunks again
        # from their start states); short ones token by token
        cr = _mat_chunks(seg, H, V)
        chunks, c0, cs, cx, cdec, nch = None, None, None, None, None, 0
        if cr is not None:
            chunks, c0 = cr
            nch = chunks.shape[0]
            cs = scratch(nch * H * D * V, torch.float32, x.device)
            cx = scratch(nch * H * D, torch.float32, x.device)
            cdec = scratch(nch * H, torch.float32, x.device)
        check(lib().k8s_matrix_memory(ptr(x), x.stride(0), ptr(gate_bias), float(cap), ptr(state), ptr(nstate),
                                      ptr(mstate), ptr(seg.seg_row0), ptr(seg.seg_pos0), ptr(seg.seg_slot), ptr(ab),
                                      ptr(nq), ptr(mul), ptr(out), seg.n_seg, T, H, D, V, float(DEN_EPS),
                                      0 if defer_scale else 1, stream_ptr(x), ptr(chunks), nch, ptr(c0), ptr(cs),
                                      ptr(cx), ptr(cdec)), "matrix_memory")
        return (out, mul) if defer_scale else out
    HD, HV = H * D, H * V
    q = x[:, :HD].view(T, H, D) * D ** -0.5
    k = x[:, HD:2 * HD].view(T, H, D)
    v = x[:, 2 * HD:2 * HD + HV].view(T, H, V)
    gi = x[:, 2 * HD + 2 * HV:2 * HD + 2 * HV + H] + gate_bias[:H]
    gf = x[:, 2 * HD + 2 * HV + H:] + gate_bias[H:]
    gi = cap * torch.tanh(gi / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(gf / cap))
    for s in range(seg.n_seg):
        r0, r1, p0, sl = seg.row0_host[s], seg.row0_host[s + 1], seg.pos0_host[s], seg.slot_host[s]
        if p0 > 0:
            S, n, m = state[sl].clone(), nstate[sl].clone(), mstate[sl].clone()
        else:
            S, n, m = torch.zeros(H, D, V), torch.zeros(H, D), torch.zeros(H)
        for r in range(r0, r1):
            mn = torch.maximum(gf[r] + m, gi[r])
            fa, ia = torch.exp(gf[r] + m - mn), torch.exp(gi[r] - mn)
            S = fa[:, None, None] * S + ia[:, None, None] * k[r][:, :, None] * v[r][:, None, :]
            n = fa[:, None] * n + ia[:, None] * k[r]
            m = mn
            den = torch.maximum((n * q[r]).sum(-1).abs(), torch.exp(-m)) + DEN_EPS
            out[r] = (torch.einsum("hdv,hd->hv", S, q[r]) / den[:, None]).reshape(-1)
        state[sl], nstate[sl], mstate[sl] = S, n, m
    return (out, None) if defer_scale else out
