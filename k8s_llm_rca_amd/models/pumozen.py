"""Pumozen decoder: post-sublayer norms -- each sublayer reads the raw fp32 residual and only its result is normed,

    x <- x + LN1(mixer(x));   x <- x + LN2(ff(x));   x <- x + rms(side_i(x, token)) w_side

with layer norms (weight and bias) on the sublayer outputs, three kinds of mixer, a dense or mixture-of-experts
feed-forward, and a per-layer token input behind the feed-forward.

``attention``:    q = W_q x, k = W_k x; keys double as values: what is cached as the value is the key projection
                  itself, taken in front of its norm and rotation (there is no value projection).  q and k get one
                  RMS norm each across ALL their heads (a weight as wide as the projection), then the rotation on
                  the first ``rot.dims`` entries of every head (rotate-half pairs); causal softmax whose denominator
                  holds one extra term e^0 (a sink without a value).
``mamba2``:       state-space duality: one projection gives ``z | x | B | C | dt``; ``x | B | C`` pass a short causal
                  convolution with bias and SiLU; ``dt = softplus(dt + dt_bias)``; per head
                  ``S <- exp(-e^(A_log) dt) S + dt B x^T``, ``y = S^T C + D x``; ``y silu(z)`` is RMS-normed in
                  ``norm_groups`` parts, times a weight.
``attention_2``:  differential attention: two score maps per head (q and k laid out [head][map]) with a softmax each
                  over the same values, ``o = a1 - lambda a2`` with one ``lambda = e^(lq1.lk1) - e^(lq2.lk2) + diff`` per
                  layer, a unit norm per head times ``1 - diff``, a sigmoid output gate ``W_g x``; q and k RMS-normed
                  per head and map with a shared weight; no rotation, but a query temperature
                  ``1 + coef ln(floor((p + 1) / every) + 1)``.  A layer with ``kv_from`` reads another layer's pages
                  with queries of its own.
feed-forward:     the clamped gated unit ``g sigmoid(1.702 g) (u + 1)`` with ``g = min(W_g h, limit)``,
                  ``u = clamp(W_u h, +-limit)``; dense, or experts chosen by a softmax router (top-k of the scores,
                  renormalised, times ``router.scale``) plus a shared expert gated by one sigmoid per token.
token side:       ``e = side.embed[token][i dim : (i + 1) dim]``; ``y = W_proj (gelu_tanh(W_gate x) e)``;
                  ``x <- x + y / rms(y) * w``.
Output:           the final layer norm, then the embedding table as the head.

What a sequence carries from step to step: keys and values of the attention layers that project their own, in
cache pages (:class:`~..engine.kv_cache.WindowKVPool`), and in its state slot every mamba2 layer's convolution tail
and state (fp32).  Every size, and every constant that can differ between checkpoints, comes from the
configuration or from a tensor's shape.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..ops import moe as M
from ..ops import norm as N
from ..ops import seq_ops as S
from ..ops.linear import linear, linear_f32out
from ..parallel.groups import ParallelContext, single
from .moe import MoELayerSet

GLU_ALPHA = 1.702       # g * sigmoid(GLU_ALPHA g) * (u + 1)
RENORM_EPS = 1e-20      # chosen scores / (their sum + RENORM_EPS)


@dataclass(frozen=True)
class SinkAttnSpec:
    """``attention``: keys double as values (``vdim == dim``)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int = 0           # 0: no rotation
    rot_base: float = 10000.0
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class DiffAttnSpec:
    """``attention_2``: two score maps per head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    temp_coef: float = 0.0
    temp_every: int = 0         # 0: no query temperature
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class SsdSpec:
    """``mamba2``."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim


@dataclass(frozen=True)
class FfSpec:
    kind: str                   # 'dense' | 'moe'
    ff: int                     # dense: its width; moe: an expert's
    limit: float
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    shared_ff: int = 0          # 0: no shared expert
    shared_limit: float = 0.0


@dataclass(frozen=True)
class LayerSpec:
    kind: str                   # 'attention' | 'mamba2' | 'attention_2'
    attn: Optional[SinkAttnSpec] = None
    diff: Optional[DiffAttnSpec] = None
    ssd: Optional[SsdSpec] = None
    mlp: Optional[FfSpec] = None


@dataclass(frozen=True)
class PumozenConfig:
    name: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    norm_eps: float = 1e-5
    side_dim: int = 0              # 0: no per-layer token input
    max_position: int = 1 << 20    # no tabulated positions: any length the cache holds
    arch: str = "pumozen"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "pumozen") -> "PumozenConfig":
        layers = []
        for L in d["layers"]:
            m, f = L.get("mixer") or {}, L.get("mlp")
            mlp = None
            if f is not None:
                kind = f.get("kind", "dense")
                if kind == "dense":
                    mlp = FfSpec("dense", int(f["ff"]), float(f["limit"]))
                elif kind == "moe":
                    e, r, sh = f["expert"], f["router"], f.get("shared")
                    mlp = FfSpec("moe", int(e["ff"]), float(e["limit"]), int(r["experts"]), int(r["top"]),
                                 float(r.get("scale", 1.0)), int(sh["ff"]) if sh else 0,
                                 float(sh["limit"]) if sh else 0.0)
                else:
                    raise ValueError(f"unknown feed-forward kind {kind!r}")
            kind = L["type"]
            kvf = m.get("kv_from")
            kvf = int(kvf) if kvf is not None else None
            if kind == "attention":
                rot = m.get("rot") or {}
                layers.append(LayerSpec(kind, attn=SinkAttnSpec(
                    int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                    float(m["scale"]), int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), kvf), mlp=mlp))
            elif kind == "attention_2":
                qt = m.get("q_temp") or {}
                layers.append(LayerSpec(kind, diff=DiffAttnSpec(
                    int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                    float(m["scale"]), float(m["diff"]), float(qt.get("coef", 0.0)), int(qt.get("every", 0)), kvf),
                    mlp=mlp))
            elif kind == "mamba2":
                layers.append(LayerSpec(kind, ssd=SsdSpec(
                    int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1)), int(m.get("conv", 1)),
                    int(m.get("norm_groups", 1))), mlp=mlp))
            else:
                raise ValueError(f"unknown mixer type {kind!r}")
        return cls(name, int(d["vocab"]), int(d["width"]), tuple(layers), norm_eps=float(d["norm"]["eps"]),
                   side_dim=int((d.get("token_side") or {}).get("dim", 0)))

    def to_json(self) -> dict:
        layers = []
        for L in self.layers:
            if L.kind == "attention":
                a = L.attn
                m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
                if a.rot_dims:
                    m["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
                if a.kv_from is not None:
                    m["kv_from"] = a.kv_from
            elif L.kind == "attention_2":
                a = L.diff
                m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                     "diff": a.diff}
                if a.temp_every:
                    m["q_temp"] = {"coef": a.temp_coef, "every": a.temp_every}
                if a.kv_from is not None:
                    m["kv_from"] = a.kv_from
            else:
                c = L.ssd
                m = {"heads": c.heads, "vdim": c.vdim, "state": c.state, "groups": c.groups, "conv": c.conv,
                     "norm_groups": c.norm_groups}
            f = L.mlp
            if f is None:
                mlp = None
            elif f.kind == "dense":
                mlp = {"kind": "dense", "ff": f.ff, "limit": f.limit}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit},
                       "router": {"experts": f.experts, "top": f.top, "scale": f.router_scale},
                       "shared": {"ff": f.shared_ff, "limit": f.shared_limit} if f.shared_ff else None}
            layers.append({"type": L.kind, "mixer": m, "mlp": mlp})
        d = {"architecture": "Pumozen", "vocab": self.vocab_size, "width": self.hidden, "layers": layers,
             "norm": {"eps": self.norm_eps}}
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        return d


def _stack(n_groups: int, W: int, heads: int, kv_heads: int, dim: int, ff: int, experts: int, state: int):
    """Groups of (mamba2 + dense, attention_2 + experts, attention + dense, attention_2 on the first one's pages +
    experts).  The two-map attention has half the head size for its scores and the full one for its values."""
    dense = FfSpec("dense", ff, 7.0)
    moe = FfSpec("moe", ff // 4, 7.0, experts, 2, 1.5, ff // 4, 7.0)
    out = []
    for g in range(n_groups):
        b = 4 * g
        two = dict(heads=heads, kv_heads=kv_heads, dim=dim // 2, vdim=dim, scale=1.0 / math.sqrt(dim // 2), diff=0.6,
                   temp_coef=0.2, temp_every=512)
        out += [LayerSpec("mamba2", ssd=SsdSpec(2 * W // 64, 64, state, max(1, heads // 8), 4, 2), mlp=dense),
                LayerSpec("attention_2", diff=DiffAttnSpec(**two), mlp=moe),
                LayerSpec("attention", attn=SinkAttnSpec(heads, kv_heads, dim, dim, 1.0 / math.sqrt(dim), dim // 2,
                                                         500000.0), mlp=dense),
                LayerSpec("attention_2", diff=DiffAttnSpec(kv_from=b + 1, **two), mlp=moe)]
    return tuple(out)


PRESETS: Dict[str, PumozenConfig] = {
    "tiny-pumozen": PumozenConfig("tiny-pumozen", 8192, 256, _stack(1, 256, 4, 2, 32, 512, 4, 16), side_dim=16),
    # sizes of a ~1B-class decoder's layers (benchmarks; random weights)
    "pumozen-1b": PumozenConfig("pumozen-1b", 32768, 2048, _stack(3, 2048, 16, 2, 128, 8192, 8, 64), side_dim=256),
}


class PumozenModel:
    stateful = True            # per-sequence state slots besides cache pages: no rewinding, no page sharing
    step_layout = "segments"   # the engine packs steps as segments (ops.seq_ops.SegStepInputs)
    graph_capturable = False

    def __init__(self, cfg: PumozenConfig, device, dtype=torch.bfloat16, pc: Optional[ParallelContext] = None,
                 seed: int = 0, init: bool = True):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Pumozen runs in bfloat16 or float32")
        self.dtype = dtype
        self.pc = pc or single()
        if self.pc.tp_size != 1:
            raise ValueError("Pumozen runs on one device per replica (no tensor-parallel sharding of its mixers)")
        self.logits_f32 = True
        self.layers: List[Dict[str, object]] = []
        # layer -> index of the key / value pages it reads (its own or, with kv_from, another layer's),
        # and of its mamba2 state
        self.cache_of: List[Optional[int]] = []
        self.cache_dims: List[Tuple[int, int, int, int, int]] = []     # (H, G, maps, D, V) per projecting attention
        self.ssd_of: List[Optional[int]] = []
        n_ssd = 0
        for i, L in enumerate(cfg.layers):
            a = L.attn or L.diff
            self.ssd_of.append(None)
            if a is None:
                c = L.ssd
                if c.heads % c.groups or c.inner % c.norm_groups or not 1 <= c.conv <= 16 or not 1 <= c.state <= 128:
                    raise ValueError(f"layer {i}: heads a multiple of groups, heads * vdim a multiple of "
                                     f"norm_groups, conv 1..16, state 1..128")
                self.cache_of.append(None)
                self.ssd_of[i] = n_ssd
                n_ssd += 1
                continue
            if a.heads % a.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            maps = 2 if L.kind == "attention_2" else 1
            if L.kind == "attention":
                if a.vdim != a.dim:
                    raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
                if a.rot_dims % 2 or a.rot_dims > a.dim:
                    raise ValueError(f"layer {i}: an even rot.dims <= dim")
            dims = (a.heads, a.kv_heads, maps, a.dim, a.vdim)
            if a.kv_from is None:
                self.cache_of.append(len(self.cache_dims))
                self.cache_dims.append(dims)
            else:
                j = a.kv_from
                if not 0 <= j < i or cfg.layers[j].kind != L.kind or (cfg.layers[j].attn or cfg.layers[j].diff).kv_from \
                        is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier layer of the same kind that projects "
                                     f"its own keys and values")
                if self.cache_dims[self.cache_of[j]] != dims:
                    raise ValueError(f"layer {i}: head counts and sizes must equal those of layer {j}")
                self.cache_of.append(self.cache_of[j])
            f = L.mlp
            if f is not None and f.kind == "moe" and not 1 <= f.top <= f.experts:
                raise ValueError(f"layer {i}: top must be 1..experts")
        if init:
            self._random_init(seed)

    # ------------------------------------------------------- what the engine allocates for this model
    def _twins(self) -> List[bool]:
        """Per cached attention: whether the matrix-core kernel runs it (then its values are also cached transposed)."""
        return [S.masked_mfma_ok(H, G, D, V, self.dtype, self.device) for H, G, _, D, V in self.cache_dims]

    def _widths(self) -> List[Tuple[int, int]]:
        return [(G * m * D, G * V) for _, G, m, D, V in self.cache_dims]

    def cache_bytes_per_block(self, block_size: int) -> int:
        per = sum(a + (2 * b if tw else b) for (a, b), tw in zip(self._widths(), self._twins()))
        return max(1, per) * block_size * (2 if self.dtype == torch.bfloat16 else 4)

    def make_cache(self, num_blocks: int, block_size: int):
        from ..engine.kv_cache import WindowKVPool
        return WindowKVPool(self._widths(), num_blocks, block_size, self.device, self.dtype, self._twins())

    def state_spec(self) -> Dict[str, Tuple[int, ...]]:
        """Per-slot fp32 state tensors: name -> shape behind the slot dimension."""
        spec: Dict[str, Tuple[int, ...]] = {}
        for i, L in enumerate(self.cfg.layers):
            if L.kind == "mamba2":
                j, c = self.ssd_of[i], L.ssd
                spec[f"conv{j}"] = (c.conv - 1, c.inner + 2 * c.groups * c.state)
                spec[f"ssd{j}"] = (c.inner, c.state)
        return spec

    def workspace_bytes(self, tokens: int) -> int:
        w = self.cfg.hidden
        widest = w
        for L in self.cfg.layers:
            a = L.attn or L.diff
            if a is not None:
                m = 2 if L.kind == "attention_2" else 1
                widest = max(widest, 2 * (a.heads * m * (a.dim + a.vdim) + a.kv_heads * (m * a.dim + a.vdim)))
            else:
                widest = max(widest, 4 * L.ssd.inner + 4 * L.ssd.groups * L.ssd.state)
            f = L.mlp
            if f is not None:
                widest = max(widest, 3 * f.ff * max(1, f.top) + w * f.top, 3 * f.shared_ff)
        return int(tokens * (4 * w * 4 + widest * 8) + (2 << 30))

    # --------------------------------------------------------------- weights
    def _random_init(self, seed: int) -> None:
        t = random_tensors(self.cfg, seed, self.device)
        self.load_tensors(t.__getitem__)

    def load_tensors(self, get, has=None) -> None:
        """Build the fused device layout from checkpoint tensors (``get(name)`` -> tensor; names of the
        safetensors file: ``embed``, ``side.embed``, ``l<i>.norm1``, ``l<i>.mix.q`` ...)."""
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def put(*names, dtype=dt):
            ts = [get(n) for n in names]
            t = ts[0] if len(ts) == 1 else torch.cat([x.reshape(x.shape[0], -1) if x.dim() > 1 else x for x in ts], 0)
            return t.to(device=dev, dtype=dtype).contiguous()

        def f32(*names):
            return put(*names, dtype=torch.float32)

        def norm(name):
            return f32(name), f32(name + ".b")

        self.embed = put("embed")
        self.side_embed = put("side.embed") if cfg.side_dim else None
        self.final_norm = norm("final.norm")
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p = f"l{i}.mix."
            L: Dict[str, object] = {"norm1": norm(f"l{i}.norm1")}
            if spec.kind == "attention":
                a = spec.attn
                own = a.kv_from is None
                L["w_in"] = put(p + "q", p + "k") if own else put(p + "q")       # one fp32-out GEMM: q | k (= v)
                L["q_w"] = f32(p + "q.norm")
                L["k_w"] = f32(p + "k.norm") if own else None
                L["sink"] = torch.zeros(a.heads, dtype=torch.float32, device=dev)   # the sink's score is 0
                L["wo"] = put(p + "o")
            elif spec.kind == "attention_2":
                a = spec.diff
                own = a.kv_from is None
                L["w_in"] = put(p + "q", p + "k", p + "v", p + "g") if own else put(p + "q", p + "g")
                L["q_w"] = f32(p + "q.norm")
                L["k_w"] = f32(p + "k.norm") if own else None

                def dot(x, y):
                    return float((get(p + x).double() * get(p + y).double()).sum())

                L["lam"] = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + a.diff
                L["wo"] = put(p + "o")
            else:
                L["w_in"] = put(p + "in")                                        # z | x | B | C | dt, fp32 out
                L["conv_w"], L["conv_b"] = f32(p + "conv"), f32(p + "conv.b")
                L["dt_bias"] = f32(p + "dt_bias")
                L["rate"] = torch.exp(f32(p + "A_log")).contiguous()
                L["D"] = f32(p + "D")
                L["ssd_norm"] = f32(p + "norm")
                L["wo"] = put(p + "o")
            f = spec.mlp
            if f is not None:
                m = f"l{i}.mlp."
                L["norm2"] = norm(f"l{i}.norm2")
                if f.kind == "dense":
                    L["w13"] = put(m + "gate", m + "up")
                    L["w2"] = put(m + "down")
                else:
                    # the shared expert's per-token gate rides behind the experts' rows of the router
                    L["router"] = put(m + "router", m + "shared.sg") if f.shared_ff else put(m + "router")
                    L["w13"] = torch.stack([put(m + f"e{e}.gate", m + f"e{e}.up") for e in range(f.experts)]).contiguous()
                    L["w2"] = torch.stack([put(m + f"e{e}.down") for e in range(f.experts)]).contiguous()
                    if f.shared_ff:
                        L["ws13"] = put(m + "shared.gate", m + "shared.up")
                        L["ws2"] = put(m + "shared.down")
            if cfg.side_dim:
                L["side_gate"], L["side_proj"] = put(f"l{i}.side.gate"), put(f"l{i}.side.proj")
                L["side_norm"] = f32(f"l{i}.side.norm")
            self.layers.append(L)

    def weight_bytes(self) -> int:
        def size(v):
            if isinstance(v, tuple):
                return sum(size(t) for t in v)
            return v.numel() * v.element_size() if isinstance(v, torch.Tensor) else 0
        n = sum(size(t) for L in self.layers for t in L.values())
        return n + sum(size(t) for t in (self.embed, self.side_embed, self.final_norm))

    # -------------------------------------------------------------- forward
    def _lin32(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w.T with an fp32 result (fp32 accumulation either way)."""
        return linear_f32out(x, w) if self.dtype == torch.bfloat16 else linear(x, w)

    def _attention(self, li: int, h, inp: S.SegStepInputs, kcs, vcs, vts) -> torch.Tensor:
        L, a = self.layers[li], self.cfg.layers[li].attn
        ci = self.cache_of[li]
        H, G, D = a.heads, a.kv_heads, a.dim
        own = a.kv_from is None
        x = self._lin32(h, L["w_in"])                                  # [T, H D (+ G D)] fp32
        q = S.attn_prep(x, None, H, G if own else 0, D, D, inp.positions, inp.slots, kcs[ci] if own else None,
                        vcs[ci] if own else None, self.dtype, norm="all", q_w=L["q_w"], k_w=L["k_w"],
                        eps=self.cfg.norm_eps, rot_dims=a.rot_dims, rot_base=a.rot_base,
                        vt=vts[ci] if own else None, v_is_k=own)
        o = S.masked_attention(q, H, G, D, D, kcs[ci], vcs[ci], inp.seg, a.scale, sink=L["sink"], vt=vts[ci])
        return self._lin32(o, L["wo"])

    def _attention_2(self, li: int, h, inp: S.SegStepInputs, kcs, vcs, vts) -> torch.Tensor:
        L, a = self.layers[li], self.cfg.layers[li].diff
        ci = self.cache_of[li]
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        own = a.kv_from is None
        x = self._lin32(h, L["w_in"])                                  # q | k | v | gate, or q | gate; fp32
        nq = 2 * H * D + (2 * G * D + G * V if own else 0)
        q = S.attn_prep(x[:, :nq], None, H, G if own else 0, D, V, inp.positions, inp.slots,
                        kcs[ci] if own else None, vcs[ci] if own else None, self.dtype, norm="head", q_w=L["q_w"],
                        k_w=L["k_w"], eps=self.cfg.norm_eps, vt=vts[ci] if own else None, maps=2,
                        q_temp=(a.temp_coef, a.temp_every) if a.temp_every else None)
        o2 = S.masked_attention(q, H, G, D, V, kcs[ci], vcs[ci], inp.seg, a.scale, vt=vts[ci], maps=2, out_f32=True)
        o = S.head_norm_gate(o2, x[:, nq:], None, H, V, self.cfg.norm_eps, self.dtype, sub_lambda=L["lam"],
                             out_scale=1.0 - a.diff)
        return self._lin32(o, L["wo"])

    def _mamba2(self, li: int, h, inp: S.SegStepInputs, states) -> torch.Tensor:
        L, c = self.layers[li], self.cfg.layers[li].ssd
        j = self.ssd_of[li]
        inner, gn = c.inner, c.groups * c.state
        zx = self._lin32(h, L["w_in"])                                 # [T, 2 inner + 2 G N + heads] fp32
        xbc = S.short_conv(zx[:, inner:2 * inner + 2 * gn], L["conv_w"], L["conv_b"], states[f"conv{j}"], inp.seg,
                           act=True)
        y = S.ssd_scan(xbc[:, :inner], xbc[:, inner:], zx[:, 2 * inner + 2 * gn:], L["dt_bias"], L["rate"], L["D"],
                       zx[:, :inner], c.heads, c.vdim, c.groups, c.state, states[f"ssd{j}"], inp.seg,
                       fast_exp=self.dtype == torch.bfloat16)
        o = S.head_norm_gate(y, None, L["ssd_norm"], c.norm_groups, inner // c.norm_groups, self.cfg.norm_eps,
                             self.dtype)
        return self._lin32(o, L["wo"])

    def _unit(self, gu: torch.Tensor, limit: float) -> torch.Tensor:
        return M.glu_clamp(gu, GLU_ALPHA, limit, 1.0)

    def _moe(self, li: int, h: torch.Tensor):
        """(routed experts' output, shared expert's output or None, the shared expert's gate logits or None);
        outputs fp32 [T, W]."""
        L, f = self.layers[li], self.cfg.layers[li].mlp
        T = h.shape[0]
        r = M.route_direct(h, L["router"], f.top, scoring="softmax", renorm=True, renorm_eps=RENORM_EPS,
                           scale=f.router_scale, extra_rows=1 if f.shared_ff else 0)
        w, ids = r[0], r[1]
        order, inv, offsets = M.align(ids, f.experts)
        xp = M.gather_rows(h, order, f.top)
        rows = xp.shape[0]
        dev16 = xp.is_cuda and xp.dtype == torch.bfloat16
        if dev16 and rows <= MoELayerSet.GLDS_MAX_ROWS:
            # decode sizes: the weight-streaming kernels the Mixtral block runs there (LDS-DMA strips for
            # gate | up; the down projection below with its K split over workgroups)
            gu = M.grouped_gemm(xp, L["w13"], offsets, glds=MoELayerSet.GLDS_UP[0], splits=MoELayerSet.GLDS_UP[1])
        else:
            gu = M.grouped_auto(xp, L["w13"], offsets)
        act = self._unit(gu, f.limit)
        if dev16 and rows <= MoELayerSet.SPLIT_MAX_ROWS:
            yp = M.grouped_gemm(act, L["w2"], offsets, splits=MoELayerSet.DOWN_SPLITS)
        else:
            yp = M.grouped_auto(act, L["w2"], offsets)
        routed = M.combine_f32(yp, inv, T, f.top, w)
        if not f.shared_ff:
            return routed, None, None
        shared = self._lin32(self._unit(linear(h, L["ws13"]), f.shared_limit), L["ws2"])
        return routed, shared, r[2]

    def forward(self, inp: S.SegStepInputs, kcs: List[torch.Tensor], vcs: List[torch.Tensor],
                vts: List[Optional[torch.Tensor]], states: Dict[str, torch.Tensor],
                layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits [len(logits_idx), vocab] fp32.  ``kcs`` / ``vcs``: the paged keys and values of every attention that
        projects its own (``vts``: the values' transposed twins, or None); ``states``: the per-slot tensors of
        :meth:`state_spec`.  ``layers_out`` (debugging): receives a copy of the residual after every layer."""
        cfg, eps, dt = self.cfg, self.cfg.norm_eps, self.dtype
        T, W = inp.input_ids.shape[0], cfg.hidden
        x = torch.empty(T, W, dtype=torch.float32, device=self.device)
        h = N.embed_rows(inp.input_ids, self.embed, x, out_dtype=dt)     # h: the residual as the GEMMs read it
        for li, (spec, L) in enumerate(zip(cfg.layers, self.layers)):
            if spec.kind == "attention":
                y = self._attention(li, h, inp, kcs, vcs, vts)
            elif spec.kind == "attention_2":
                y = self._attention_2(li, h, inp, kcs, vcs, vts)
            else:
                y = self._mamba2(li, h, inp, states)
            h = N.ln_residual(x, y, *L["norm1"], eps, x, out_dtype=dt, cast=True)
            f = spec.mlp
            if f is not None and f.kind == "dense":
                y = self._lin32(self._unit(linear(h, L["w13"]), f.limit), L["w2"])
                h = N.ln_residual(x, y, *L["norm2"], eps, x, out_dtype=dt, cast=True)
            elif f is not None:
                routed, shared, sg = self._moe(li, h)
                h = N.ln_residual(x, routed, *L["norm2"], eps, x, y2=shared, merge="gated", row_gate=sg,
                                  out_dtype=dt, cast=True)
            if cfg.side_dim:
                g = N.token_gate(self._lin32(h, L["side_gate"]), inp.input_ids, self.side_embed, li * cfg.side_dim, dt)
                h = N.ln_residual(x, self._lin32(g, L["side_proj"]), L["side_norm"], None, eps, x, kind="rms",
                                  out_dtype=dt, cast=True)
            if layers_out is not None:
                layers_out.append(x.clone())
        xr = x.index_select(0, inp.logits_idx).contiguous()
        return self._lin32(N.layernorm(xr, *self.final_norm, eps, dt), self.embed)


def random_tensors(cfg: PumozenConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint's names, bfloat16 (so a bfloat16 and a float32 model
    built from them hold the same numbers)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W = cfg.hidden

    def rnd(*shape, std=0.02, mean=0.0):
        return torch.empty(*shape, dtype=torch.float32, device=dev).normal_(mean, std, generator=g).to(torch.bfloat16)

    def lin(n_out, n_in, gain=1.0):
        return rnd(n_out, n_in, std=gain / math.sqrt(n_in))

    t: Dict[str, torch.Tensor] = {"embed": rnd(cfg.vocab_size, W, std=1.0)}
    if cfg.side_dim:
        t["side.embed"] = rnd(cfg.vocab_size, cfg.side_dim * cfg.n_layers, std=1.0)

    def norm(name):
        t[name] = rnd(W, std=0.1, mean=1.0)
        t[name + ".b"] = rnd(W, std=0.05)

    def unit(p, ff):
        t[p + "gate"], t[p + "up"], t[p + "down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff)

    norm("final.norm")
    for i, L in enumerate(cfg.layers):
        p = f"l{i}.mix."
        norm(f"l{i}.norm1")
        if L.kind == "attention":
            a = L.attn
            t[p + "q"], t[p + "o"] = lin(a.heads * a.dim, W), lin(W, a.heads * a.vdim)
            t[p + "q.norm"] = rnd(a.heads * a.dim, std=0.2, mean=1.5)
            if a.kv_from is None:
                t[p + "k"] = lin(a.kv_heads * a.dim, W)
                t[p + "k.norm"] = rnd(a.kv_heads * a.dim, std=0.2, mean=1.5)
        elif L.kind == "attention_2":
            a = L.diff
            t[p + "q"], t[p + "o"] = lin(a.heads * 2 * a.dim, W), lin(W, a.heads * a.vdim)
            t[p + "g"] = lin(a.heads * a.vdim, W, 2.0)
            t[p + "q.norm"] = rnd(a.dim, std=0.2, mean=1.5)
            for n_ in ("lq1", "lk1", "lq2", "lk2"):
                t[p + n_] = rnd(a.dim, std=0.15)
            if a.kv_from is None:
                t[p + "k"], t[p + "v"] = lin(a.kv_heads * 2 * a.dim, W), lin(a.kv_heads * a.vdim, W)
                t[p + "k.norm"] = rnd(a.dim, std=0.2, mean=1.5)
        else:
            c = L.ssd
            ch = c.inner + 2 * c.groups * c.state
            t[p + "in"] = lin(c.inner + ch + c.heads, W)
            t[p + "conv"], t[p + "conv.b"] = rnd(ch, c.conv, std=0.5), rnd(ch, std=0.1)
            t[p + "dt_bias"] = rnd(c.heads, std=0.5, mean=-1.0)
            t[p + "A_log"] = rnd(c.heads, std=0.5, mean=-1.0)
            t[p + "D"] = rnd(c.heads, std=0.3, mean=1.0)
            t[p + "norm"] = rnd(c.inner, std=0.1, mean=1.0)
            t[p + "o"] = lin(W, c.inner)
        f = L.mlp
        if f is not None:
            m = f"l{i}.mlp."
            norm(f"l{i}.norm2")
            if f.kind == "dense":
                unit(m, f.ff)
            else:
                t[m + "router"] = lin(f.experts, W, 2.0)
                for e in range(f.experts):
                    unit(m + f"e{e}.", f.ff)
                if f.shared_ff:
                    unit(m + "shared.", f.shared_ff)
                    t[m + "shared.sg"] = lin(1, W, 2.0)
        if cfg.side_dim:
            t[f"l{i}.side.gate"], t[f"l{i}.side.proj"] = lin(cfg.side_dim, W, 2.0), lin(W, cfg.side_dim)
            t[f"l{i}.side.norm"] = rnd(W, std=0.1, mean=0.5)
    return t


def load_checkpoint(path: str, device, dtype, pc=None) -> PumozenModel:
    """A folder with config.json and model.safetensors (bfloat16 weights) -> the model on ``device``."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = PumozenConfig.from_json(json.load(f), name=os.path.basename(os.path.normpath(path)) or "pumozen")
    model = PumozenModel(cfg, device, dtype, pc, init=False)
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as h:
        model.load_tensors(h.get_tensor, set(h.keys()).__contains__)
    return model


def save_checkpoint(cfg: PumozenConfig, tensors: Dict[str, torch.Tensor], path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) in the layout :func:`load_checkpoint` reads."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
