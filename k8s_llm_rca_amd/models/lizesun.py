"""Lizesun decoder: pre-normed sublayers over an fp32 residual with the Dynamic Tanh norm
(``tanh(alpha x) w + b``: no statistics), three kinds of mixer and a dense squared-ReLU feed-forward.

    x <- x + mixer(dyt1(x));   x <- x + down(relu(up(dyt2(x)))^2)      # the second when the layer has a feed-forward

``attention``:     q / k / v with biases, RMS norm (plain weight) on every q and k head, no positions in the
                   scores, ``s = softcap tanh(scale q.k / softcap)``, a CHUNKED causal mask (i sees j <= i of its own
                   chunk of ``mask.size`` positions), values mixed with the first such layer's values of the same
                   token (``(1 - lam) v + lam v_first``, the mixed values are cached), one sigmoid gate per head.
``parallel``:      ``left_scale * left + right_scale * right`` of two mixers reading the same input:
                   left  -- rotary q / k (rotate-half pairs on the first ``rot.dims`` entries), then q and k divided
                            by their root mean square, sliding window that also keeps the sequence's first
                            ``mask.keep_first`` tokens, a learned sink per head in the softmax's denominator;
                   right -- a matrix memory with exponential input / forget gates (soft-capped, stabilised by a
                            running maximum), normaliser state, per-head unit norm, sigmoid gate.
``channel_delta``: short causal convolution + SiLU on q, k, v; unit-length q / k; the gated delta rule with one
                   decay per head and key channel (low-rank projection, softplus step size); per-head unit norm,
                   low-rank sigmoid gate.
Output:            the final Dynamic Tanh norm, then the head.

What a sequence carries from step to step: keys and values of the attention layers in cache pages
(:class:`~..engine.kv_cache.WindowKVPool`), and in its state slot the convolution tails, delta-rule states and
matrix memories with their normalisers and maxima (fp32).  Every size and every constant that can differ
between checkpoints comes from the configuration or from a tensor's shape.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..ops import norm as N
from ..ops import seq_ops as S
from ..ops.linear import linear, linear_f32out
from ..parallel.groups import ParallelContext, single


@dataclass(frozen=True)
class ChunkAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    chunk: int              # 0: plain causal
    scale: float
    softcap: float = 0.0    # 0: scores are not capped
    v_mix: bool = False


@dataclass(frozen=True)
class WindowSinkSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int             # 0: plain causal
    keep_first: int
    scale: float
    rot_dims: int = 0       # 0: no rotation
    rot_base: float = 10000.0


@dataclass(frozen=True)
class MemorySpec:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class DeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    # ranks of the decay's and the gate's low-rank projections: a checkpoint's tensors give them
    # (config.json does not); these are what random initialisation uses
    a_rank: int = 16
    g_rank: int = 16


@dataclass(frozen=True)
class LayerSpec:
    kind: str                               # 'attention' | 'parallel' | 'channel_delta'
    attn: Optional[ChunkAttnSpec] = None
    left: Optional[WindowSinkSpec] = None
    right: Optional[MemorySpec] = None
    delta: Optional[DeltaSpec] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    ff: int = 0                             # 0: no feed-forward


@dataclass(frozen=True)
class LizesunConfig:
    name: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    norm_eps: float = 1e-5
    embed_scale: float = 1.0
    max_position: int = 1 << 20    # no tabulated positions: any length the cache holds
    arch: str = "lizesun"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "lizesun") -> "LizesunConfig":
        layers = []
        for L in d["layers"]:
            m = L.get("mixer") or {}
            f = L.get("mlp")
            ff = 0
            if f is not None:
                if f.get("kind", "dense") != "dense":
                    raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
                ff = int(f["ff"])
            kind = L["type"]
            if kind == "attention":
                layers.append(LayerSpec(kind, attn=ChunkAttnSpec(
                    int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                    int((m.get("mask") or {}).get("size", 0)), float(m["scale"]), float(m.get("softcap") or 0.0),
                    bool(m.get("v_mix", False))), ff=ff))
            elif kind == "parallel":
                a, b = m["left"], m["right"]
                mask, rot = a.get("mask") or {}, a.get("rot") or {}
                layers.append(LayerSpec(
                    kind,
                    left=WindowSinkSpec(int(a["heads"]), int(a.get("kv_heads", a["heads"])), int(a["dim"]),
                                        int(a.get("vdim", a["dim"])), int(mask.get("size", 0)),
                                        int(mask.get("keep_first", 0)), float(a["scale"]), int(rot.get("dims", 0)),
                                        float(rot.get("base", 10000.0))),
                    right=MemorySpec(int(b["heads"]), int(b["dim"]), int(b.get("vdim", b["dim"])),
                                     float(b["gate_cap"])),
                    left_scale=float(m.get("left_scale", 1.0)), right_scale=float(m.get("right_scale", 1.0)), ff=ff))
            elif kind == "channel_delta":
                layers.append(LayerSpec(kind, delta=DeltaSpec(
                    int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                    int(m.get("conv", 1)), int(m.get("a_rank", 16)), int(m.get("g_rank", 16))), ff=ff))
            else:
                raise ValueError(f"unknown mixer type {kind!r}")
        return cls(name, int(d["vocab"]), int(d["width"]), tuple(layers), norm_eps=float(d["norm"]["eps"]),
                   embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)))

    def to_json(self) -> dict:
        layers = []
        for L in self.layers:
            if L.kind == "attention":
                a = L.attn
                m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                     "v_mix": a.v_mix}
                if a.chunk:
                    m["mask"] = {"size": a.chunk}
                if a.softcap:
                    m["softcap"] = a.softcap
            elif L.kind == "parallel":
                a, b = L.left, L.right
                left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
                if a.window:
                    left["mask"] = {"size": a.window, "keep_first": a.keep_first}
                if a.rot_dims:
                    left["rot"] = {"dims": a.rot_dims, "base": a.rot_base}
                m = {"left": left, "right": {"heads": b.heads, "dim": b.dim, "vdim": b.vdim, "gate_cap": b.gate_cap},
                     "left_scale": L.left_scale, "right_scale": L.right_scale}
            else:
                c = L.delta
                m = {"heads": c.heads, "kv_heads": c.kv_heads, "dim": c.dim, "vdim": c.vdim, "conv": c.conv,
                     "a_rank": c.a_rank, "g_rank": c.g_rank}
            layers.append({"type": L.kind, "mixer": m, "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None})
        return {"architecture": "Lizesun", "vocab": self.vocab_size, "width": self.hidden,
                "embedding": {"scale": self.embed_scale}, "layers": layers, "norm": {"eps": self.norm_eps}}


def _stack(n_groups: int, W: int, heads: int, kv_heads: int, dim: int, chunk: int, window: int, ff: int):
    """Groups of (attention, parallel, channel_delta, attention), every layer with a feed-forward."""
    att = LayerSpec("attention", attn=ChunkAttnSpec(heads, kv_heads, dim, dim, chunk, 1.0 / math.sqrt(dim), 30.0,
                                                    True), ff=ff)
    par = LayerSpec("parallel",
                    left=WindowSinkSpec(heads, kv_heads, dim, dim, window, 4, 1.0 / math.sqrt(dim) * 8.0, dim // 2,
                                        50000.0),
                    right=MemorySpec(heads, dim // 2, dim, 15.0), left_scale=0.7, right_scale=0.9, ff=ff)
    dlt = LayerSpec("channel_delta", delta=DeltaSpec(heads, kv_heads, dim // 2, dim, 4, max(8, W // 32),
                                                     max(8, W // 32)), ff=ff)
    return tuple([att, par, dlt, att] * n_groups)


PRESETS: Dict[str, LizesunConfig] = {
    "tiny-lizesun": LizesunConfig("tiny-lizesun", 8192, 256, _stack(1, 256, 4, 2, 32, 40, 24, 512), embed_scale=4.0),
    # sizes of a ~1B-class decoder's layers (benchmarks; random weights)
    "lizesun-1b": LizesunConfig("lizesun-1b", 32768, 2048, _stack(3, 2048, 16, 2, 128, 1024, 1024, 8192),
                                embed_scale=8.0),
}


class LizesunModel:
    stateful = True            # per-sequence state slots besides cache pages: no rewinding, no page sharing
    step_layout = "segments"   # the engine packs steps as segments (ops.seq_ops.SegStepInputs)
    graph_capturable = False

    def __init__(self, cfg: LizesunConfig, device, dtype=torch.bfloat16, pc: Optional[ParallelContext] = None,
                 seed: int = 0, init: bool = True):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lizesun runs in bfloat16 or float32")
        self.dtype = dtype
        self.pc = pc or single()
        if self.pc.tp_size != 1:
            raise ValueError("Lizesun runs on one device per replica (no tensor-parallel sharding of its mixers)")
        self.logits_f32 = True
        self.layers: List[Dict[str, object]] = []
        # layer -> index of its key / value pages, of its delta-rule state, of its matrix memory
        self.cache_of: List[Optional[int]] = []
        self.cache_dims: List[Tuple[int, int, int, int]] = []     # (H, G, D, V) per attention
        self.delta_of: List[Optional[int]] = []
        self.mem_of: List[Optional[int]] = []
        self.vmix_first: Optional[int] = None                     # the first layer that mixes values
        n_delta = n_mem = 0
        vmix_width = None
        for i, L in enumerate(cfg.layers):
            a = L.attn if L.kind == "attention" else L.left
            if a is not None:
                if a.heads % a.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                self.cache_of.append(len(self.cache_dims))
                self.cache_dims.append((a.heads, a.kv_heads, a.dim, a.vdim))
            else:
                self.cache_of.append(None)
            if L.kind == "attention" and a.v_mix:
                if self.vmix_first is None:
                    self.vmix_first, vmix_width = i, (a.kv_heads, a.vdim)
                elif (a.kv_heads, a.vdim) != vmix_width:
                    raise ValueError(f"layer {i}: layers that mix values must have values of one size")
            if L.kind == "parallel":
                if L.left.rot_dims % 2 or L.left.rot_dims > L.left.dim:
                    raise ValueError(f"layer {i}: an even rot.dims <= dim")
                self.mem_of.append(n_mem)
                n_mem += 1
            else:
                self.mem_of.append(None)
            if L.kind == "channel_delta":
                c = L.delta
                if c.heads % c.kv_heads or not 1 <= c.conv <= 16:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads, conv 1..16")
                self.delta_of.append(n_delta)
                n_delta += 1
            else:
                self.delta_of.append(None)
        if init:
            self._random_init(seed)

    # ------------------------------------------------------- what the engine allocates for this model
    def _twins(self) -> List[bool]:
        """Per attention: whether the matrix-core kernel runs it (then its values are also cached transposed)."""
        return [S.masked_mfma_ok(H, G, D, V, self.dtype, self.device) for H, G, D, V in self.cache_dims]

    def _widths(self) -> List[Tuple[int, int]]:
        return [(G * D, G * V) for _, G, D, V in self.cache_dims]

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
            if L.kind == "channel_delta":
                j, c = self.delta_of[i], L.delta
                spec[f"dconv{j}"] = (c.conv - 1, 2 * c.kv_heads * c.dim + c.heads * c.vdim)
                spec[f"delta{j}"] = (c.heads, c.dim, c.vdim)
            elif L.kind == "parallel":
                j, b = self.mem_of[i], L.right
                spec[f"mem{j}"] = (b.heads, b.dim, b.vdim)
                spec[f"memn{j}"] = (b.heads, b.dim)
                spec[f"memm{j}"] = (b.heads,)
        return spec

    def workspace_bytes(self, tokens: int) -> int:
        w = self.cfg.hidden
        widest = w
        for L in self.cfg.layers:
            for a in (L.attn, L.left):
                if a is not None:
                    widest = max(widest, 2 * (a.heads * (a.dim + a.vdim) + a.kv_heads * (a.dim + a.vdim)))
            if L.right is not None:
                widest = max(widest, 3 * L.right.heads * (L.right.dim + L.right.vdim))
            if L.delta is not None:
                widest = max(widest, 3 * L.delta.heads * (L.delta.dim + L.delta.vdim))
            widest = max(widest, 2 * L.ff)
        return int(tokens * (3 * w * 4 + widest * 8) + (2 << 30))

    # --------------------------------------------------------------- weights
    def _random_init(self, seed: int) -> None:
        t = random_tensors(self.cfg, seed, self.device)
        self.load_tensors(t.__getitem__)

    def load_tensors(self, get, has=None) -> None:
        """Build the fused device layout from checkpoint tensors (``get(name)`` -> tensor; names of the
        safetensors file: ``embed``, ``l<i>.norm1``, ``l<i>.mix.left.q`` ...)."""
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def put(*names, dtype=dt):
            ts = [get(n) for n in names]
            t = ts[0] if len(ts) == 1 else torch.cat([x.reshape(x.shape[0], -1) if x.dim() > 1 else x for x in ts], 0)
            return t.to(device=dev, dtype=dtype).contiguous()

        def f32(*names):
            return put(*names, dtype=torch.float32)

        def norm(name):   # (alpha, w, b)
            return float(get(name + ".alpha").float().item()), f32(name), f32(name + ".b")

        self.embed = put("embed")
        self.final_norm = norm("final.norm")
        self.lm_head = put("head")
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p = f"l{i}.mix."
            L: Dict[str, object] = {"norm1": norm(f"l{i}.norm1")}
            if spec.kind == "attention":
                a = spec.attn
                L["w_in"] = put(p + "q", p + "k", p + "v", p + "g")            # one fp32-out GEMM: q | k | v | gate
                L["bias"] = f32(p + "q.b", p + "k.b", p + "v.b")
                L["q_w"], L["k_w"] = f32(p + "q.norm"), f32(p + "k.norm")
                L["lam"] = float(get(p + "vmix").float().item()) if a.v_mix and i != self.vmix_first else 0.0
                L["wo"] = put(p + "o")
            elif spec.kind == "parallel":
                a, b = p + "left.", p + "right."
                L["w_in"] = put(a + "q", a + "k", a + "v", b + "q", b + "k", b + "v", b + "g", b + "i", b + "f")
                L["sink"] = f32(a + "sink")
                L["wo_l"] = put(a + "o")
                L["gate_bias"] = f32(b + "i.b", b + "f.b")
                L["mem_norm"] = f32(b + "norm")
                L["wo_r"] = put(b + "o")
            else:
                L["w_qkv"] = put(p + "q", p + "k", p + "v")
                L["conv_w"] = f32(p + "q.conv", p + "k.conv", p + "v.conv")
                L["ra"], L["rg"] = int(get(p + "a1").shape[0]), int(get(p + "g1").shape[0])
                L["w_agb"] = put(p + "a1", p + "g1", p + "b")                   # one fp32-out GEMM
                L["w_a2"], L["w_g2"] = put(p + "a2"), put(p + "g2")
                L["rate"] = torch.exp(f32(p + "A_log")).contiguous()
                L["dt_bias"] = f32(p + "dt_bias")
                L["delta_norm"] = f32(p + "norm")
                L["wo"] = put(p + "o")
            if spec.ff:
                L["norm2"] = norm(f"l{i}.norm2")
                L["w_up"], L["w_down"] = put(f"l{i}.mlp.up"), put(f"l{i}.mlp.down")
            self.layers.append(L)

    def weight_bytes(self) -> int:
        def size(v):
            if isinstance(v, tuple):
                return sum(size(t) for t in v)
            return v.numel() * v.element_size() if isinstance(v, torch.Tensor) else 0
        n = sum(size(t) for L in self.layers for t in L.values())
        return n + sum(size(t) for t in (self.embed, self.lm_head, self.final_norm))

    # -------------------------------------------------------------- forward
    def _lin32(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w.T with an fp32 result (fp32 accumulation either way)."""
        return linear_f32out(x, w) if self.dtype == torch.bfloat16 else linear(x, w)

    def _act(self, x32: torch.Tensor) -> torch.Tensor:
        """A column slice of an fp32 GEMM result as the next GEMM's operand."""
        return x32.to(self.dtype).contiguous()

    def _chunk_attention(self, li: int, h, inp: S.SegStepInputs, kcs, vcs, vts, vmix: dict) -> torch.Tensor:
        L, a = self.layers[li], self.cfg.layers[li].attn
        ci = self.cache_of[li]
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        x = self._lin32(h, L["w_in"])                                  # [T, H D + G D + G V + H] fp32
        keep = other = None
        if a.v_mix:
            if li == self.vmix_first:
                keep = vmix["v"] = torch.empty(x.shape[0], G * V, dtype=torch.float32, device=x.device)
            else:
                other = vmix["v"]
        q = S.attn_prep(x[:, :H * D + G * (D + V)], L["bias"], H, G, D, V, inp.positions, inp.slots, kcs[ci], vcs[ci], self.dtype, norm=True,
                        q_w=L["q_w"], k_w=L["k_w"], eps=self.cfg.norm_eps, lam=L["lam"], v_other=other, v_keep=keep,
                        vt=vts[ci])
        o = S.masked_attention(q, H, G, D, V, kcs[ci], vcs[ci], inp.seg, a.scale, softcap=a.softcap, chunk=a.chunk,
                               gate=x[:, H * D + G * (D + V):], vt=vts[ci])
        return self._lin32(o, L["wo"])

    def _parallel(self, li: int, h, inp: S.SegStepInputs, kcs, vcs, vts, states):
        L, spec = self.layers[li], self.cfg.layers[li]
        a, b = spec.left, spec.right
        ci, j = self.cache_of[li], self.mem_of[li]
        H, G, D, V = a.heads, a.kv_heads, a.dim, a.vdim
        nl = H * D + G * (D + V)
        x = self._lin32(h, L["w_in"])                                  # left q | k | v, right q | k | v | g | i | f
        q = S.attn_prep(x[:, :nl], None, H, G, D, V, inp.positions, inp.slots, kcs[ci], vcs[ci], self.dtype, norm=True,
                        eps=self.cfg.norm_eps, rot_dims=a.rot_dims, rot_base=a.rot_base, vt=vts[ci])
        ol = S.masked_attention(q, H, G, D, V, kcs[ci], vcs[ci], inp.seg, a.scale, window=a.window,
                                keep_first=a.keep_first, sink=L["sink"], vt=vts[ci])
        xr = x[:, nl:]
        hd, hv = b.heads * b.dim, b.heads * b.vdim
        o, mul = S.matrix_memory(xr, b.heads, b.dim, b.vdim, L["gate_bias"], b.gate_cap, states[f"mem{j}"],
                                 states[f"memn{j}"], states[f"memm{j}"], inp.seg, defer_scale=True)
        orr = S.head_norm_gate(o, xr[:, 2 * hd + hv:2 * hd + 2 * hv], L["mem_norm"], b.heads, b.vdim,
                               self.cfg.norm_eps, self.dtype, mul=mul)
        return self._lin32(ol, L["wo_l"]), self._lin32(orr, L["wo_r"])

    def _delta(self, li: int, h, inp: S.SegStepInputs, states) -> torch.Tensor:
        L, c = self.layers[li], self.cfg.layers[li].delta
        j, ra, rg = self.delta_of[li], L["ra"], L["rg"]
        qkv = linear(h, L["w_qkv"])                                    # [T, 2 G D + H V]
        qkv = S.short_conv(qkv, L["conv_w"], None, states[f"dconv{j}"], inp.seg, act=True)
        agb = self._lin32(h, L["w_agb"])                               # [T, ra + rg + H] fp32
        dec = self._lin32(self._act(agb[:, :ra]), L["w_a2"])           # [T, H D] fp32, before bias and softplus
        gate = self._lin32(self._act(agb[:, ra:ra + rg]), L["w_g2"])   # [T, H V] fp32, before the sigmoid
        o = S.gated_delta(qkv, c.heads, c.kv_heads, c.dim, c.vdim, dec, L["rate"], L["dt_bias"], agb[:, ra + rg:],
                          states[f"delta{j}"], inp.seg)
        o = S.head_norm_gate(o, gate, L["delta_norm"], c.heads, c.vdim, self.cfg.norm_eps, self.dtype)
        return self._lin32(o, L["wo"])

    def forward(self, inp: S.SegStepInputs, kcs: List[torch.Tensor], vcs: List[torch.Tensor],
                vts: List[Optional[torch.Tensor]], states: Dict[str, torch.Tensor],
                layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits [len(logits_idx), vocab] fp32.  ``kcs`` / ``vcs``: the paged keys and values of every
        attention (``vts``: the values' transposed twins, or None); ``states``: the per-slot tensors of
        :meth:`state_spec`.  ``layers_out`` (debugging): receives a copy of the residual after every layer."""
        cfg, dt = self.cfg, self.dtype
        T, W, nl = inp.input_ids.shape[0], cfg.hidden, cfg.n_layers
        x = torch.empty(T, W, dtype=torch.float32, device=self.device)
        first = self.layers[0]["norm1"] if nl else (1.0, None, None)
        h = N.embed_scale_dyt(inp.input_ids, self.embed, cfg.embed_scale, x, *first, out_dtype=dt)
        vmix: dict = {}
        for li, (spec, L) in enumerate(zip(cfg.layers, self.layers)):
            nxt = self.layers[li + 1]["norm1"] if li + 1 < nl else (1.0, None, None)   # the final norm: wanted rows only
            after = L["norm2"] if spec.ff else nxt
            if spec.kind == "attention":
                h = N.add_dyt(x, self._chunk_attention(li, h, inp, kcs, vcs, vts, vmix), 1.0, None, 1.0, *after,
                              out_dtype=dt)
            elif spec.kind == "parallel":
                yl, yr = self._parallel(li, h, inp, kcs, vcs, vts, states)
                h = N.add_dyt(x, yl, spec.left_scale, yr, spec.right_scale, *after, out_dtype=dt)
            else:
                h = N.add_dyt(x, self._delta(li, h, inp, states), 1.0, None, 1.0, *after, out_dtype=dt)
            if spec.ff:
                y = self._lin32(N.relu_sq(linear(h, L["w_up"])), L["w_down"])
                h = N.add_dyt(x, y, 1.0, None, 1.0, *nxt, out_dtype=dt)
            if layers_out is not None:
                layers_out.append(x.clone())
        xr = x.index_select(0, inp.logits_idx).contiguous()
        h = N.add_dyt(xr, None, 1.0, None, 1.0, *self.final_norm, out_dtype=dt)
        return self._lin32(h, self.lm_head)


def random_tensors(cfg: LizesunConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
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

    t: Dict[str, torch.Tensor] = {"embed": rnd(cfg.vocab_size, W, std=1.0 / max(cfg.embed_scale, 1e-6)),
                                  "head": lin(cfg.vocab_size, W)}

    def norm(name):
        t[name] = rnd(W, std=0.1, mean=1.0)
        t[name + ".b"] = rnd(W, std=0.05)
        t[name + ".alpha"] = rnd((), std=0.05, mean=0.7)

    norm("final.norm")
    for i, L in enumerate(cfg.layers):
        p = f"l{i}.mix."
        norm(f"l{i}.norm1")
        if L.kind == "attention":
            a = L.attn
            t[p + "q"], t[p + "k"] = lin(a.heads * a.dim, W), lin(a.kv_heads * a.dim, W)
            t[p + "v"], t[p + "o"] = lin(a.kv_heads * a.vdim, W), lin(W, a.heads * a.vdim)
            t[p + "q.b"], t[p + "k.b"] = rnd(a.heads * a.dim, std=0.1), rnd(a.kv_heads * a.dim, std=0.1)
            t[p + "v.b"] = rnd(a.kv_heads * a.vdim, std=0.1)
            t[p + "q.norm"], t[p + "k.norm"] = rnd(a.dim, std=0.2, mean=1.5), rnd(a.dim, std=0.2, mean=1.5)
            t[p + "vmix"] = rnd((), std=0.05, mean=0.3)
            t[p + "g"] = lin(a.heads, W)
        elif L.kind == "parallel":
            a, b = L.left, L.right
            q, m = p + "left.", p + "right."
            t[q + "q"], t[q + "k"] = lin(a.heads * a.dim, W), lin(a.kv_heads * a.dim, W)
            t[q + "v"], t[q + "o"] = lin(a.kv_heads * a.vdim, W), lin(W, a.heads * a.vdim)
            t[q + "sink"] = rnd(a.heads, std=1.0)
            t[m + "q"], t[m + "k"] = lin(b.heads * b.dim, W), lin(b.heads * b.dim, W)
            t[m + "v"], t[m + "g"] = lin(b.heads * b.vdim, W), lin(b.heads * b.vdim, W)
            t[m + "o"] = lin(W, b.heads * b.vdim)
            t[m + "norm"] = rnd(b.heads * b.vdim, std=0.1, mean=1.0)
            t[m + "i"], t[m + "f"] = lin(b.heads, W, 2.0), lin(b.heads, W, 2.0)
            t[m + "i.b"], t[m + "f.b"] = rnd(b.heads, std=0.5), rnd(b.heads, std=0.5, mean=2.0)
        else:
            c = L.delta
            t[p + "q"], t[p + "k"] = lin(c.kv_heads * c.dim, W), lin(c.kv_heads * c.dim, W)
            t[p + "v"], t[p + "o"] = lin(c.heads * c.vdim, W), lin(W, c.heads * c.vdim)
            for n_, ch in (("q", c.kv_heads * c.dim), ("k", c.kv_heads * c.dim), ("v", c.heads * c.vdim)):
                t[p + n_ + ".conv"] = rnd(ch, c.conv, std=0.5)
            t[p + "b"] = lin(c.heads, W)
            t[p + "A_log"] = rnd(c.heads, std=0.5, mean=-1.0)
            t[p + "norm"] = rnd(c.vdim, std=0.1, mean=1.0)
            t[p + "a1"], t[p + "a2"] = lin(c.a_rank, W), lin(c.heads * c.dim, c.a_rank)
            t[p + "dt_bias"] = rnd(c.heads * c.dim, std=0.5, mean=-1.0)
            t[p + "g1"], t[p + "g2"] = lin(c.g_rank, W), lin(c.heads * c.vdim, c.g_rank)
        if L.ff:
            norm(f"l{i}.norm2")
            t[f"l{i}.mlp.up"], t[f"l{i}.mlp.down"] = lin(L.ff, W), lin(W, L.ff, 0.5)
    return t


def load_checkpoint(path: str, device, dtype, pc=None) -> LizesunModel:
    """A folder with config.json and model.safetensors (bfloat16 weights) -> the model on ``device``."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = LizesunConfig.from_json(json.load(f), name=os.path.basename(os.path.normpath(path)) or "lizesun")
    model = LizesunModel(cfg, device, dtype, pc, init=False)
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as h:
        model.load_tensors(h.get_tensor, set(h.keys()).__contains__)
    return model


def save_checkpoint(cfg: LizesunConfig, tensors: Dict[str, torch.Tensor], path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) in the layout :func:`load_checkpoint` reads."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
