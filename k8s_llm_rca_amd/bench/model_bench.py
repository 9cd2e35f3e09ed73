"""Prefill and decode throughput of one or more model presets, side by side
(``python bench.py --model-throughput zasapel-1b,ligipel-1b,mixtral-1b``, ``... lizesun-1b,llama-1b``,
``... pumozen-1b,ligipel-1b``).

Random weights, one GPU, the engine's own step (``LLMEngine.feed``: given
tokens, no sampling): a prefill step is ``batch`` prompts of ``seq`` tokens in
one forward, a decode step one token for each of ``batch`` sequences that hold
``ctx`` cached tokens.  Prints ONE JSON line with tokens/s per model and shape;
the headline benchmark (no flag) is untouched.
"""
from __future__ import annotations

import argparse
import json
import time
from typing import Any, Dict, List

import torch

# presets made for this comparison: the existing architectures at the new ones' layer sizes
EXTRA = {
    "mixtral-1b": ("mixtral-8x7b", dict(vocab_size=32768, hidden=2048, n_layers=12, n_heads=16, n_kv_heads=2,
                                        intermediate=2048, max_position=32768)),
    "llama-1b": ("llama3-8b", dict(vocab_size=32768, hidden=2048, n_layers=12, n_heads=16, n_kv_heads=2,
                                   intermediate=8192, max_position=32768)),
}


def _engine(name: str, tokens: int):
    from ..engine.engine import EngineConfig, LLMEngine
    model, over = EXTRA.get(name, (name, {}))
    nb = tokens // 64 + 64
    return LLMEngine(EngineConfig(model=model, model_overrides=over, device="cuda", dtype=torch.bfloat16,
                                  num_blocks=nb, block_size=64, max_batch_tokens=1 << 17, max_context=1 << 16,
                                  max_decode_seqs=1024, state_slots=1024, use_graphs=False, prefix_sharing=False))


def _time(fn, warmup: int, steps: int) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_model(name: str, shapes: List[tuple], steps: int, warmup: int) -> Dict[str, Any]:
    out: Dict[str, Any] = {}
    total = max(b * (s + steps + warmup + 8) for b, s in shapes) + 4096
    eng = _engine(name, total)
    out["weights_gb"] = round(eng.model.weight_bytes() / 2 ** 30, 2)
    g = torch.Generator().manual_seed(0)
    vocab = eng.mc.vocab_size
    for b, s in shapes:
        toks = torch.randint(0, vocab, (b, s + steps + warmup + 8), generator=g).tolist()

        def prefill():
            sids = [eng.new_sequence() for _ in range(b)]
            eng.feed([(sid, toks[i][:s], []) for i, sid in enumerate(sids)])
            return sids

        def prefill_and_free():
            for sid in prefill():
                eng.release_sequence(sid)

        dt_p = _time(prefill_and_free, warmup, steps)
        sids = prefill()
        at = [s]

        def decode():
            eng.feed([(sid, [toks[i][at[0]]], [0]) for i, sid in enumerate(sids)])
            at[0] += 1

        dt_d = _time(decode, warmup, steps)
        for sid in sids:
            eng.release_sequence(sid)
        out[f"b{b}_s{s}"] = {"prefill_tok_s": round(b * s / dt_p), "prefill_ms": round(dt_p * 1e3, 3),
                             "decode_tok_s": round(b / dt_d), "decode_ms": round(dt_d * 1e3, 3)}
    return out


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--model-throughput", required=True, help="comma-separated presets")
    p.add_argument("--shapes", default="1x2048,8x2048,64x512", help="batch x tokens, comma-separated")
    p.add_argument("--steps", type=int, default=10)
    p.add_argument("--warmup", type=int, default=3)
    a, _ = p.parse_known_args(argv)
    shapes = [tuple(int(v) for v in s.split("x")) for s in a.shapes.split(",")]
    res = {"metric": "model_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
           "steps": a.steps, "warmup": a.warmup, "models": {}}
    for name in a.model_throughput.split(","):
        res["models"][name] = bench_model(name, shapes, a.steps, a.warmup)
        torch.cuda.empty_cache()
    print(json.dumps(res), flush=True)
    return 0
