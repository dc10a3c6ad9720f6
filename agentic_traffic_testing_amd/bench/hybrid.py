"""Prefill and decode throughput of the hybrid decoders (Ledazen, Soselix, Semezen, Lovapel) next to the
models of the same layer geometry - Llama, and for Soselix and Semezen also the closest earlier
hybrid family (softmax + recurrent mixers on the same cache and kernels) - through the serving
engine (scheduler, paged cache / state slots, kernels).

Random-init weights, synthetic token ids.  Per model and shape:
  prefill  - B prompts of P tokens admitted together, one generated token each: prompt tok/s
  decode   - the same B sequences generating N more tokens: generated tok/s
``python bench.py --hybrid [ledazen|soselix|semezen|lovapel]`` prints one JSON line per measurement.
"""
from __future__ import annotations

import json
import time

import numpy as np

PAIRS = (("ledazen-small", "small"), ("ledazen-3b-slice", "llama-3b-slice"),
         ("ledazen-8b-slice", "llama-8b-slice"))
SOSELIX = (("soselix-small", "ledazen-small", "small"),
           ("soselix-3b-slice", "ledazen-3b-slice", "llama-3b-slice"),
           ("soselix-8b-slice", "ledazen-8b-slice", "llama-8b-slice"))
SEMEZEN = (("semezen-small", "soselix-small", "small"),
           ("semezen-3b-slice", "soselix-3b-slice", "llama-3b-slice"),
           ("semezen-8b-slice", "soselix-8b-slice", "llama-8b-slice"))
LOVAPEL = (("lovapel-small", "semezen-small", "small"),
           ("lovapel-3b-slice", "semezen-3b-slice", "llama-3b-slice"),
           ("lovapel-8b-slice", "semezen-8b-slice", "llama-8b-slice"))
FAMILIES = {"ledazen": PAIRS, "soselix": SOSELIX, "semezen": SEMEZEN, "lovapel": LOVAPEL}


def _engine(model: str, device: str, dtype: str, max_len: int, seqs: int, budget: int):
    from ..config import EngineConfig
    from ..engine.llm_engine import LLMEngine

    cfg = EngineConfig(model=model, device=device, dtype=dtype, max_model_len=max_len,
                       max_num_seqs=seqs, max_num_batched_tokens=budget,
                       num_kv_blocks=(seqs + 1) * (max_len // 16 + 1), enable_prefix_caching=False,
                       startup_warmup=False, load_format="dummy")
    return LLMEngine(cfg)


def _sync(device):
    if device.startswith("cuda"):
        import torch

        torch.cuda.synchronize()


def measure(model: str, device: str = "cuda", dtype: str = "bfloat16", prompt: int = 2048,
            batch: int = 4, gen: int = 64, repeats: int = 3) -> dict:
    from ..engine.sequence import SamplingParams

    eng = _engine(model, device, dtype, prompt + gen + 64, batch, max(2048, prompt * batch))
    vocab = eng.model_cfg.vocab_size
    rng = np.random.default_rng(0)

    def prompts():
        return [rng.integers(1, min(vocab, 30000), prompt).tolist() for _ in range(batch)]

    one = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
    many = SamplingParams(temperature=0.0, max_tokens=gen + 1, ignore_eos=True)
    eng.generate(prompts(), many)            # warm-up: code objects, library heuristics, graphs
    t_pre, t_all = [], []
    for _ in range(repeats):
        p = prompts()
        _sync(device)
        t0 = time.perf_counter()
        eng.generate(p, one)
        _sync(device)
        t_pre.append(time.perf_counter() - t0)
        p = prompts()
        _sync(device)
        t0 = time.perf_counter()
        eng.generate(p, many)
        _sync(device)
        t_all.append(time.perf_counter() - t0)
    pre, dec = min(t_pre), max(1e-9, min(t_all) - min(t_pre))
    return {"model": model, "dtype": dtype, "batch": batch, "prompt_tokens": prompt,
            "generated": gen, "prefill_tok_s": round(batch * prompt / pre, 1),
            "decode_tok_s": round(batch * gen / dec, 1), "prefill_ms": round(pre * 1e3, 2),
            "decode_ms_per_step": round(dec / gen * 1e3, 3),
            "weight_bytes": eng.runner.model.weight_bytes()}


def run(device: str = "cuda", dtype: str = "bfloat16", pairs=PAIRS, shapes=None, out=print):
    shapes = shapes or ((2048, 4, 64), (512, 16, 64), (1024, 1, 64))
    rows = []
    for group in pairs:
        for prompt, batch, gen in shapes:
            for model in group:
                r = measure(model, device, dtype, prompt, batch, gen)
                rows.append(r)
                out(json.dumps(r))
    return rows
