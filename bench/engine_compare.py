"""Engine-level prefill / decode throughput of several model configurations side by side
(``python bench.py --engine-compare nulazen-2k,llama-2k-4l``): random weights, token-id
prompts, the engine's own scheduler, graphs and sampler.

Per model:  prefill tok/s = P / (time of one P-token prompt to its first token), for
each P; decode tok/s = B * N / (time of B sequences generating 1 + N tokens minus the
time of the same B prompts generating 1), for each batch B at a context of ``ctx``
tokens.  Best of ``reps`` runs; every run uses fresh random prompts and prefix caching
is off.  One JSON line per measurement, then a table on stderr.
"""
from __future__ import annotations

import json
import sys
import time

import numpy as np


def _prompts(rng, n, length, vocab):
    return [rng.integers(1, vocab, size=length).tolist() for _ in range(n)]


def measure(model: str, prompt_lens, batches, gen: int, ctx: int, reps: int, dtype: str = "bfloat16"):
    import torch

    from fasttalk_llm_microservice_amd.engine.config import EngineConfig
    from fasttalk_llm_microservice_amd.engine.engine import LLMEngine
    from fasttalk_llm_microservice_amd.engine.sampling_params import SamplingParams

    max_len = max(max(prompt_lens), ctx + gen) + 64
    eng = LLMEngine(EngineConfig(model=model, device="cuda", dtype=dtype, max_model_len=max_len,
                                 max_num_seqs=max(batches), max_num_batched_tokens=max(max(prompt_lens), 8192),
                                 num_kv_blocks=(max(batches) * (ctx + gen + 64) + max(prompt_lens)) // 16 + 64,
                                 enable_prefix_caching=False, prefill_chunk=0, swap_space_gb=0.0))
    vocab = eng.model_cfg.vocab_size
    rng = np.random.default_rng(0)
    eng.runner.warmup(list(batches))
    out = []

    def timed(prompts, n_new):
        sp = SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        res = eng.generate(prompts, sp)
        torch.cuda.synchronize()
        assert all(len(r) == n_new for r in res)
        return time.perf_counter() - t0

    timed(_prompts(rng, 1, 64, vocab), 4)   # lazy initialisation
    for p in prompt_lens:
        best = min(timed(_prompts(rng, 1, p, vocab), 1) for _ in range(reps))
        out.append({"model": model, "phase": "prefill", "tokens": p, "ms": round(1e3 * best, 3),
                    "tok_s": round(p / best, 1)})
        print(json.dumps(out[-1]), flush=True)
    for b in batches:
        t1 = min(timed(_prompts(rng, b, ctx, vocab), 1) for _ in range(reps))
        t2 = min(timed(_prompts(rng, b, ctx, vocab), 1 + gen) for _ in range(reps))
        dt = max(t2 - t1, 1e-9)
        out.append({"model": model, "phase": "decode", "batch": b, "ctx": ctx, "new_tokens": gen,
                    "ms_per_step": round(1e3 * dt / gen, 3), "tok_s": round(b * gen / dt, 1),
                    "graph_replays": eng.runner.stats.get("graph_replays", 0)})
        print(json.dumps(out[-1]), flush=True)
    eng.shutdown() if hasattr(eng, "shutdown") else None
    del eng
    torch.cuda.empty_cache()
    return out


def main(models, prompt_lens=(512, 2048, 4096), batches=(1, 8, 32), gen=64, ctx=512, reps=2,
         dtype="bfloat16"):
    rows = []
    for m in models:
        rows += measure(m, list(prompt_lens), list(batches), gen, ctx, reps, dtype)
    w = sys.stderr.write
    w("\n%-16s %-8s %10s %12s %12s\n" % ("model", "phase", "size", "ms", "tok/s"))
    for r in rows:
        size = r["tokens"] if r["phase"] == "prefill" else r["batch"]
        ms = r["ms"] if r["phase"] == "prefill" else r["ms_per_step"]
        w("%-16s %-8s %10d %12.3f %12.1f\n" % (r["model"], r["phase"], size, ms, r["tok_s"]))
    return rows
