"""Shared cases of the Bagasun tests: small configurations with random weights, run
through the framework's engine (scheduler, block / state-slot pools, model runner,
kernels or the CPU backend) and compared with tests/bagasun_oracle.py.

None of the configurations is a real model's; they vary what a single model would
leave equal or 1 (heads vs kv heads, key vs value sizes, rotary dims vs key size, with
and without frequency scaling, one group, one norm group, one tap, windows shorter than
a page and longer than the prompt, a window of 1, state sizes that are no multiple of
8, an attention layer first, a layer without feed-forward, borrowed weights)."""
import copy
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import bagasun_oracle as O  # noqa: E402

from fasttalk_llm_microservice_amd.engine.config import EngineConfig  # noqa: E402
from fasttalk_llm_microservice_amd.engine.engine import LLMEngine  # noqa: E402
from fasttalk_llm_microservice_amd.models import bagasun as B  # noqa: E402


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _sig(heads, kv, dim, vdim, window, scale):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale}


def _dif(heads, kv, dim, vdim, window, scale, diff, dims, base, scaling=None):
    rot = {"dims": dims, "base": base}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale,
            "diff": diff, "rot": rot}


def _ff(n):
    return {"kind": "dense", "ff": n}


CONFIGS = {
    # every mixer, then two of them again on borrowed weights; windows off page borders
    "a": {"architecture": "Bagasun", "vocab": 101, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
          "layers": [
              {"type": "mamba2", "mixer": _ssm(4, 8, 12, 2, 3, 2), "mlp": _ff(96)},
              {"type": "attention_2", "mixer": _dif(4, 2, 8, 12, 19, 0.3, 0.7, 4, 50.0, (3.0, 1.0, 3.0, 64)), "mlp": _ff(80)},
              {"type": "attention", "mixer": _sig(3, 1, 16, 10, 7, 0.2), "mlp": None},
              {"type": "mamba2", "mixer": _ssm(4, 8, 12, 2, 3, 2), "mlp": _ff(96), "weights_of": 0},
              {"type": "attention", "mixer": _sig(3, 1, 16, 10, 7, 0.2), "mlp": None, "weights_of": 2}]},
    # attention first; kv heads = heads, one group, one norm group, one tap, full rotary dims
    # without scaling, a window of one token and a window longer than any prompt here
    "b": {"architecture": "Bagasun", "vocab": 77, "width": 48, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
          "layers": [
              {"type": "attention", "mixer": _sig(2, 2, 12, 6, 1, 0.25), "mlp": _ff(50)},
              {"type": "mamba2", "mixer": _ssm(3, 40, 5, 1, 1, 1), "mlp": None},
              {"type": "attention_2", "mixer": _dif(2, 2, 6, 6, 400, 0.4, 0.2, 6, 10000.0), "mlp": _ff(64)}]},
    # window = page size and page size + 1, a value size over 64, two taps
    "c": {"architecture": "Bagasun", "vocab": 64, "width": 40, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.5},
          "layers": [
              {"type": "attention_2", "mixer": _dif(3, 1, 10, 72, 16, 0.3, 0.5, 2, 100.0, (2.0, 1.0, 2.0, 32)), "mlp": _ff(64)},
              {"type": "mamba2", "mixer": _ssm(2, 12, 20, 2, 2, 4), "mlp": _ff(56)},
              {"type": "attention", "mixer": _sig(4, 2, 8, 8, 17, 0.35), "mlp": _ff(48)},
              {"type": "attention_2", "mixer": _dif(3, 1, 10, 72, 16, 0.3, 0.5, 2, 100.0, (2.0, 1.0, 2.0, 32)), "mlp": _ff(64),
               "weights_of": 0}]},
}


def make_model(name, seed, tmp_path, tweak=None):
    """(checkpoint dir, config dict, fp32 tensors of the bf16 weights)."""
    cfg = copy.deepcopy(CONFIGS[name])
    bcfg = B.config_from_dict(cfg, name)
    t = B.random_tensors(bcfg, seed, torch.bfloat16)
    if tweak:
        tweak(t)
    d = os.path.join(str(tmp_path), f"{name}-{seed}")
    B.save_checkpoint(bcfg, t, d)
    return d, cfg, {k: v.float() for k, v in t.items()}


def make_engine(ckpt, device, dtype="float32", pages=64, seqs=4, page=16, graphs=False):
    """``graphs``: decode steps replay captured graphs and are queued ahead (the
    serving configuration on a GPU); otherwise every step runs eagerly."""
    return LLMEngine(EngineConfig(model=ckpt, weights=ckpt, device=device, dtype=dtype, num_kv_blocks=pages,
                                  block_size=page, max_num_seqs=seqs, max_model_len=pages * page,
                                  max_num_batched_tokens=pages * page, enforce_eager=not graphs,
                                  async_output=graphs, swap_space_gb=0.0))


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay(eng, reqs, schedule):
    """reqs: id -> tokens.  schedule: steps, each a list of (id, count).  Every position's
    logits are asked for.  Returns id -> [T, vocab] tensor."""
    at = {i: 0 for i in reqs}
    rows = {i: [] for i in reqs}
    for step in schedule:
        entries, end = [], []
        for i, n in step:
            lo, hi = at[i], at[i] + n
            entries.append((i, reqs[i][lo:hi], list(range(n))))
            at[i] = hi
            if hi == len(reqs[i]):
                end.append(i)
        lg = torch.from_numpy(eng.replay_step(entries, end).copy())
        k = 0
        for i, n in step:
            rows[i].append(lg[k:k + n])
            k += n
    return {i: torch.cat(v) for i, v in rows.items()}


def close(got, want, dtype="float32"):
    if dtype == "float32":
        torch.testing.assert_close(got, want, rtol=2e-4, atol=3e-4)
        return
    # bf16: rounding differs from the fp32 oracle everywhere
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert err.median() < 0.08 and err.max() < 0.3, err


def oracle(cfg, P, toks):
    return O.forward(cfg, P, toks)


def portions(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out
