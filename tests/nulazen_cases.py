"""Shared cases of the Nulazen tests: small configurations with random weights, run
through the framework's engine (scheduler, block / state-slot pools, model runner,
kernels or the CPU backend) and compared with tests/nulazen_oracle.py.

None of the configurations is a real model's; they vary what a single model would
leave equal (heads vs kv heads, key vs value sizes, rotary dims vs rotated size, one
group, top 1, one tap, a loop from layer 0, no loop, no token-side input, a layer
without feed-forward)."""
import copy
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import nulazen_oracle as O  # noqa: E402

from fasttalk_llm_microservice_amd.engine.config import EngineConfig  # noqa: E402
from fasttalk_llm_microservice_amd.engine.engine import LLMEngine  # noqa: E402
from fasttalk_llm_microservice_amd.models import nulazen as N  # noqa: E402


def _delta(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _latent(heads, dim, rot_dim, dims, vdim, rank, scale, base=100.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
            "scale": scale, "rot": {"base": base, "dims": dims}}


def _moe(e, top, ff, limit, groups=None, shared=None):
    r = {"experts": e, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


CONFIGS = {
    # loop from layer 0, partial rotary dims, grouped routing + shared expert, a layer without ff
    "a": {"architecture": "Nulazen", "vocab": 101, "width": 64, "norm": {"eps": 1e-5},
          "layers": [
              {"type": "channel_delta", "mixer": _delta(4, 2, 8, 12, 3), "mlp": {"kind": "dense", "ff": 96}},
              {"type": "latent_attention", "mixer": _latent(3, 8, 6, 4, 10, 20, 0.3),
               "mlp": _moe(6, 2, 24, 1.2, groups=(3, 2), shared=(40, 0.9))},
              {"type": "channel_delta", "mixer": _delta(2, 2, 16, 8, 2), "mlp": None}],
          "loop": {"start": 0, "stop": 2, "times": 2}, "token_side": {"dim": 5}},
    # no loop, no token side, latent first, top 1, one group, no shared expert, one tap, one kv head
    "b": {"architecture": "Nulazen", "vocab": 77, "width": 48, "norm": {"eps": 1e-6},
          "layers": [
              {"type": "latent_attention", "mixer": _latent(2, 12, 4, 4, 6, 33, 0.25, base=10000.0),
               "mlp": _moe(5, 1, 16, 2.5)},
              {"type": "channel_delta", "mixer": _delta(3, 1, 10, 7, 1), "mlp": {"kind": "dense", "ff": 50}}]},
    # a looped latent layer (each pass its own cache) next to a looped delta layer
    "c": {"architecture": "Nulazen", "vocab": 64, "width": 40, "norm": {"eps": 1e-5},
          "layers": [
              {"type": "channel_delta", "mixer": _delta(2, 1, 12, 12, 4), "mlp": {"kind": "dense", "ff": 64}},
              {"type": "latent_attention", "mixer": _latent(4, 6, 8, 8, 6, 16, 0.4),
               "mlp": _moe(8, 3, 12, 1.0, groups=(2, 1), shared=(16, 2.0))},
              {"type": "channel_delta", "mixer": _delta(5, 5, 4, 6, 5), "mlp": _moe(4, 4, 8, 3.0)}],
          "loop": {"start": 1, "stop": 3, "times": 3}, "token_side": {"dim": 3}},
    # dense feed-forwards only: bf16 runs are compared with the fp32 oracle on this one (a
    # routing choice that flips under bf16 rounding changes a row's output entirely, so
    # bf16 expert layers are checked per mechanism instead)
    "d": {"architecture": "Nulazen", "vocab": 90, "width": 64, "norm": {"eps": 1e-5},
          "layers": [
              {"type": "channel_delta", "mixer": _delta(4, 2, 16, 8, 3), "mlp": {"kind": "dense", "ff": 80}},
              {"type": "latent_attention", "mixer": _latent(2, 16, 8, 8, 12, 24, 0.2), "mlp": {"kind": "dense", "ff": 72}},
              {"type": "channel_delta", "mixer": _delta(2, 2, 8, 16, 2), "mlp": None}],
          "loop": {"start": 1, "stop": 3, "times": 2}, "token_side": {"dim": 4}},
}


def make_model(name, seed, tmp_path, tweak=None):
    """(checkpoint dir, config dict, fp32 tensors of the bf16 weights)."""
    cfg = copy.deepcopy(CONFIGS[name])
    ncfg = N.config_from_dict(cfg, name)
    t = N.random_tensors(ncfg, seed, torch.bfloat16, low_rank=6)
    if tweak:
        tweak(t)
    d = os.path.join(str(tmp_path), f"{name}-{seed}")
    N.save_checkpoint(ncfg, t, d)
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
    # bf16: rounding differs from the fp32 oracle everywhere, and a routing choice can flip
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert err.median() < 0.1 and err.max() < 0.4, err


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
