"""Nulazen: a decoder-only model that stacks, in an order its configuration gives,
latent-attention layers (paged latent cache) and channel-decay delta-rule layers
(recurrent state slots), each followed by a dense or mixture-of-experts feed-forward
and a per-layer token-side input, with a span of layers that is run several times in
a row on shared weights.

Per layer, with an fp32 residual x:  x += norm1b(mixer(norm1 x));
x += norm2b(ff(norm2 x)) (if the layer has a feed-forward);
x += rms(side(x, token)) * side.norm (if the model has token-side inputs).
Looped span: layers start..stop-1 run ``times`` times; before each pass
``loop.step[pass]`` is added to x, and every pass owns its cache / state.

Every size comes from ``config.json`` (keys: vocab, width, norm.eps, layers[].type /
mixer / mlp, loop, token_side) or from tensor shapes.  Tensor names: embed, head,
final.norm, loop.step, side.embed, l<i>.{norm1,norm1b,norm2,norm2b}, l<i>.mix.*,
l<i>.mlp.*, l<i>.side.*.
"""
from __future__ import annotations

import dataclasses
import logging
import os
from typing import Dict, List, Optional, Tuple

import torch

from ..parallel.comm import SINGLE, TPComm
from .mixers import ChannelDelta, DenseFF, LatentAttention, MoEFF, TokenSide
from .registry import Architecture, register
from .stacked import StackedCache, StackedLayer, StackedModel

log = logging.getLogger(__name__)

LATENT, DELTA = "latent_attention", "channel_delta"


@dataclasses.dataclass(frozen=True)
class NulazenConfig:
    name: str
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    layers: tuple                      # per layer: dict(type=, mixer=, mlp=)
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)
    side_dim: int = 0                  # 0: no token-side input
    max_position_embeddings: int = 1 << 17
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = False
    architecture = "nulazen"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> List[Tuple[int, Optional[int]]]:
        """Execution order: (layer index, index of the loop.step row added right
        before it or None)."""
        n = len(self.layers)
        if not self.loop:
            return [(i, None) for i in range(n)]
        a, b, times = self.loop
        out = [(i, None) for i in range(a)]
        for t in range(times):
            out += [(i, t if i == a else None) for i in range(a, b)]
        return out + [(i, None) for i in range(b, n)]

    def num_params(self) -> int:
        return sum(int(torch.Size(s).numel()) for s in tensor_shapes(self).values())

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum((self.layers[i]["mixer"]["kv_rank"] + self.layers[i]["mixer"]["rot_dim"])
                   * dtype_bytes for i, _ in self.runs() if self.layers[i]["type"] == LATENT)


def config_from_dict(c: dict, name: str = "nulazen") -> NulazenConfig:
    layers = []
    for l in c["layers"]:
        if l["type"] not in (LATENT, DELTA):
            raise ValueError(f"unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp["kind"] not in ("dense", "moe"):
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        layers.append({"type": l["type"], "mixer": dict(l["mixer"]), "mlp": mlp})
    lp = c.get("loop")
    loop = None
    if lp and int(lp.get("times", 1)) >= 1 and lp["stop"] > lp["start"]:
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not 0 <= loop[0] < loop[1] <= len(layers):
            raise ValueError("loop span outside the layer list")
    norm = c.get("norm", {})
    if norm.get("kind", "rms") != "rms":
        raise ValueError(f"unknown norm kind {norm.get('kind')!r}")
    side = c.get("token_side") or {}
    return NulazenConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                         rms_norm_eps=float(norm.get("eps", 1e-5)), layers=tuple(layers), loop=loop,
                         side_dim=int(side.get("dim", 0)),
                         max_position_embeddings=int(c.get("max_positions", 1 << 17)))


def config_to_dict(cfg: NulazenConfig) -> dict:
    c = {"architecture": "Nulazen", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
         "norm": {"eps": cfg.rms_norm_eps}, "layers": [dict(l) for l in cfg.layers]}
    if cfg.loop:
        c["loop"] = {"start": cfg.loop[0], "stop": cfg.loop[1], "times": cfg.loop[2]}
    if cfg.side_dim:
        c["token_side"] = {"dim": cfg.side_dim}
    return c


def tensor_shapes(cfg: NulazenConfig, low_rank: int = 0) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration (random init, tests).
    ``low_rank``: inner size of the decay / output-gate projections (0: width / 16)."""
    w, v = cfg.hidden_size, cfg.vocab_size
    t: Dict[str, tuple] = {"embed": (v, w), "head": (v, w), "final.norm": (w,)}
    if cfg.loop:
        t["loop.step"] = (cfg.loop[2], w)
    if cfg.side_dim:
        t["side.embed"] = (v, cfg.side_dim * len(cfg.layers))
    lr = low_rank or max(8, w // 16)
    for i, l in enumerate(cfg.layers):
        p, m = f"l{i}.", l["mixer"]
        t[p + "norm1"] = t[p + "norm1b"] = (w,)
        if l["type"] == LATENT:
            h, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            t.update({p + "mix.q": (h * (dn + dr), w), p + "mix.dkv": (r + dr, w),
                      p + "mix.dkv.norm": (r,), p + "mix.uk": (h * dn, r), p + "mix.uv": (h * dv, r),
                      p + "mix.o": (w, h * dv)})
        else:
            h, kh, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for n, rows in (("q", kh * dk), ("k", kh * dk), ("v", h * dv)):
                t[p + f"mix.{n}"] = (rows, w)
                t[p + f"mix.{n}.conv"] = (rows, taps)
            t.update({p + "mix.b": (h, w), p + "mix.A_log": (h,), p + "mix.norm": (dv,),
                      p + "mix.a1": (lr, w), p + "mix.a2": (h * dk, lr), p + "mix.dt_bias": (h * dk,),
                      p + "mix.g1": (lr, w), p + "mix.g2": (h * dv, lr), p + "mix.o": (w, h * dv)})
        mlp = l["mlp"]
        if mlp is not None:
            t[p + "norm2"] = t[p + "norm2b"] = (w,)
            if mlp["kind"] == "dense":
                t.update({p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"])})
            else:
                ff = mlp["expert"]["ff"]
                for e in range(mlp["router"]["experts"]):
                    t.update({p + f"mlp.e{e}.gate": (ff, w), p + f"mlp.e{e}.up": (ff, w),
                              p + f"mlp.e{e}.down": (w, ff)})
                t.update({p + "mlp.router": (mlp["router"]["experts"], w),
                          p + "mlp.correction": (mlp["router"]["experts"],)})
                if mlp.get("shared"):
                    fs = mlp["shared"]["ff"]
                    t.update({p + "mlp.shared.gate": (fs, w), p + "mlp.shared.up": (fs, w),
                              p + "mlp.shared.down": (w, fs), p + "mlp.shared.sg": (1, w)})
        if cfg.side_dim:
            t.update({p + "side.gate": (cfg.side_dim, w), p + "side.proj": (w, cfg.side_dim),
                      p + "side.norm": (w,)})
    return t


def random_tensors(cfg: NulazenConfig, seed: int = 0, dtype=torch.bfloat16, device="cpu",
                   low_rank: int = 0) -> Dict[str, torch.Tensor]:
    """Random weights of the configuration's shapes: projections ~ N(0, 1/fan_in), norm
    weights near 1, decays / biases in ranges that keep the recurrence lively."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for name, shape in tensor_shapes(cfg, low_rank).items():
        leaf = name.split(".")[-1]
        if len(shape) == 1:
            r = torch.rand(shape, generator=g, device=device)
            if leaf == "A_log":
                x = torch.log(0.5 + 4.0 * r)
            elif leaf == "dt_bias":
                x = -3.0 + 3.0 * r
            elif leaf == "correction":
                x = 0.2 * (r - 0.5)
            else:
                x = 0.75 + 0.5 * r
        elif leaf == "conv":
            x = torch.randn(shape, generator=g, device=device) * 0.5
        elif name in ("embed", "side.embed", "loop.step"):
            x = torch.randn(shape, generator=g, device=device)
        else:
            x = torch.randn(shape, generator=g, device=device) * shape[1] ** -0.5
        out[name] = x.to(dtype)
    return out


def save_checkpoint(cfg: NulazenConfig, tensors: Dict[str, torch.Tensor], out_dir: str):
    import json

    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.contiguous().cpu() for k, v in tensors.items()},
              os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(config_to_dict(cfg), f, indent=1)


_Layer = StackedLayer
NulazenCache = StackedCache


class NulazenModel(StackedModel):
    family = "Nulazen"
    # decode steps up to this many rows run without a host round trip (per-pair expert
    # kernels) and are captured in hipGraphs; larger steps sort rows by expert on the host
    max_graph_rows = MoEFF.PAIR_ROWS

    def __init__(self, cfg: NulazenConfig, device, dtype=torch.bfloat16, comm: TPComm = SINGLE,
                 max_model_len: int = 8192, quantization: Optional[str] = None):
        super().__init__(cfg, device, dtype, comm, max_model_len, quantization)
        self.side_embed = None

    # ------------------------------------------------------------------ weights
    def load_tensors(self, get, has=lambda n: True):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        eps = cfg.rms_norm_eps
        f32 = lambda n: get(n).to(dev, torch.float32)   # noqa: E731
        self.load_head(get)
        self.final_norm = f32("final.norm")
        self.loop_step = f32("loop.step") if cfg.loop else None
        self.side_embed = get("side.embed").to(dev, dt).contiguous() if cfg.side_dim else None
        max_pos = max(self.max_model_len, 16) + 1
        self.layers = []
        for i, l in enumerate(cfg.layers):
            p, m = f"l{i}.", l["mixer"]
            mget = lambda n, p=p: get(p + "mix." + n)   # noqa: E731
            if l["type"] == LATENT:
                rot = m.get("rot", {})
                mixer = LatentAttention(mget, cfg.hidden_size, m["heads"], m["dim"], m["rot_dim"],
                                        m["vdim"], m["kv_rank"], m["scale"],
                                        rot.get("dims", m["rot_dim"]), rot.get("base", 10000.0), eps,
                                        dt, dev, max_pos)
            else:
                mixer = ChannelDelta(mget, cfg.hidden_size, m["heads"], m.get("kv_heads", m["heads"]),
                                     m["dim"], m["vdim"], m["conv"], eps, dt, dev)
            L = StackedLayer(l["type"], f32(p + "norm1"), f32(p + "norm1b"), mixer)
            mlp = l["mlp"]
            if mlp is not None:
                fget = lambda n, p=p: get(p + "mlp." + n)   # noqa: E731
                L.norm2, L.norm2b = f32(p + "norm2"), f32(p + "norm2b")
                if mlp["kind"] == "dense":
                    L.ff = DenseFF(fget, dt, dev)
                else:
                    r = mlp["router"]
                    grp = r.get("groups") or {}
                    sh = mlp.get("shared")
                    L.ff = MoEFF(fget, r["experts"], r["top"], mlp["expert"]["limit"],
                                 int(grp.get("count", 1)), int(grp.get("keep", grp.get("count", 1))),
                                 sh["limit"] if sh else None, dt, dev)
            if cfg.side_dim:
                L.side = TokenSide(lambda n, p=p: get(p + "side." + n), self.side_embed,
                                   i * cfg.side_dim, cfg.side_dim, dt, dev)
            self.layers.append(L)
        return self

    def random_tensors(self, seed: int, device):
        return random_tensors(self.cfg, seed, torch.bfloat16, device=device)


# ---------------------------------------------------------------------------------------
# registry: shapes for random-init runs (benchmarks, smoke tests)
# ---------------------------------------------------------------------------------------

def _delta(heads, dim, vdim, kv_heads=None, conv=4):
    return {"heads": heads, "kv_heads": kv_heads or heads, "dim": dim, "vdim": vdim, "conv": conv}


def _latent(heads, dim, rot_dim, vdim, rank, base=10000.0):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
            "scale": (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim}}


def _moe(experts, top, ff, shared_ff, groups=1, keep=1, limit=7.0):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff, "limit": limit}
    return m


def _preset(name, vocab, width, layers, loop=None, side=0):
    return config_from_dict({"vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "layers": layers,
                             "loop": ({"start": loop[0], "stop": loop[1], "times": loop[2]}
                                      if loop else None),
                             "token_side": {"dim": side} if side else None}, name)


PRESETS = {
    # CPU-test sized
    "nulazen-tiny": _preset("nulazen-tiny", 320, 96, [
        {"type": DELTA, "mixer": _delta(4, 16, 24, kv_heads=2, conv=3), "mlp": {"kind": "dense", "ff": 160}},
        {"type": LATENT, "mixer": _latent(3, 16, 8, 24, 40), "mlp": _moe(6, 2, 48, 64, groups=3, keep=2)},
        {"type": DELTA, "mixer": _delta(4, 16, 24, kv_heads=2, conv=3), "mlp": None},
    ], loop=(1, 3, 2), side=8),
    # a 2048-wide stack (benchmarks): 3 delta layers per latent layer, MoE feed-forwards
    "nulazen-2k": _preset("nulazen-2k", 32768, 2048, [
        {"type": DELTA, "mixer": _delta(16, 128, 128), "mlp": {"kind": "dense", "ff": 8192}},
        {"type": DELTA, "mixer": _delta(16, 128, 128), "mlp": _moe(32, 4, 1024, 2048, groups=4, keep=2)},
        {"type": DELTA, "mixer": _delta(16, 128, 128), "mlp": _moe(32, 4, 1024, 2048, groups=4, keep=2)},
        {"type": LATENT, "mixer": _latent(16, 128, 64, 128, 512), "mlp": _moe(32, 4, 1024, 2048, groups=4, keep=2)},
    ], side=64),
    # the same stack at 4096 width
    "nulazen-4k": _preset("nulazen-4k", 32768, 4096, [
        {"type": DELTA, "mixer": _delta(32, 128, 128), "mlp": {"kind": "dense", "ff": 14336}},
        {"type": DELTA, "mixer": _delta(32, 128, 128), "mlp": _moe(64, 6, 1408, 2816, groups=8, keep=4)},
        {"type": DELTA, "mixer": _delta(32, 128, 128), "mlp": _moe(64, 6, 1408, 2816, groups=8, keep=4)},
        {"type": LATENT, "mixer": _latent(32, 128, 64, 128, 512), "mlp": _moe(64, 6, 1408, 2816, groups=8, keep=4)},
    ], side=64),
}


def _build(cfg, device, dtype, comm, max_model_len, quantization):
    return NulazenModel(cfg, device, dtype, comm, max_model_len, quantization)


register(Architecture(
    name="nulazen",
    matches=lambda c: str(c.get("architecture", "")).lower() == "nulazen",
    parse=lambda c, name: config_from_dict(c, name),
    build=_build,
    presets=PRESETS,
))
