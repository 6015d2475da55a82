"""Bagasun: a decoder-only model whose configuration lists, layer by layer, one of three
mixers -- windowed attention with sigmoid weights and a logarithmic distance bias
(``attention``), windowed differential attention with rotary positions
(``attention_2``) and a selective state-space mixer (``mamba2``) -- each followed by an
optional gated feed-forward.  A layer may borrow another layer's weights
(``weights_of``) while keeping a cache or state of its own.  Norms sit before and after
every sublayer and carry one number each; the residual stream is fp32 and starts as
``embed[token] * embedding.scale``.

Every size comes from ``config.json`` (keys: vocab, width, norm.eps, embedding.scale,
layers[].type / mixer / mlp / weights_of) or from tensor shapes.  Tensor names: embed,
head, final.norm, l<i>.{norm1,norm1b,norm2,norm2b}, l<i>.mix.*, l<i>.mlp.*.

The model body (layer runs, fused norms, caches, logits) is
:class:`..models.stacked.StackedModel`; the sublayers are in :mod:`.mixers`.
"""
from __future__ import annotations

import dataclasses
import os
from typing import Dict, List, Optional, Tuple

import torch

from .mixers import DifferentialAttention, GatedFF, SigmoidAttention, StateSpaceMixer
from .registry import Architecture, register
from .stacked import StackedLayer, StackedModel

SIGMOID, DIFF, SSM = "attention", "attention_2", "mamba2"


@dataclasses.dataclass(frozen=True)
class BagasunConfig:
    name: str
    vocab_size: int
    hidden_size: int
    rms_norm_eps: float
    embed_scale: float
    layers: tuple                      # per layer: dict(type=, mixer=, mlp=, weights_of=)
    max_position_embeddings: int = 1 << 17
    bos_token_id: int = 0
    eos_token_ids: tuple = ()
    tie_word_embeddings: bool = False
    architecture = "bagasun"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> List[Tuple[int, Optional[int]]]:
        """Execution order: every listed layer runs once, on its own weights or on the
        weights of the layer it names."""
        return [(l["weights_of"] if l["weights_of"] is not None else i, None)
                for i, l in enumerate(self.layers)]

    def owners(self) -> List[int]:
        return [i for i, l in enumerate(self.layers) if l["weights_of"] is None]

    def num_params(self) -> int:
        return sum(int(torch.Size(s).numel()) for s in tensor_shapes(self).values())

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        total = 0
        for l in self.layers:
            m = l["mixer"]
            if l["type"] == SIGMOID:
                total += m["kv_heads"] * (m["dim"] + m["vdim"]) * dtype_bytes
            elif l["type"] == DIFF:
                total += m["kv_heads"] * (2 * m["dim"] + m["vdim"]) * dtype_bytes
        return total


def config_from_dict(c: dict, name: str = "bagasun") -> BagasunConfig:
    layers = []
    for i, l in enumerate(c["layers"]):
        if l["type"] not in (SIGMOID, DIFF, SSM):
            raise ValueError(f"unknown mixer type {l['type']!r}")
        mlp = l.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
        src, hops = l.get("weights_of"), 0
        while src is not None:                   # a borrowed layer may borrow in turn
            src, hops = int(src), hops + 1
            if not 0 <= src < len(c["layers"]) or hops > len(c["layers"]):
                raise ValueError(f"layer {i}: weights_of does not lead to a layer with weights of its own")
            if c["layers"][src].get("weights_of") is None:
                break
            src = c["layers"][src]["weights_of"]
        if src is not None and c["layers"][src]["type"] != l["type"]:
            raise ValueError(f"layer {i}: weights_of names a layer of another type")
        layers.append({"type": l["type"], "mixer": dict(l["mixer"]), "mlp": dict(mlp) if mlp else None,
                       "weights_of": src})
    return BagasunConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                         rms_norm_eps=float(c.get("norm", {}).get("eps", 1e-6)),
                         embed_scale=float(c.get("embedding", {}).get("scale", 1.0)), layers=tuple(layers),
                         max_position_embeddings=int(c.get("max_positions", 1 << 17)))


def config_to_dict(cfg: BagasunConfig) -> dict:
    layers = []
    for l in cfg.layers:
        d = {"type": l["type"], "mixer": dict(l["mixer"]), "mlp": dict(l["mlp"]) if l["mlp"] else None}
        if l["weights_of"] is not None:
            d["weights_of"] = l["weights_of"]
        layers.append(d)
    return {"architecture": "Bagasun", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "norm": {"eps": cfg.rms_norm_eps}, "embedding": {"scale": cfg.embed_scale}, "layers": layers}


def tensor_shapes(cfg: BagasunConfig) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint of this configuration (random init, tests)."""
    w, v = cfg.hidden_size, cfg.vocab_size
    t: Dict[str, tuple] = {"embed": (v, w), "head": (v, w), "final.norm": ()}
    for i in cfg.owners():
        l = cfg.layers[i]
        p, m = f"l{i}.", l["mixer"]
        t[p + "norm1"] = t[p + "norm1b"] = ()
        if l["type"] == SSM:
            h, dv, n, g, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            ch = h * dv + 2 * g * n
            t.update({p + "mix.in": (h * dv + ch + h, w), p + "mix.conv": (ch, taps), p + "mix.conv.b": (ch,),
                      p + "mix.dt_bias": (h,), p + "mix.A_log": (h,), p + "mix.D": (h,),
                      p + "mix.norm": (h * dv,), p + "mix.o": (w, h * dv)})
        else:
            h, g, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            maps = 2 if l["type"] == DIFF else 1
            t.update({p + "mix.q": (h * maps * dk, w), p + "mix.k": (g * maps * dk, w), p + "mix.v": (g * dv, w),
                      p + "mix.o": (w, h * dv)})
            if l["type"] == DIFF:
                t.update({p + f"mix.{n}": (dk,) for n in ("lq1", "lk1", "lq2", "lk2")})
                t[p + "mix.g"] = (h, w)
            else:
                t.update({p + "mix.q.b": (h * dk,), p + "mix.k.b": (g * dk,), p + "mix.v.b": (g * dv,),
                          p + "mix.q.norm": (h * dk,), p + "mix.k.norm": (g * dk,),
                          p + "mix.r1": (h,), p + "mix.r2": (h,), p + "mix.pb": (h,)})
        if l["mlp"] is not None:
            ff = l["mlp"]["ff"]
            t[p + "norm2"] = t[p + "norm2b"] = ()
            t.update({p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return t


def random_tensors(cfg: BagasunConfig, seed: int = 0, dtype=torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    """Random weights of the configuration's shapes: projections ~ N(0, 1/fan_in), norm
    weights near 1, decays / step biases in ranges that keep the recurrence lively."""
    g = torch.Generator(device=device).manual_seed(seed)
    out: Dict[str, torch.Tensor] = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        r = torch.rand(shape, generator=g, device=device)
        n = torch.randn(shape, generator=g, device=device)
        if len(shape) == 2 and leaf != "conv":
            x = n * (1.0 if name == "embed" else shape[1] ** -0.5)
        elif leaf == "conv":
            x = n * 0.5
        elif leaf == "A_log":
            x = torch.log(0.3 + 3.0 * r)
        elif leaf == "dt_bias":
            x = -3.0 + 3.0 * r
        elif leaf == "b":
            x = 0.2 * n
        elif leaf in ("r1", "r2"):
            x = 0.2 + 0.8 * r
        elif leaf == "pb":
            x = -2.0 + r
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            x = 0.3 * n
        else:                                    # norm weights, D
            x = 0.75 + 0.5 * r
        out[name] = x.to(dtype)
    return out


def save_checkpoint(cfg: BagasunConfig, tensors: Dict[str, torch.Tensor], out_dir: str):
    import json

    from safetensors.torch import save_file

    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.contiguous().cpu() for k, v in tensors.items()},
              os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(config_to_dict(cfg), f, indent=1)


def _window(mixer: dict) -> int:
    """Keys a position sees, itself included (0: every earlier key, when no mask is given)."""
    return int((mixer.get("mask") or {}).get("size", 0))


class BagasunModel(StackedModel):
    family = "Bagasun"

    def load_tensors(self, get, has=lambda n: True):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        eps, width = cfg.rms_norm_eps, cfg.hidden_size
        self.load_head(get)
        self.embed_scale = cfg.embed_scale
        self.final_norm = self.norm_weight(get("final.norm"))
        max_pos = max(self.max_model_len, 16) + 1
        self.layers = [None] * len(cfg.layers)
        for i in cfg.owners():
            l = cfg.layers[i]
            p, m = f"l{i}.", l["mixer"]
            mget = lambda n, p=p: get(p + "mix." + n)   # noqa: E731
            if l["type"] == SSM:
                mixer = StateSpaceMixer(mget, width, m["heads"], m["vdim"], m["state"], m.get("groups", 1),
                                        m["conv"], m.get("norm_groups", 1), eps, dt, dev)
            elif l["type"] == SIGMOID:
                mixer = SigmoidAttention(mget, width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"],
                                         m["vdim"], _window(m), m["scale"], eps, dt, dev)
            else:
                rot = m.get("rot") or {}
                sc = rot.get("scaling")
                mixer = DifferentialAttention(
                    mget, width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"],
                    _window(m), m["scale"], m["diff"], int(rot.get("dims", 0)),
                    float(rot.get("base", 10000.0)),
                    (sc["factor"], sc["low"], sc["high"], sc["original"]) if sc else None, eps, dt, dev, max_pos)
            nw = lambda n, p=p: self.norm_weight(get(p + n))   # noqa: E731
            L = StackedLayer(l["type"], nw("norm1"), nw("norm1b"), mixer)
            if l["mlp"] is not None:
                L.norm2, L.norm2b = nw("norm2"), nw("norm2b")
                L.ff = GatedFF(lambda n, p=p: get(p + "mlp." + n), dt, dev)
            self.layers[i] = L
        return self

    def random_tensors(self, seed: int, device):
        return random_tensors(self.cfg, seed, torch.bfloat16, device=device)


# ---------------------------------------------------------------------------------------
# registry: shapes for random-init runs (benchmarks, smoke tests)
# ---------------------------------------------------------------------------------------

def _ssm(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
            "norm_groups": norm_groups}


def _sig(heads, kv_heads, dim, vdim, window):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
            "scale": dim ** -0.5}


def _dif(heads, kv_heads, dim, vdim, window, diff=0.5, rot_dims=None, base=500000.0):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
            "scale": dim ** -0.5, "diff": diff,
            "rot": {"dims": rot_dims or dim, "base": base,
                    "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}


def _preset(name, vocab, width, layers, scale=1.0):
    return config_from_dict({"vocab": vocab, "width": width, "norm": {"eps": 1e-6},
                             "embedding": {"scale": scale}, "layers": layers}, name)


def _ff(n):
    return {"kind": "dense", "ff": n}


PRESETS = {
    # CPU-test sized: every mixer once, then the first two again on shared weights
    "bagasun-tiny": _preset("bagasun-tiny", 320, 96, [
        {"type": SSM, "mixer": _ssm(4, 16, 12, groups=2, conv=3, norm_groups=2), "mlp": _ff(128)},
        {"type": DIFF, "mixer": _dif(4, 2, 8, 16, 24, rot_dims=4), "mlp": _ff(128)},
        {"type": SIGMOID, "mixer": _sig(3, 1, 16, 24, 20), "mlp": None},
        {"type": SSM, "mixer": _ssm(4, 16, 12, groups=2, conv=3, norm_groups=2), "mlp": _ff(128), "weights_of": 0},
        {"type": DIFF, "mixer": _dif(4, 2, 8, 16, 24, rot_dims=4), "mlp": _ff(128), "weights_of": 1},
    ], scale=4.0),
    # a 2048-wide stack (benchmarks): two state-space layers per attention layer
    "bagasun-2k": _preset("bagasun-2k", 32768, 2048, [
        {"type": SSM, "mixer": _ssm(32, 128, 128, groups=8, norm_groups=8), "mlp": _ff(8192)},
        {"type": DIFF, "mixer": _dif(16, 4, 64, 128, 1024), "mlp": _ff(8192)},
        {"type": SSM, "mixer": _ssm(32, 128, 128, groups=8, norm_groups=8), "mlp": _ff(8192)},
        {"type": SIGMOID, "mixer": _sig(16, 4, 128, 128, 1024), "mlp": _ff(8192)},
    ], scale=16.0),
    # the same stack at 4096 width
    "bagasun-4k": _preset("bagasun-4k", 32768, 4096, [
        {"type": SSM, "mixer": _ssm(64, 128, 128, groups=8, norm_groups=8), "mlp": _ff(14336)},
        {"type": DIFF, "mixer": _dif(32, 8, 64, 128, 2048), "mlp": _ff(14336)},
        {"type": SSM, "mixer": _ssm(64, 128, 128, groups=8, norm_groups=8), "mlp": _ff(14336)},
        {"type": SIGMOID, "mixer": _sig(32, 8, 128, 128, 2048), "mlp": _ff(14336)},
    ], scale=16.0),
}


def _build(cfg, device, dtype, comm, max_model_len, quantization):
    return BagasunModel(cfg, device, dtype, comm, max_model_len, quantization)


register(Architecture(
    name="bagasun",
    matches=lambda c: str(c.get("architecture", "")).lower() == "bagasun",
    parse=lambda c, name: config_from_dict(c, name),
    build=_build,
    presets=PRESETS,
))
