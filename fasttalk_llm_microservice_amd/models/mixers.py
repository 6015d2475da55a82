"""Reusable sublayers built on :mod:`fasttalk_llm_microservice_amd.ops.mixers`:
latent attention (paged latent cache), the channel-decay gated delta rule (state
slots), dense and mixture-of-experts feed-forwards and the per-layer token-side input.

Each class takes its sizes and constants as constructor arguments and a ``get(name)``
callable that returns a weight tensor ([out, in] for projections), so a model file only
describes which sublayers it stacks.  Matrix products are vendor GEMMs (``F.linear`` /
``torch.bmm``) in the compute dtype with fp32 accumulation; everything around them runs
in the HIP kernels (GPU) or their PyTorch twins (CPU backend).
"""
from __future__ import annotations

from typing import Callable, List, Optional

import torch
import torch.nn.functional as F

from ..ops import mixers as M

Get = Callable[[str], torch.Tensor]


class StepContext:
    """What a sublayer needs to know about the step: rows' token ids, positions and
    cache slots, and the row segments (one per scheduled sequence)."""

    def __init__(self, ids, positions, slot_mapping, seg: M.Segments):
        self.ids = ids
        self.positions = positions
        self.slot_mapping = slot_mapping
        self.seg = seg


class LatentAttention:
    """Multi-head attention whose keys and values are up-projections of one cached
    latent row per token plus one rotated key part shared by all heads.

    The cache holds [rms_norm(latent) | rope(shared key)] per token.  Queries are taken
    into latent space (q_unrotated W_uk, per head), so the attention kernel reads the
    cache rows directly and returns latent-space sums that W_uv maps to the values."""

    def __init__(self, get: Get, width: int, heads: int, dim: int, rot_dim: int, vdim: int,
                 kv_rank: int, scale: float, rot_dims: int, rot_base: float, eps: float,
                 dtype, device, max_pos: int):
        self.heads, self.dn, self.dr, self.dv, self.rank = heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.rot_dims, self.eps, self.dtype = float(scale), int(rot_dims), eps, dtype
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError("rotary dims must be even and within the rotated part")
        self.nq = heads * (dim + rot_dim)
        # q and the latent / shared-key down-projection in one product
        self.wqd = torch.cat([get("q"), get("dkv")], 0).to(device, dtype).contiguous()
        self.dkv_norm = get("dkv.norm").to(device, torch.float32)
        # W_uk [heads, dim, rank] and W_uv^T [heads, rank, vdim], fp32 (small; the
        # absorbed products run on fp32 queries / attention sums)
        self.wuk = get("uk").to(device, torch.float32).view(heads, dim, kv_rank).contiguous()
        self.wuvT = get("uv").to(device, torch.float32).view(heads, vdim, kv_rank) \
            .transpose(1, 2).contiguous()
        self.wo = get("o").to(device, dtype).contiguous()
        self.table = M.rope_table(max_pos, rot_dims, rot_base, device=device)

    # segments of this many rows or more run as matrix products (ops.mixers
    # latent_attention_products), shorter ones and decode rows in the per-row kernel
    PRODUCT_ROWS = 32

    def cache_width(self) -> int:
        return self.rank + self.dr

    def __call__(self, h, ctx: StepContext, cache) -> torch.Tensor:
        t = h.shape[0]
        qd = F.linear(h, self.wqd)
        q, dkv = qd[:, :self.nq], qd[:, self.nq:]
        M.latent_kv_write(dkv, self.dkv_norm, self.eps, self.table, self.rot_dims, ctx.positions,
                          ctx.slot_mapping, cache, self.rank)
        qn, qr = M.latent_q_rope(q, self.table, self.rot_dims, ctx.positions, self.heads, self.dn,
                                 self.dr)
        qa = torch.bmm(qn.transpose(0, 1), self.wuk)                 # [heads, T, rank]
        seg = ctx.seg
        if seg.host is not None and seg.max_rows >= self.PRODUCT_ROWS:
            # prefill chunks: two tiled products per segment; short segments and decode
            # rows (if any) keep the per-row kernel
            ol = torch.zeros_like(qa)
            M.latent_attention(qa, qr, cache, seg, self.scale, self.rank, skip_from=self.PRODUCT_ROWS,
                               out=ol)
            M.latent_attention_products(ol, qa, qr, cache, seg, self.scale, self.rank,
                                        self.PRODUCT_ROWS, self.dtype)
        else:
            ol = M.latent_attention(qa, qr, cache, seg, self.scale, self.rank)
        o = torch.bmm(ol, self.wuvT)                                  # [heads, T, vdim]
        o = o.transpose(0, 1).reshape(t, self.heads * self.dv).to(self.dtype)
        return F.linear(o, self.wo)


class ChannelDelta:
    """Gated delta rule with a decay per head and key channel, behind short causal
    convolutions on q, k and v; output normed per head and gated."""

    def __init__(self, get: Get, width: int, heads: int, kv_heads: int, dim: int, vdim: int,
                 taps: int, eps: float, dtype, device):
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kvh, self.dk, self.dv, self.taps = heads, kv_heads, dim, vdim, taps
        self.eps, self.dtype = eps, dtype
        self.wqkv = torch.cat([get("q"), get("k"), get("v")], 0).to(device, dtype).contiguous()
        self.channels = self.wqkv.shape[0]
        self.conv_w = torch.cat([get("q.conv"), get("k.conv"), get("v.conv")], 0) \
            .to(device, torch.float32).contiguous()
        if self.conv_w.shape != (self.channels, taps):
            raise ValueError("convolution weights do not fit the projections")
        a1, g1, b = get("a1"), get("g1"), get("b")
        self.ra, self.rg = a1.shape[0], g1.shape[0]
        # the two low-rank down-projections and beta's projection in one product
        self.wlo = torch.cat([a1, g1, b], 0).to(device, dtype).contiguous()
        self.wa2 = get("a2").to(device, dtype).contiguous()
        self.wg2 = get("g2").to(device, dtype).contiguous()
        self.a_log = get("A_log").to(device, torch.float32)
        self.dt_bias = get("dt_bias").to(device, torch.float32)
        self.norm = get("norm").to(device, torch.float32)
        self.wo = get("o").to(device, dtype).contiguous()

    def state_shapes(self):
        return (self.heads, self.dk, self.dv), (max(self.taps - 1, 0), self.channels)

    def __call__(self, h, ctx: StepContext, state) -> torch.Tensor:
        s_rec, s_conv = state
        qkv = F.linear(h, self.wqkv)
        lo = F.linear(h, self.wlo)
        a = F.linear(lo[:, :self.ra], self.wa2)
        gp = F.linear(lo[:, self.ra:self.ra + self.rg], self.wg2)
        b = lo[:, self.ra + self.rg:].contiguous()
        qkv = M.short_conv_silu(qkv, self.conv_w, s_conv, ctx.seg)
        o = M.gated_delta_rule(qkv, a, b, self.a_log, self.dt_bias, s_rec, ctx.seg, self.heads,
                               self.kvh, self.dk, self.dv)
        y = M.head_rms_gate(o, self.norm, gp, self.eps, self.heads, self.dv, self.dtype)
        return F.linear(y, self.wo)


class DenseFF:
    """down(relu(up h)^2)."""

    def __init__(self, get: Get, dtype, device):
        self.up = get("up").to(device, dtype).contiguous()
        self.down = get("down").to(device, dtype).contiguous()

    def __call__(self, h, ctx=None) -> torch.Tensor:
        return F.linear(M.relu_sq(F.linear(h, self.up)), self.down)


def _glu_weights(get: Get, prefix: str, dtype, device, extra: Optional[torch.Tensor] = None):
    parts = [get(prefix + "gate"), get(prefix + "up")] + ([extra] if extra is not None else [])
    return (torch.cat(parts, 0).to(device, dtype).contiguous(),
            get(prefix + "down").to(device, dtype).contiguous())


class MoEFF:
    """Top-k mixture of clamped-GLU experts with group-limited routing, an additive
    selection bias that does not enter the weights, and an optional gated shared expert.

    Expert: g = min(W_gate h, limit), u = clamp(W_up h, +-limit),
    y = g sigmoid(1.702 g) (u + 1), out = W_down y.  Router logits are fp32."""

    def __init__(self, get: Get, experts: int, top: int, limit: float, groups: int, keep: int,
                 shared_limit: Optional[float], dtype, device):
        if groups < 1 or experts % groups or not 1 <= keep <= groups or top > experts // groups * keep:
            raise ValueError("expert groups do not fit the expert count")
        self.e, self.top, self.limit, self.groups, self.keep = experts, top, float(limit), groups, keep
        self.dtype = dtype
        self.router = get("router").to(device, torch.float32).contiguous()
        self.correction = get("correction").to(device, torch.float32).contiguous()
        gus, downs = zip(*[_glu_weights(get, f"e{i}.", dtype, device) for i in range(experts)])
        self.wgu = torch.stack(gus).contiguous()       # [E, 2 ff, width]
        self.wdown = torch.stack(downs).contiguous()   # [E, width, ff]
        self.shared = None
        if shared_limit is not None:
            # the shared expert's per-token gate logit rides as one more output row
            self.shared = _glu_weights(get, "shared.", dtype, device, extra=get("shared.sg"))
            self.shared_limit = float(shared_limit)

    def __call__(self, h, ctx=None) -> torch.Tensor:
        t, width = h.shape
        out = torch.zeros(t, width, dtype=torch.float32, device=h.device)
        z = F.linear(h.float(), self.router)
        idx, wts = M.moe_topk(z, self.correction, self.top, self.groups, self.keep)
        if t <= self.PAIR_ROWS:
            # decode-size steps: per-pair weight streaming, nothing read back on the host
            M.moe_pairs(out, h, idx, wts, self.wgu, self.wdown, self.limit)
            return self._shared(out, h)
        flat = idx.view(-1).long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=self.e).tolist()
        rows = (order // self.top).int()
        w = wts.view(-1).index_select(0, order)
        hs = h.index_select(0, rows.long())
        a = 0
        for e, n in enumerate(counts):
            if n == 0:
                continue
            y = M.clamp_swiglu(F.linear(hs[a:a + n], self.wgu[e]), self.limit)
            M.scale_add_rows(out, F.linear(y, self.wdown[e]), rows[a:a + n], w[a:a + n])
            a += n
        return self._shared(out, h)

    # rows up to which every (row, expert) pair streams its expert's weights (decode);
    # above, rows are sorted by expert and each expert runs one tiled product
    PAIR_ROWS = 64

    def _shared(self, out, h):
        if self.shared is not None:
            wgu, wdown = self.shared
            gu = F.linear(h, wgu)
            y = M.clamp_swiglu(gu, self.shared_limit)
            M.scale_add_rows(out, F.linear(y, wdown), None, gu[:, -1].contiguous(), sigmoid=True)
        return out


class TokenSide:
    """Per-layer token input: y = proj(gelu_tanh(gate x) * side_embed[token, part]);
    the caller adds rms_norm(y) * norm to the residual."""

    def __init__(self, get: Get, table: torch.Tensor, col0: int, dim: int, dtype, device):
        self.table, self.col0, self.dim = table, col0, dim
        self.gate = get("gate").to(device, dtype).contiguous()
        self.proj = get("proj").to(device, dtype).contiguous()
        self.norm = get("norm").to(device, torch.float32)

    def __call__(self, xc, ctx: StepContext) -> torch.Tensor:
        g = M.side_gate(F.linear(xc, self.gate), self.table, ctx.ids, self.col0, self.dim)
        return F.linear(g, self.proj)
