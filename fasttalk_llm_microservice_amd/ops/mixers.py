"""Sequence-mixer and mixture-of-experts ops: latent (low-rank KV) attention over a
paged latent cache, the gated delta-rule recurrence with per-channel decay over state
slots, short causal convolutions, grouped top-k routing, clamped-GLU experts, and the
fp32-residual norms that tie them together.

GPU tensors run the gfx950 kernels of the ``_C_mixers`` extension (``csrc/mixers``),
fp32 or bf16 activations with fp32 statistics / scores / state; CPU tensors run the
PyTorch implementations in :mod:`.mixers_ref`.  As in :mod:`fasttalk_llm_microservice_amd.ops`
there is no silent fallback for GPU tensors.

A step's rows are described by :class:`Segments`: every scheduled sequence contributes
one segment of consecutive rows (a decode row is a segment of one row, a prefill chunk
a longer one), with the position of its first row, its state slot and its block table.
"""
from __future__ import annotations

import dataclasses
import importlib
import os
import threading
from typing import Optional

import torch

from . import mixers_ref as ref

_lock = threading.Lock()
_M = None


def native_mixers():
    """The loaded ``_C_mixers`` extension, built in-tree on first use if allowed."""
    global _M
    if _M is not None:
        return _M
    with _lock:
        if _M is not None:
            return _M
        try:
            mod = importlib.import_module("fasttalk_llm_microservice_amd._C_mixers")
        except ImportError as e:
            if os.environ.get("FT_AUTOBUILD", "1") == "0":
                raise RuntimeError("fasttalk native extension _C_mixers is not built; run "
                                   "`python -m fasttalk_llm_microservice_amd.ops.build --only mixers`") from e
            from .build import build_mixers

            build_mixers(verbose=True)
            mod = importlib.import_module("fasttalk_llm_microservice_amd._C_mixers")
        _M = mod
        return _M


@dataclasses.dataclass
class Segments:
    """Row segments of one step (device int32 tensors; ``num`` / ``max_rows`` host ints)."""
    start: torch.Tensor          # [num + 1] first row of each segment, then the row count
    pos0: torch.Tensor           # [num] sequence position of the segment's first row
    slot: torch.Tensor           # [num] recurrent-state slot (-1: padding, state untouched)
    kv_len: torch.Tensor         # [num] context length once this step's rows are written
    block_tables: torch.Tensor   # [num, max_blocks]
    num: int
    max_rows: int                # longest segment (rows)
    max_kv: int = 0              # longest context (tokens); 0 = unknown
    # host copies of start / pos0 / kv_len (eager steps; None inside captured graphs)
    host: Optional[tuple] = None


# ---------------------------------------------------------------------------------
# residual stream (fp32) and norms
# ---------------------------------------------------------------------------------

def embed_rows(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """fp32 residual rows table[ids]."""
    if ids.is_cuda:
        out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=ids.device)
        native_mixers().embed_rows(out, ids, table)
        return out
    return ref.embed_rows(ids, table)


def rms_norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype,
                  add_vec: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = x / sqrt(mean(x^2) + eps) * w of fp32 rows x, rounded to ``out_dtype``;
    with ``add_vec`` the rows are first updated in place, x += add_vec."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        native_mixers().add_rms_norm(x, None, None, add_vec, w, out, None, eps)
        return out
    return ref.rms_norm_rows(x, w, eps, out_dtype, add_vec)


def add_rms_norm_rows(residual: torch.Tensor, y: torch.Tensor, wb: torch.Tensor, eps: float,
                      add_vec: Optional[torch.Tensor] = None, next_w: Optional[torch.Tensor] = None,
                      out_dtype=None, want_cast: bool = False):
    """residual (fp32, in place) += rms_norm(y) * wb (+ add_vec); returns
    (rms_norm(residual) * next_w or None, residual cast to out_dtype or None)."""
    out_dtype = out_dtype or y.dtype
    if residual.is_cuda:
        out = torch.empty(residual.shape, dtype=out_dtype, device=y.device) if next_w is not None else None
        cast = torch.empty(residual.shape, dtype=out_dtype, device=y.device) if want_cast else None
        native_mixers().add_rms_norm(residual, y, wb, add_vec, next_w, out, cast, eps)
        return out, cast
    return ref.add_rms_norm_rows(residual, y, wb, eps, add_vec, next_w, out_dtype, want_cast)


# ---------------------------------------------------------------------------------
# rotary positions (partial, rotate-half pairs, fp32 angles)
# ---------------------------------------------------------------------------------

rope_table = ref.rope_table


# ---------------------------------------------------------------------------------
# short convolution + gated delta rule (recurrent state slots)
# ---------------------------------------------------------------------------------

def short_conv_silu(x: torch.Tensor, conv_w: torch.Tensor, conv_state: torch.Tensor, seg: Segments):
    """Per-channel causal convolution over time, then SiLU.  ``conv_w`` [C, taps] fp32
    (last column = the current row); ``conv_state`` [slots, taps-1, C] fp32 holds each
    sequence's last inputs and is updated; a segment at position 0 starts from zeros."""
    if x.is_cuda:
        out = torch.empty_like(x)
        native_mixers().short_conv_silu(out, x, conv_w, conv_state, seg.start, seg.pos0, seg.slot,
                                        seg.num, seg.max_rows)
        return out
    return ref.short_conv_silu(x, conv_w, conv_state, seg)


def gated_delta_rule(qkv, a, b, a_log, dt_bias, state, seg: Segments, heads: int, kv_heads: int,
                     dk: int, dv: int) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel.

    Rows of ``qkv`` are [q (kv_heads*dk) | k (kv_heads*dk) | v (heads*dv)] after the
    short convolution; q and k are unit-normalised per head here (q also * dk^-1/2),
    beta = sigmoid(b), decay = exp(-exp(a_log) * softplus(a + dt_bias)).  Per head and
    row:  S <- decay (.) S (rows of S);  u = beta (v - S^T k);  S <- S + k u^T;
    o = S^T q.  ``state`` [slots, heads, dk, dv] fp32 is read (zeros at position 0)
    and left at the segment's last row.  Returns o fp32 [T, heads*dv]."""
    if qkv.is_cuda:
        o = torch.empty(qkv.shape[0], heads * dv, dtype=torch.float32, device=qkv.device)
        native_mixers().gated_delta_rule(o, qkv, a, b, a_log, dt_bias, state, seg.start, seg.pos0,
                                         seg.slot, seg.num, heads, kv_heads, dk, dv)
        return o
    return ref.gated_delta_rule(qkv, a, b, a_log, dt_bias, state, seg, heads, kv_heads, dk, dv)


def head_rms_gate(o, w, gate_pre, eps: float, heads: int, dv: int, out_dtype):
    """Per head: o / rms(o) * w * sigmoid(gate_pre), rounded to ``out_dtype``."""
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        native_mixers().head_rms_gate(out, o, w, gate_pre, eps, heads, dv)
        return out
    return ref.head_rms_gate(o, w, gate_pre, eps, heads, dv, out_dtype)


# ---------------------------------------------------------------------------------
# latent attention (paged cache of [normed latent | rotated shared key])
# ---------------------------------------------------------------------------------

def latent_kv_write(dkv, norm_w, eps: float, table, rot_dims: int, positions, slot_mapping, cache,
                    rank: int):
    """Cache row = [rms_norm(dkv[:rank]) * norm_w | rope(dkv[rank:])] at each row's slot."""
    if dkv.is_cuda:
        native_mixers().latent_kv_write(dkv, norm_w, eps, table, rot_dims, positions, slot_mapping,
                                        cache, rank)
    else:
        ref.latent_kv_write(dkv, norm_w, eps, table, rot_dims, positions, slot_mapping, cache, rank)


def latent_q_rope(q, table, rot_dims: int, positions, heads: int, dn: int, dr: int):
    """q rows [heads x (dn unrotated | dr rotated)] -> fp32 ([T, heads, dn], [T, heads, dr] rotated)."""
    if q.is_cuda:
        t = q.shape[0]
        qn = torch.empty(t, heads, dn, dtype=torch.float32, device=q.device)
        qr = torch.empty(t, heads, dr, dtype=torch.float32, device=q.device)
        native_mixers().latent_q_rope(qn, qr, q, table, rot_dims, positions, heads, dn, dr)
        return qn, qr
    return ref.latent_q_rope(q, table, rot_dims, positions, heads, dn, dr)


def latent_attention(qa, qr, cache, seg: Segments, scale: float, rank: int,
                     skip_from: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal softmax attention over the paged latent cache.  ``qa`` fp32 [heads, T,
    rank]: the unrotated query parts carried into latent space (q W_uk); ``qr`` fp32
    [T, heads, dr]: the rotated parts.  Score = (qa . c + qr . k_rot) * scale; all heads
    share the cached row, whose first ``rank`` entries are also the value.  Returns
    fp32 [heads, T, rank].  ``skip_from`` > 0: segments of that many rows or more are
    left to the caller (:func:`latent_attention_products`)."""
    if qa.is_cuda:
        if out is None:
            out = torch.empty_like(qa)
        native_mixers().latent_attention(out, qa, qr, cache, seg.start, seg.pos0, seg.kv_len,
                                         seg.block_tables, seg.num, seg.max_rows, scale, rank,
                                         skip_from, seg.max_kv)
        return out
    r = ref.latent_attention(qa, qr, cache, seg, scale, rank)
    if out is not None:
        out.copy_(r)
        return out
    return r


def causal_softmax(s, rows_per_head: int, first_pos: int, scale: float, out_dtype):
    """P = softmax(scale * S) per row over the keys j <= first_pos + (row mod
    rows_per_head), zeros beyond; S fp32 [heads * rows_per_head, keys]."""
    if s.is_cuda:
        p = torch.empty(s.shape, dtype=out_dtype, device=s.device)
        native_mixers().causal_softmax(p, s, rows_per_head, first_pos, scale)
        return p
    return ref.causal_softmax(s, rows_per_head, first_pos, scale, out_dtype)


_MM_F32_OUT = {}


def mm_f32(a, b):
    """a @ b with fp32 accumulation and fp32 output (operands fp32, or bf16 where the
    vendor library returns fp32 from bf16 operands; otherwise widened first)."""
    if a.dtype == torch.float32:
        return torch.mm(a, b)
    ok = _MM_F32_OUT.get(a.device.type)
    if ok is None and a.is_cuda:
        try:
            torch.mm(a[:1], b[:, :1], out_dtype=torch.float32)
            ok = True
        except (TypeError, RuntimeError):
            ok = False
        _MM_F32_OUT[a.device.type] = ok
    return torch.mm(a, b, out_dtype=torch.float32) if ok else torch.mm(a.float(), b.float())


# bytes of fp32 scores the product path holds at once
PRODUCT_SCORE_BYTES = 256 << 20


def latent_attention_products(out, qa, qr, cache, seg: Segments, scale: float, rank: int,
                              min_rows: int, dtype):
    """Segments of ``min_rows`` rows or more as two matrix products: all heads share
    the cached rows, so with M = heads x rows the scores are Q [M, rank+dr] C^T and the
    sums P [M, keys] C[:, :rank], with a causal softmax (fp32 statistics) in between.
    Needs the segments' host copies; writes its rows of ``out`` [heads, T, rank]."""
    start, pos0, kv_len = seg.host
    heads = qa.shape[0]
    bs = cache.shape[1]
    width = cache.shape[2]
    for s in range(seg.num):
        a, b = start[s], start[s + 1]
        n = b - a
        if n < min_rows:
            continue
        nblk = (kv_len[s] + bs - 1) // bs
        kv = cache.index_select(0, seg.block_tables[s, :nblk].long()).view(nblk * bs, width)
        step = max(1, min(n, PRODUCT_SCORE_BYTES // (4 * heads * max(1, kv_len[s]))))
        for c0 in range(0, n, step):
            c1 = min(n, c0 + step)
            keys = min(kv_len[s], pos0[s] + c1)          # the chunk's last row sees this many
            q = torch.cat([qa[:, a + c0:a + c1], qr[a + c0:a + c1].transpose(0, 1)], -1) \
                .reshape(heads * (c1 - c0), width).to(dtype)
            sc = mm_f32(q, kv[:keys].t())
            p = causal_softmax(sc, c1 - c0, pos0[s] + c0, scale, dtype)
            out[:, a + c0:a + c1] = mm_f32(p, kv[:keys, :rank]).view(heads, c1 - c0, rank)
    return out


# ---------------------------------------------------------------------------------
# mixture of experts
# ---------------------------------------------------------------------------------

def moe_topk(z, correction, top: int, groups: int, keep: int):
    """Router: s = softmax(z) (fp32); choice = s + correction; experts outside the
    ``keep`` best of ``groups`` equal groups (by their best choice score) are excluded;
    the ``top`` best choices are returned with their s as weights (not renormalised)."""
    if z.is_cuda:
        t = z.shape[0]
        idx = torch.empty(t, top, dtype=torch.int32, device=z.device)
        wts = torch.empty(t, top, dtype=torch.float32, device=z.device)
        native_mixers().moe_topk(idx, wts, z, correction, top, groups, keep)
        return idx, wts
    return ref.moe_topk(z, correction, top, groups, keep)


def moe_pairs(out, h, idx, wts, wgu, wdown, limit: float):
    """Few rows (decode): out (fp32, in place) += sum_k wts[:, k] * expert_{idx[:, k]}(h),
    every (row, expert) pair streaming its expert's [gate | up] and down matrices; no
    host round trip, so the step can be captured in a hipGraph."""
    if out.is_cuda:
        native_mixers().moe_pairs(out, h, idx, wts, wgu, wdown, float(limit))
    else:
        ref.moe_pairs(out, h, idx, wts, wgu, wdown, limit)


def clamp_swiglu(gu, limit: float):
    """[gate | up (| extra)] rows -> min(gate, limit) * sigmoid(1.702 gate') * (clamp(up) + 1)."""
    if gu.is_cuda:
        ff = gu.shape[1] // 2
        out = torch.empty(gu.shape[0], ff, dtype=gu.dtype, device=gu.device)
        native_mixers().clamp_swiglu(out, gu, float(limit))
        return out
    return ref.clamp_swiglu(gu, limit)


def relu_sq(x):
    if x.is_cuda:
        native_mixers().relu_sq(x)
        return x
    return ref.relu_sq(x)


def side_gate(gpre, table, ids, col0: int, sd: int):
    """gelu_tanh(gpre) * table[ids, col0:col0+sd]."""
    if gpre.is_cuda:
        out = torch.empty_like(gpre)
        native_mixers().side_gate(out, gpre, table, ids, col0)
        return out
    return ref.side_gate(gpre, table, ids, col0, sd)


def scale_add_rows(out, y, rows, weights, sigmoid: bool = False):
    """out[rows[i]] += w_i * y[i] (fp32 out; rows None = identity; w = sigmoid(weights)
    if ``sigmoid``).  ``rows`` must not repeat within one call."""
    if out.is_cuda:
        native_mixers().scale_add_rows(out, y, rows, weights, sigmoid)
    else:
        ref.scale_add_rows(out, y, rows, weights, sigmoid)
