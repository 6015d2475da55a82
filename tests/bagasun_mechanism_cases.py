"""Each Bagasun mechanism of models/mixers.py (and the ops under it) alone against the
oracle's function for it: one whole sequence, then the same sequence cut in two steps
through the cache / state the first step left; with and without the banded products."""
import torch

import bagasun_oracle as O

from fasttalk_llm_microservice_amd.models import mixers as X
from fasttalk_llm_microservice_amd.ops import mixers as M

CASES = ["rope_scaling", "sigmoid", "sigmoid_products", "sigmoid_window_edge", "sigmoid_far_key", "diff",
         "diff_products", "diff_no_rot_one_kv", "diff_window_edge", "ssm", "ssm_one_group_one_tap", "ssm_wide",
         "ssm_slow_decay", "gated_ff", "scalar_norm_and_embed"]
EPS = 1e-5


def _rand(g, *shape, s=1.0):
    return (torch.randn(*shape, generator=g) * s).bfloat16().float()


def _ctx(T, device, cut=None, page=4, slot=1, host=False):
    """StepContexts of one sequence of T rows: whole, or [0, cut) then [cut, T)."""
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)   # noqa: E731
    nb = (T + page - 1) // page
    table = list(range(nb - 1, -1, -1))            # pages in reverse order
    out = []
    for a, b in ([(0, T)] if cut is None else [(0, cut), (cut, T)]):
        pos = list(range(a, b))
        seg = M.Segments(start=i32([0, b - a]), pos0=i32([a]), slot=i32([slot]), kv_len=i32([b]),
                         block_tables=i32([table]), num=1, max_rows=b - a, max_kv=b,
                         host=([0, b - a], [a], [b]) if host else None)
        slots = [table[p // page] * page + p % page for p in pos]
        out.append((a, b, X.StepContext(None, i32(pos), i32(slots), seg)))
    return out


def _tol(dtype):
    return dict(rtol=3e-4, atol=3e-4) if dtype == torch.float32 else dict(rtol=6e-2, atol=6e-2)


def _close(got, want, dtype):
    """fp32: sharp.  bf16: rounding of the activations, measured against the output's size."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=3e-4, atol=3e-4)
    else:
        assert float((got - want).abs().max()) <= 0.05 * float(want.abs().max()) + 0.02


def _run_attention(mix, h, T, device, dtype, cuts, host, page=4):
    outs = []
    for cut in cuts:
        cache = mix.alloc_cache((T + page - 1) // page, page, dtype, 0, device)
        outs.append(torch.cat([mix(h[a:b].to(device, dtype), ctx, cache).float().cpu()
                               for a, b, ctx in _ctx(T, device, cut, page=page, host=host)]))
    return outs


def _sigmoid_weights(g, W, H, G, dk, dv):
    return {"q": _rand(g, H * dk, W, s=0.4), "k": _rand(g, G * dk, W, s=0.4), "v": _rand(g, G * dv, W, s=0.4),
            "q.b": _rand(g, H * dk, s=0.2), "k.b": _rand(g, G * dk, s=0.2), "v.b": _rand(g, G * dv, s=0.2),
            "q.norm": 1 + _rand(g, H * dk, s=0.2), "k.norm": 1 + _rand(g, G * dk, s=0.2),
            "r1": _rand(g, H, s=0.3).abs() + 0.2, "r2": _rand(g, H, s=0.3).abs() + 0.3, "pb": _rand(g, H, s=0.5) - 0.5,
            "o": _rand(g, W, H * dv, s=0.3)}


def _sigmoid(device, dtype, host, T=45, window=9, H=4, G=2, dk=10, dv=7, cuts=(None, 1, 2, 13, 36), tweak=None,
             rows=None):
    g = torch.Generator().manual_seed(3)
    W = 40
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "mask": {"size": window}, "scale": 0.3}
    P = _sigmoid_weights(g, W, H, G, dk, dv)
    h = _rand(g, T, W)
    if tweak:
        tweak(P, h)
    want = O.sigmoid_attention(P, "", m, h, EPS)
    mix = X.SigmoidAttention(P.__getitem__, W, H, G, dk, dv, window, 0.3, EPS, dtype, device)
    for got in _run_attention(mix, h, T, device, dtype, cuts, host):
        _close(got if rows is None else got[rows], want if rows is None else want[rows], dtype)
    return want


def _diff(device, dtype, host, T=45, window=11, H=4, G=2, dk=8, dv=12, dims=4, scaling=(3.0, 1.0, 5.0, 40),
          cuts=(None, 1, 2, 13, 36), tweak=None):
    g = torch.Generator().manual_seed(4)
    W = 40
    rot = {"dims": dims, "base": 30.0}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "mask": {"size": window}, "scale": 0.4, "diff": 0.35,
         "rot": rot if dims else None}
    P = {"q": _rand(g, H * 2 * dk, W, s=0.5), "k": _rand(g, G * 2 * dk, W, s=0.5), "v": _rand(g, G * dv, W, s=0.4),
         "g": _rand(g, H, W, s=0.4), "o": _rand(g, W, H * dv, s=0.3)}
    P.update({n: _rand(g, dk, s=0.3) for n in ("lq1", "lk1", "lq2", "lk2")})
    h = _rand(g, T, W)
    if tweak:
        tweak(P, h)
    want = O.differential_attention(P, "", m, h, EPS)
    mix = X.DifferentialAttention(P.__getitem__, W, H, G, dk, dv, window, 0.4, 0.35, dims, 30.0, scaling, EPS,
                                  dtype, device, 128)
    for got in _run_attention(mix, h, T, device, dtype, cuts, host):
        _close(got, want, dtype)


def _edge_tweak(window, T):
    """Inputs so that, for the last row, the key just outside the window would dominate
    if it were seen, and the key just inside it carries most of the visible weight."""
    def tweak(P, h):
        h[T - 1 - window] = h[T - 1] * 3.0            # just outside: aligned with the query's input
        h[T - window] = h[T - 1] * 2.0                # just inside
        for n in ("q", "k"):
            P[n].copy_((P["q"][:P[n].shape[0]] if n == "k" else P[n]))   # keys made from the query rows
    return tweak


def _ssm(device, dtype, heads, vdim, n, groups, taps, norm_groups, T=37, a_log=None):
    g = torch.Generator().manual_seed(5)
    W = 36
    inner, ch = heads * vdim, heads * vdim + 2 * groups * n
    m = {"heads": heads, "vdim": vdim, "state": n, "groups": groups, "conv": taps, "norm_groups": norm_groups}
    P = {"in": _rand(g, inner + ch + heads, W, s=0.4), "conv": _rand(g, ch, taps, s=0.6), "conv.b": _rand(g, ch, s=0.2),
         "dt_bias": _rand(g, heads) - 1.0, "A_log": _rand(g, heads, s=0.5) - 1.0, "D": 1 + _rand(g, heads, s=0.2),
         "norm": 1 + _rand(g, inner, s=0.1), "o": _rand(g, W, inner, s=0.3)}
    if a_log is not None:
        P["A_log"].fill_(a_log)
    h = _rand(g, T, W)
    want = O.mamba2(P, "", m, h, EPS)
    mix = X.StateSpaceMixer(P.__getitem__, W, heads, vdim, n, groups, taps, norm_groups, EPS, dtype, device)
    for cut in (None, 1, 2, 17, 35):
        state = tuple(torch.full_like(s, 7.0) for s in mix.alloc_cache(0, 0, dtype, 3, device))
        got = torch.cat([mix(h[a:b].to(device, dtype), ctx, state).float().cpu() for a, b, ctx in _ctx(T, device, cut)])
        _close(got, want, dtype)
        assert float(state[0][0].min()) == 7.0 and float(state[0][2].max()) == 7.0   # other slots untouched
    if a_log is not None:
        # the state matters: with the first row changed the last output differs
        h2 = h.clone()
        h2[0] += 1.0
        assert (O.mamba2(P, "", m, h2, EPS)[-1] - want[-1]).abs().max() > 1e-3


def run(case, device, dtype):
    g = torch.Generator().manual_seed(1)
    if case == "rope_scaling":
        for sc in (None, (5.0, 1.0, 3.0, 64), (8.0, 0.5, 3.0, 20)):
            scaling = dict(zip(("factor", "low", "high", "original"), sc)) if sc else None
            f = O.rotary_frequencies(8, 37.0, scaling)
            tab = M.rope_table(50, 8, 37.0, scaling=sc)
            ang = torch.arange(50, dtype=torch.float32)[:, None] * f[None]
            torch.testing.assert_close(tab, torch.cat([ang.cos(), ang.sin()], -1), rtol=1e-5, atol=2e-5)
        # all three branches of the rescaling occur in the second table
        f0 = O.rotary_frequencies(8, 37.0)
        f1 = O.rotary_frequencies(8, 37.0, {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 64})
        ratio = (f1 / f0).tolist()
        assert ratio[0] == 1.0 and abs(ratio[-1] - 0.2) < 1e-6 and any(0.21 < r < 0.99 for r in ratio)
    elif case == "sigmoid":
        _sigmoid(device, dtype, host=False)
    elif case == "sigmoid_products":
        _sigmoid(device, dtype, host=True, T=77, window=9, cuts=(None, 33, 40))
        _sigmoid(device, dtype, host=True, T=77, window=50, H=3, G=3, dk=16, dv=70, cuts=(None, 35))
    elif case == "sigmoid_window_edge":
        for host in (False, True):
            _sigmoid(device, dtype, host=host, T=40, window=6, cuts=(None, 3, 34, 35), tweak=_edge_tweak(6, 40))
    elif case == "sigmoid_far_key":
        # a window longer than the sequence; the first token's value is large, so its
        # weight (no normalisation: it does not fade among hundreds of keys) shows in every row
        def tweak(P, h):
            h[0] *= 4.0
        for host in (False, True):
            _sigmoid(device, dtype, host=host, T=230, window=1000, cuts=(None, 229, 100), tweak=tweak)
    elif case == "diff":
        _diff(device, dtype, host=False)
    elif case == "diff_products":
        _diff(device, dtype, host=True, T=80, cuts=(None, 33, 47))
    elif case == "diff_no_rot_one_kv":
        _diff(device, dtype, host=False, H=3, G=1, dk=6, dv=5, dims=0, scaling=None, window=200)
        _diff(device, dtype, host=False, H=2, G=2, dk=6, dv=5, dims=6, scaling=None, window=1)
    elif case == "diff_window_edge":
        def tweak(P, h):
            P["q"] *= 4.0        # peaked maps: a lost or extra key moves the whole row
        for host in (False, True):
            _diff(device, dtype, host=host, T=70, window=33, cuts=(None, 32, 33, 34), tweak=tweak)
    elif case == "ssm":
        _ssm(device, dtype, 4, 8, 12, 2, 3, 2)
    elif case == "ssm_one_group_one_tap":
        _ssm(device, dtype, 3, 5, 7, 1, 1, 1)
    elif case == "ssm_wide":
        _ssm(device, dtype, 2, 40, 70, 2, 4, 4)
    elif case == "ssm_slow_decay":
        _ssm(device, dtype, 2, 6, 9, 1, 2, 1, T=150, a_log=-7.0)
    elif case == "gated_ff":
        P = {"gate": _rand(g, 24, 16, s=0.5), "up": _rand(g, 24, 16, s=0.5), "down": _rand(g, 16, 24, s=0.4)}
        h = _rand(g, 9, 16)
        got = X.GatedFF(P.__getitem__, dtype, device)(h.to(device, dtype)).float().cpu()
        torch.testing.assert_close(got, O.feed_forward(P, "", h), **_tol(dtype))
    elif case == "scalar_norm_and_embed":
        table = _rand(g, 11, 20)
        ids = torch.tensor([3, 0, 10, 3], dtype=torch.int32)
        x = M.embed_rows(ids.to(device), table.to(device, dtype), 2.5)
        torch.testing.assert_close(x.cpu(), table[ids.long()].to(dtype).float() * 2.5)
        w = torch.full((20,), 1.3, device=device)
        y = _rand(g, 4, 20).to(device)
        res = x.clone()
        out, _ = M.add_rms_norm_rows(res, y, w, EPS, next_w=w, out_dtype=torch.float32)
        want = x.cpu() + O.unit_rms(y.cpu(), EPS) * 1.3
        torch.testing.assert_close(res.cpu(), want, rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(out.cpu(), O.unit_rms(want, EPS) * 1.3, rtol=1e-5, atol=1e-5)
    else:
        raise KeyError(case)
