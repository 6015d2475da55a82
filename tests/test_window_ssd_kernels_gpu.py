"""HIP kernels of the windowed attention and the state-space scan against the PyTorch
implementation of the same op (ops.mixers_ref) on identical inputs: fp32 and bf16
activations and caches, odd sizes, several segments per step (continuing, fresh,
one-row), shuffled pages, windows inside and across pages, padding segments."""
import pytest
import torch

from fasttalk_llm_microservice_amd.ops import mixers as M
from fasttalk_llm_microservice_amd.ops import mixers_ref as R
from test_mixer_kernels_gpu import DEV, DTYPES, make_seg, rnd, to_dev, tol

pytestmark = pytest.mark.gpu


def _spec(heads, kv, dk, dv, window, maps, sigmoid, g, dev="cpu"):
    hq = heads * maps
    r = lambda lo, hi: (lo + (hi - lo) * torch.rand(hq, generator=g)).to(dev)   # noqa: E731
    return M.WindowSpec(heads, kv, dk, dv, window, 0.3, maps=maps, sigmoid=sigmoid,
                        r1=r(0.1, 0.6) if sigmoid else None, r2=r(0.2, 1.0) if sigmoid else None,
                        pb=r(-1.0, 0.5) if sigmoid else None)


def _spec_dev(sp):
    mv = lambda t: t.to(DEV) if t is not None else None   # noqa: E731
    return M.WindowSpec(sp.heads, sp.kv_heads, sp.dk, sp.dv, sp.window, sp.scale, sp.maps, sp.sigmoid,
                        mv(sp.r1), mv(sp.r2), mv(sp.pb))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("norm,rot", [(True, 0), (False, 6), (False, 0), (True, 4)])
def test_attn_prep(dt, norm, rot):
    g = torch.Generator().manual_seed(2)
    nq, nk, nv, hd = 4 * 10, 2 * 10, 2 * 7, 10
    seg, blocks = make_seg([5, 1, 9], [3, 20, 0], [0, 1, 2])
    t = 15
    qkv = rnd(t, nq + nk + nv + 3, dt=dt, g=g)[:, :nq + nk + nv]       # rows wider than the op's part
    wq, wk = (1 + rnd(nq, g=g, scale=0.2), 1 + rnd(nk, g=g, scale=0.2)) if norm else (None, None)
    table = M.rope_table(40, rot, 50.0, scaling=(3.0, 0.5, 2.0, 30)) if rot else None
    pos = torch.tensor([3, 4, 5, 6, 7, 20, 0, 1, 2, 3, 4, 5, 6, 7, 8], dtype=torch.int32)
    slots = torch.randperm(blocks * 4)[:t].int()
    slots[4] = -1                                                       # a padding row writes nothing
    kc1, vc1 = torch.zeros(blocks, 4, nk, dtype=dt), torch.zeros(blocks, 4, nv, dtype=dt)
    kc2, vc2 = kc1.to(DEV), vc1.to(DEV)
    q1 = R.attn_prep(qkv, nq, nk, wq, wk, 1e-5, table, rot, hd, pos, slots, kc1, vc1)
    mv = lambda x: x.to(DEV) if x is not None else None   # noqa: E731
    q2 = M.attn_prep(qkv.to(DEV), nq, nk, mv(wq), mv(wk), 1e-5, mv(table), rot, hd, pos.to(DEV), slots.to(DEV), kc2, vc2)
    torch.testing.assert_close(q2.cpu(), q1, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(kc2.cpu().float(), kc1.float(), **tol(dt))
    torch.testing.assert_close(vc2.cpu().float(), vc1.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("heads,kv,dk,dv,window,maps,sigmoid", [
    (4, 2, 16, 24, 7, 1, True), (3, 3, 10, 70, 0, 1, True), (4, 1, 8, 12, 5, 2, False),
    (2, 2, 128, 128, 130, 2, False), (6, 2, 96, 200, 300, 1, False), (2, 1, 7, 5, 1, 1, False)])
def test_window_attention_rows(dt, heads, kv, dk, dv, window, maps, sigmoid):
    g = torch.Generator().manual_seed(3)
    lens, pos0 = [6, 1, 1, 31, 1], [250, 0, 129, 7, 4]
    seg, blocks = make_seg(lens, pos0, [0, 1, 2, 3, 4], block_size=16)
    seg.kv_len[4] = 0                                                   # a padding row: empty context
    t = sum(lens)
    sp = _spec(heads, kv, dk, dv, window, maps, sigmoid, g)
    q = rnd(t, heads * maps * dk, g=g)
    kc = rnd(blocks, 16, kv * maps * dk, dt=dt, g=g)
    vc = rnd(blocks, 16, kv * dv, dt=dt, g=g)
    want = R.window_attention(q, kc, vc, seg, heads, maps, kv, dk, dv, window, sp.scale, sigmoid, sp.r1, sp.r2, sp.pb)
    got = M.window_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), to_dev(seg), _spec_dev(sp))
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    assert float(got[-1].abs().max()) == 0.0


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("heads,kv,dk,dv,window,maps,sigmoid", [
    (4, 2, 16, 24, 7, 1, True), (4, 1, 8, 12, 40, 2, False), (2, 2, 64, 64, 300, 2, False), (3, 1, 10, 9, 0, 1, True)])
def test_window_attention_products_match_rows(dt, heads, kv, dk, dv, window, maps, sigmoid):
    """Segments of 32 rows or more through the banded products, the others through the
    per-row kernel, against the per-row kernel on all of them."""
    g = torch.Generator().manual_seed(4)
    lens, pos0 = [40, 1, 300, 5], [100, 9, 0, 30]
    seg, blocks = make_seg(lens, pos0, [0, 1, 2, 3], block_size=16)
    seg = to_dev(seg)
    t = sum(lens)
    sp = _spec_dev(_spec(heads, kv, dk, dv, window, maps, sigmoid, g))
    q = rnd(t, heads * maps * dk, g=g).to(DEV)
    kc = rnd(blocks, 16, kv * maps * dk, dt=dt, g=g).to(DEV)
    vc = rnd(blocks, 16, kv * dv, dt=dt, g=g).to(DEV)
    want = M.window_attention(q, kc, vc, seg, sp)
    seg.host = (seg.start.tolist(), seg.pos0.tolist(), seg.kv_len.tolist())
    got = torch.zeros_like(want)
    M.window_attention(q, kc, vc, seg, sp, skip_from=32, out=got)
    old = M.PRODUCT_CHUNK_ROWS
    M.PRODUCT_CHUNK_ROWS = 64                                           # several chunks per segment
    try:
        M.window_attention_products(got, q, kc, vc, seg, sp, 32)
    finally:
        M.PRODUCT_CHUNK_ROWS = old
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dt", DTYPES)
def test_diff_combine_and_gate_group_norm_and_glu(dt):
    g = torch.Generator().manual_seed(5)
    t, heads, dv = 9, 3, 70
    a = rnd(t, heads * 2, dv, g=g)
    wide = rnd(t, heads + 5, dt=dt, g=g)
    gate = wide[:, 2:2 + heads]
    want = R.diff_combine(a, gate, 0.37, 0.4, 1e-5, heads, dv, dt)
    got = M.diff_combine(a.to(DEV), wide.to(DEV)[:, 2:2 + heads], 0.37, 0.4, 1e-5, heads, dv, dt)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    for groups, n in ((1, 96), (4, 96), (3, 210)):
        y, w = rnd(t, n, g=g), 1 + rnd(n, g=g, scale=0.1)
        zw = rnd(t, n + 7, dt=dt, g=g)
        want = R.gate_group_norm(y, zw[:, 7:], w, 1e-5, groups, dt)
        got = M.gate_group_norm(y.to(DEV), zw.to(DEV)[:, 7:], w.to(DEV), 1e-5, groups, dt)
        torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt))
    gu = rnd(t, 2 * 50, dt=dt, g=g)
    torch.testing.assert_close(M.gelu_glu(gu.to(DEV)).cpu().float(), R.gelu_glu(gu).float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("heads,groups,n,dv,taps", [(4, 2, 12, 8, 3), (3, 1, 7, 40, 1), (2, 2, 128, 64, 4), (2, 1, 200, 33, 2)])
def test_conv_and_ssd_scan(dt, heads, groups, n, dv, taps):
    g = torch.Generator().manual_seed(6)
    lens, pos0, slots = [19, 1, 40, 1, 3], [5, 77, 0, 0, 2], [2, 0, 3, 1, -1]     # the last one is padding
    seg, _ = make_seg(lens, pos0, slots)
    t = sum(lens)
    inner, ch = heads * dv, heads * dv + 2 * groups * n
    wide = rnd(t, inner + ch + heads, dt=dt, g=g, scale=0.7)
    w, b = rnd(ch, taps, g=g, scale=0.6), rnd(ch, g=g, scale=0.2)
    a_log, dt_bias, skip = rnd(heads, g=g, scale=0.5) - 1.0, rnd(heads, g=g) - 1.0, 1 + rnd(heads, g=g, scale=0.2)
    hist1, st1 = rnd(4, max(taps - 1, 0), ch, g=g), rnd(4, heads, n, dv, g=g)
    hist2, st2 = hist1.to(DEV), st1.to(DEV)
    x1 = R.short_conv_silu(wide[:, inner:inner + ch], w, hist1, seg, b)
    y1 = R.ssd_scan(x1, wide[:, inner + ch:], a_log, dt_bias, skip, st1, seg, heads, groups, n, dv)
    wd = wide.to(DEV)
    x2 = M.short_conv_silu(wd[:, inner:inner + ch], w.to(DEV), hist2, to_dev(seg), b.to(DEV))
    live = sum(lens[:4])
    torch.testing.assert_close(x2.cpu().float()[:live], x1.float()[:live], **tol(dt))
    torch.testing.assert_close(hist2.cpu(), hist1, rtol=1e-6, atol=1e-6)
    # the scan itself on identical inputs
    y2 = M.ssd_scan(x1.to(DEV), wd[:, inner + ch:], a_log.to(DEV), dt_bias.to(DEV), skip.to(DEV), st2, to_dev(seg),
                    heads, groups, n, dv)
    torch.testing.assert_close(y2.cpu()[:live], y1[:live], rtol=2e-4, atol=2e-4)
    torch.testing.assert_close(st2.cpu(), st1, rtol=2e-4, atol=2e-4)
    assert float(y2[live:].abs().max()) == 0.0
