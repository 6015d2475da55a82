"""HIP kernels of ops.mixers against the PyTorch implementation of the same op
(ops.mixers_ref) on identical inputs: fp32 and bf16 activations, odd sizes, segments
that start at position 0 and segments that continue, padding segments, reused slots."""
import pytest
import torch

from fasttalk_llm_microservice_amd.ops import mixers as M
from fasttalk_llm_microservice_amd.ops import mixers_ref as R

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dt):
    return dict(rtol=2e-5, atol=2e-5) if dt == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def rnd(*shape, dt=torch.float32, g=None, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(dt)


def make_seg(lens, pos0, slots, block_size=4, dev="cpu", shuffle_blocks=True):
    """Segments for rows of the given lengths; block tables cover pos0 + len tokens."""
    start = [0]
    for n in lens:
        start.append(start[-1] + n)
    kv = [p + n for p, n in zip(pos0, lens)]
    nb = [(k + block_size - 1) // block_size for k in kv]
    total = sum(nb)
    perm = torch.randperm(total).tolist() if shuffle_blocks else list(range(total))
    bt = torch.zeros(len(lens), max(nb + [1]), dtype=torch.int32)
    k = 0
    for i, n in enumerate(nb):
        bt[i, :n] = torch.tensor(perm[k:k + n], dtype=torch.int32)
        k += n
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)   # noqa: E731
    seg = M.Segments(start=i32(start), pos0=i32(pos0), slot=i32(slots), kv_len=i32(kv),
                     block_tables=bt.to(dev), num=len(lens), max_rows=max(lens), max_kv=max(kv))
    return seg, total


def to_dev(seg):
    return M.Segments(seg.start.to(DEV), seg.pos0.to(DEV), seg.slot.to(DEV), seg.kv_len.to(DEV),
                      seg.block_tables.to(DEV), seg.num, seg.max_rows, seg.max_kv)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("width", [96, 2048, 1000])
def test_add_rms_norm_variants(dt, width):
    g = torch.Generator().manual_seed(1)
    x = rnd(7, width, g=g)
    y = rnd(7, width, dt=dt, g=g)
    wb, nw, vec = rnd(width, g=g), rnd(width, g=g), rnd(width, g=g)
    for add_vec in (None, vec):
        for next_w in (None, nw):
            for want_cast in (False, True):
                xc, xg = x.clone(), x.clone().to(DEV)
                o1, c1 = R.add_rms_norm_rows(xc, y, wb, 1e-5, add_vec, next_w, dt, want_cast)
                o2, c2 = M.add_rms_norm_rows(xg, y.to(DEV), wb.to(DEV), 1e-5,
                                             add_vec.to(DEV) if add_vec is not None else None,
                                             next_w.to(DEV) if next_w is not None else None, dt, want_cast)
                torch.testing.assert_close(xg.cpu(), xc, rtol=1e-5, atol=1e-5)
                if next_w is not None:
                    torch.testing.assert_close(o2.cpu().float(), o1.float(), **tol(dt))
                if want_cast:
                    torch.testing.assert_close(c2.cpu().float(), c1.float(), **tol(dt))
    # fp32 expert sums into a bf16 norm output
    xc, xg = x.clone(), x.clone().to(DEV)
    yf = rnd(7, width, g=g)
    o1, _ = R.add_rms_norm_rows(xc, yf, wb, 1e-5, None, nw, dt, False)
    o2, _ = M.add_rms_norm_rows(xg, yf.to(DEV), wb.to(DEV), 1e-5, None, nw.to(DEV), dt, False)
    torch.testing.assert_close(o2.cpu().float(), o1.float(), **tol(dt))
    h1 = R.rms_norm_rows(x.clone(), nw, 1e-5, dt, vec)
    h2 = M.rms_norm_rows(x.clone().to(DEV), nw.to(DEV), 1e-5, dt, vec.to(DEV))
    torch.testing.assert_close(h2.cpu().float(), h1.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_and_elementwise(dt):
    g = torch.Generator().manual_seed(2)
    table = rnd(50, 72, dt=dt, g=g)
    ids = torch.randint(0, 50, (9,), generator=g, dtype=torch.int32)
    torch.testing.assert_close(M.embed_rows(ids.to(DEV), table.to(DEV)).cpu(), R.embed_rows(ids, table))
    x = rnd(5, 33, dt=dt, g=g)
    torch.testing.assert_close(M.relu_sq(x.clone().to(DEV)).cpu().float(), R.relu_sq(x).float(), **tol(dt))
    for cols in (2 * 24, 2 * 24 + 1):
        gu = rnd(6, cols, dt=dt, g=g, scale=2.0)
        torch.testing.assert_close(M.clamp_swiglu(gu.to(DEV), 1.5).cpu().float(),
                                   R.clamp_swiglu(gu, 1.5).float(), **tol(dt))
    gp = rnd(9, 8, dt=dt, g=g)
    side = rnd(50, 40, dt=dt, g=g)
    torch.testing.assert_close(M.side_gate(gp.to(DEV), side.to(DEV), ids.to(DEV), 16, 8).cpu().float(),
                               R.side_gate(gp, side, ids, 16, 8).float(), **tol(dt))
    o = rnd(4, 3 * 20, g=g)
    gate = rnd(4, 3 * 20, dt=dt, g=g)
    w = rnd(20, g=g)
    torch.testing.assert_close(M.head_rms_gate(o.to(DEV), w.to(DEV), gate.to(DEV), 1e-5, 3, 20, dt).cpu().float(),
                               R.head_rms_gate(o, w, gate, 1e-5, 3, 20, dt).float(), **tol(dt))
    out = rnd(10, 48, g=g)
    y = rnd(4, 48, dt=dt, g=g)
    rows = torch.tensor([7, 0, 3, 9], dtype=torch.int32)
    wts = rnd(4, g=g)
    o1, o2 = out.clone(), out.clone().to(DEV)
    R.scale_add_rows(o1, y, rows, wts, False)
    M.scale_add_rows(o2, y.to(DEV), rows.to(DEV), wts.to(DEV), False)
    torch.testing.assert_close(o2.cpu(), o1, rtol=1e-5, atol=1e-5)
    y = rnd(10, 48, dt=dt, g=g)
    wt = rnd(10, dt=dt, g=g)
    R.scale_add_rows(o1, y, None, wt, True)
    M.scale_add_rows(o2, y.to(DEV), None, wt.to(DEV), True)
    torch.testing.assert_close(o2.cpu(), o1, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_conv_segments(dt, taps):
    g = torch.Generator().manual_seed(3)
    c = 70
    lens, pos0, slots = [1, 5, 1, 2, 3], [9, 0, 0, 4, 7], [2, -1, 0, 3, 1]
    seg, _ = make_seg(lens, pos0, slots)
    x = rnd(sum(lens), c, dt=dt, g=g)
    w = rnd(c, taps, g=g)
    hist = rnd(4, taps - 1, c, g=g)
    h1, h2 = hist.clone(), hist.clone().to(DEV)
    y1 = R.short_conv_silu(x, w, h1, seg)
    y2 = M.short_conv_silu(x.to(DEV), w.to(DEV), h2, to_dev(seg))
    torch.testing.assert_close(y2.cpu().float(), y1.float(), **tol(dt))
    torch.testing.assert_close(h2.cpu(), h1)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("heads,kvh,dk,dv", [(4, 2, 16, 24), (2, 2, 64, 64), (3, 1, 40, 33), (2, 1, 128, 128),
                                             (2, 1, 200, 40), (1, 1, 3, 70)])
def test_gated_delta_rule(dt, heads, kvh, dk, dv):
    g = torch.Generator().manual_seed(4)
    lens, pos0, slots = [1, 37, 2, 1], [5, 0, 3, 0], [1, 0, -1, 2]   # 37 rows: several staged chunks
    seg, _ = make_seg(lens, pos0, slots)
    t = sum(lens)
    qkv = rnd(t, 2 * kvh * dk + heads * dv, dt=dt, g=g)
    a = rnd(t, heads * dk, dt=dt, g=g)
    b = rnd(t, heads, dt=dt, g=g)
    a_log = torch.log(0.5 + torch.rand(heads, generator=g))
    dtb = rnd(heads * dk, g=g)
    state = rnd(3, heads, dk, dv, g=g, scale=0.3)
    s1, s2 = state.clone(), state.clone().to(DEV)
    o1 = R.gated_delta_rule(qkv, a, b, a_log, dtb, s1, seg, heads, kvh, dk, dv)
    o2 = M.gated_delta_rule(qkv.to(DEV), a.to(DEV), b.to(DEV), a_log.to(DEV), dtb.to(DEV), s2, to_dev(seg),
                            heads, kvh, dk, dv)
    torch.testing.assert_close(o2.cpu(), o1, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(s2.cpu(), s1, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", DTYPES)
# (also: more than 16 heads -> several head groups; a wide row -> the head group shrinks to fit LDS)
@pytest.mark.parametrize("heads,dn,dr,rank,dims", [(3, 16, 8, 40, 8), (2, 32, 16, 64, 8), (5, 8, 4, 130, 4),
                                                    (20, 8, 4, 24, 4), (12, 8, 100, 900, 6)])
def test_latent_attention_paged(dt, heads, dn, dr, rank, dims):
    g = torch.Generator().manual_seed(5)
    bs = 4
    lens, pos0, slots = [1, 70, 3, 1], [130, 0, 66, 0], [0, 1, 2, 3]
    seg, nblocks = make_seg(lens, pos0, slots, block_size=bs)
    t = sum(lens)
    table = R.rope_table(256, dims, 10000.0)
    cache = rnd(nblocks + 2, bs, rank + dr, dt=dt, g=g)
    c1, c2 = cache.clone(), cache.clone().to(DEV)
    positions = torch.cat([torch.arange(p, p + n) for p, n in zip(pos0, lens)]).int()
    slot_map = torch.cat([seg.block_tables[i, (torch.arange(p, p + n) // bs)].long() * bs
                          + torch.arange(p, p + n) % bs for i, (p, n) in enumerate(zip(pos0, lens))]).int()
    slot_map[2] = -1   # a row whose cache write is skipped
    dkv = rnd(t, rank + dr, dt=dt, g=g)
    nw = rnd(rank, g=g)
    R.latent_kv_write(dkv, nw, 1e-5, table, dims, positions, slot_map, c1, rank)
    M.latent_kv_write(dkv.to(DEV), nw.to(DEV), 1e-5, table.to(DEV), dims, positions.to(DEV),
                      slot_map.to(DEV), c2, rank)
    torch.testing.assert_close(c2.cpu().float(), c1.float(), **tol(dt))
    q = rnd(t, heads * (dn + dr), dt=dt, g=g)
    qn1, qr1 = R.latent_q_rope(q, table, dims, positions, heads, dn, dr)
    qn2, qr2 = M.latent_q_rope(q.to(DEV), table.to(DEV), dims, positions.to(DEV), heads, dn, dr)
    torch.testing.assert_close(qn2.cpu(), qn1)
    torch.testing.assert_close(qr2.cpu(), qr1, rtol=1e-5, atol=1e-5)
    qa = rnd(heads, t, rank, g=g, scale=0.5)
    o1 = R.latent_attention(qa, qr1, c1, seg, 0.2, rank)
    o2 = M.latent_attention(qa.to(DEV), qr1.to(DEV), c1.to(DEV), to_dev(seg), 0.2, rank)
    torch.testing.assert_close(o2.cpu(), o1, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("experts,top,groups,keep", [(8, 4, 4, 3), (6, 2, 1, 1), (64, 6, 8, 3), (130, 5, 1, 1),
                                                     (12, 1, 3, 1)])
def test_moe_topk(experts, top, groups, keep):
    g = torch.Generator().manual_seed(6)
    z = rnd(33, experts, g=g, scale=2.0)
    corr = rnd(experts, g=g, scale=0.3)   # biased scores may be negative
    i1, w1 = R.moe_topk(z, corr, top, groups, keep)
    i2, w2 = M.moe_topk(z.to(DEV), corr.to(DEV), top, groups, keep)
    assert torch.equal(i2.cpu().sort(-1).values, i1.sort(-1).values)
    torch.testing.assert_close(w2.cpu().sort(-1).values, w1.sort(-1).values, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dt", DTYPES)
def test_causal_softmax(dt):
    g = torch.Generator().manual_seed(7)
    s = rnd(3 * 5, 23, g=g, scale=3.0)
    p1 = R.causal_softmax(s, 5, 17, 0.4, dt)
    p2 = M.causal_softmax(s.to(DEV), 5, 17, 0.4, dt)
    torch.testing.assert_close(p2.cpu().float(), p1.float(), **tol(dt))
    assert float(p2[0, 18:].abs().max()) == 0.0 and float(p2[4, 21]) > 0.0 and float(p2[4, 22]) == 0.0
