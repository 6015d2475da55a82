"""A plain, slow fp32 implementation of the Nulazen design, one function per mechanism,
written from the design's equations.  It shares no code with the package: the tests
compare the framework's model, cache, scheduler and kernels against it.

A model is (cfg, P): cfg the dict that config.json holds, P a dict name -> fp32 tensor.
Everything works on one whole sequence [T, ...] at positions 0..T-1.
"""
import math

import torch


def rms(x, eps, w=None):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def rotate(x, dims, base):
    """x [T, ..., n]: pairs (i, i + dims/2), i < dims/2, turned by angle t * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    out = x.clone()
    for t in range(T):
        for i in range(half):
            ang = torch.tensor(float(t), dtype=torch.float32) * \
                torch.tensor(float(base), dtype=torch.float32) ** (-2.0 * i / dims)
            c, s = torch.cos(ang), torch.sin(ang)
            u, v = x[t, ..., i], x[t, ..., i + half]
            out[t, ..., i] = u * c - v * s
            out[t, ..., i + half] = v * c + u * s
    return out


def latent_attention(h, P, p, m, eps):
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot", {})
    dims, base = rot.get("dims", dr), rot.get("base", 10000.0)
    q = (h @ P[p + "q"].T).view(T, H, dn + dr)
    down = h @ P[p + "dkv"].T
    c = rms(down[:, :r], eps, P[p + "dkv.norm"])
    k_rot = rotate(down[:, r:], dims, base)                 # [T, dr], one for all heads
    q_rot = rotate(q[:, :, dn:], dims, base)                # [T, H, dr]
    k_plain = (c @ P[p + "uk"].T).view(T, H, dn)
    val = (c @ P[p + "uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv)
    for i in range(T):
        for hh in range(H):
            sc = (k_plain[: i + 1, hh] @ q[i, hh, :dn] + k_rot[: i + 1] @ q_rot[i, hh]) * m["scale"]
            w = torch.softmax(sc, 0)
            out[i, hh] = (w[:, None] * val[: i + 1, hh]).sum(0)
    return out.reshape(T, H * dv) @ P[p + "o"].T


def causal_conv_silu(x, w):
    """x [T, C], w [C, taps]; the last tap multiplies the current row, zeros before row 0."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += x[src] * w[:, j]
    return y * torch.sigmoid(y)


def channel_delta(h, P, p, m, eps):
    T = h.shape[0]
    H, KH, dk, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = causal_conv_silu(h @ P[p + "q"].T, P[p + "q.conv"]).view(T, KH, dk)
    k = causal_conv_silu(h @ P[p + "k"].T, P[p + "k.conv"]).view(T, KH, dk)
    v = causal_conv_silu(h @ P[p + "v"].T, P[p + "v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ P[p + "b"].T)                                    # [T, H]
    pre = ((h @ P[p + "a1"].T) @ P[p + "a2"].T + P[p + "dt_bias"]).view(T, H, dk)
    decay = torch.exp(-torch.exp(P[p + "A_log"])[None, :, None] * torch.log1p(torch.exp(pre)))
    out = torch.zeros(T, H, dv)
    for hh in range(H):
        kh = hh // (H // KH)
        S = torch.zeros(dk, dv)
        for t in range(T):
            S = decay[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hh] = S.T @ q[t, kh]
    out = rms(out, eps) * P[p + "norm"]
    gate = torch.sigmoid((h @ P[p + "g1"].T) @ P[p + "g2"].T).view(T, H, dv)
    return (out * gate).reshape(T, H * dv) @ P[p + "o"].T


def dense_ff(h, P, p):
    return torch.relu(h @ P[p + "up"].T) ** 2 @ P[p + "down"].T


def glu_expert(h, P, p, limit):
    g = torch.minimum(h @ P[p + "gate"].T, torch.tensor(float(limit)))
    u = torch.clamp(h @ P[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ P[p + "down"].T


def route(h, P, p, r):
    """Per token: (chosen expert ids, their weights)."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ P[p + "router"].T, -1)
    chosen = []
    for t in range(h.shape[0]):
        pick = (s[t] + P[p + "correction"]).clone()
        grp = r.get("groups")
        if grp and grp["keep"] < grp["count"]:
            size = E // grp["count"]
            best = torch.stack([pick[g * size:(g + 1) * size].max() for g in range(grp["count"])])
            kept = set(torch.argsort(best, descending=True)[: grp["keep"]].tolist())
            for e in range(E):
                if e // size not in kept:
                    pick[e] = float("-inf")
        ids = torch.argsort(pick, descending=True)[:top].tolist()
        chosen.append((ids, [s[t, e] for e in ids]))
    return chosen


def moe_ff(h, P, p, m):
    out = torch.zeros(h.shape[0], P[p + "e0.down"].shape[0])
    for t, (ids, ws) in enumerate(route(h, P, p, m["router"])):
        for e, w in zip(ids, ws):
            out[t] += w * glu_expert(h[t:t + 1], P, p + f"e{e}.", m["expert"]["limit"])[0]
    if m.get("shared"):
        out = out + torch.sigmoid(h @ P[p + "shared.sg"].T) * glu_expert(h, P, p + "shared.", m["shared"]["limit"])
    return out


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def run_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(lp["start"])]
    for t in range(lp["times"]):
        order += [(i, t if i == lp["start"] else None) for i in range(lp["start"], lp["stop"])]
    return order + [(i, None) for i in range(lp["stop"], n)]


def forward(cfg, P, tokens, taps=None):
    """Logits [T, vocab] of one whole sequence; ``taps`` collects the residual after every layer run."""
    eps = cfg["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    x = P["embed"][tok]
    for i, step in run_order(cfg):
        if step is not None:
            x = x + P["loop.step"][step]
        l, p = cfg["layers"][i], f"l{i}."
        mix = latent_attention if l["type"] == "latent_attention" else channel_delta
        x = x + rms(mix(rms(x, eps, P[p + "norm1"]), P, p + "mix.", l["mixer"], eps), eps, P[p + "norm1b"])
        if l.get("mlp") is not None:
            hh = rms(x, eps, P[p + "norm2"])
            y = dense_ff(hh, P, p + "mlp.") if l["mlp"]["kind"] == "dense" else moe_ff(hh, P, p + "mlp.", l["mlp"])
            x = x + rms(y, eps, P[p + "norm2b"])
        if cfg.get("token_side"):
            sd = cfg["token_side"]["dim"]
            e = P["side.embed"][tok][:, i * sd:(i + 1) * sd]
            y = (gelu_tanh(x @ P[p + "side.gate"].T) * e) @ P[p + "side.proj"].T
            x = x + rms(y, eps) * P[p + "side.norm"]
        if taps is not None:
            taps.append(x.clone())
    return rms(x, eps, P["final.norm"]) @ P["head"].T
