"""A plain, slow fp32 implementation of the Bagasun design, one function per mechanism,
written from the design's equations.  It shares no code with the package: the tests
compare the framework (engine, caches, state slots, kernels or the CPU backend) with it.

A checkpoint is a dict ``cfg`` (the parsed config.json) and a dict ``P`` of fp32
tensors.  Whole sequences only: no cache, no state carried between calls.

Notation: x residual [T, width]; u a sublayer's input; i query position, j key position.
"""
import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def band(T, size):
    """[T, T] bool: j visible from i iff 0 <= i - j < size."""
    d = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    return (d >= 0) & (d < size)


def rotary_frequencies(dims, base, scaling=None):
    """f_i for i < dims/2, with the long-context rescaling of the low frequencies."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        fac, lo, hi, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
        out = []
        for v in f:
            wl = 2.0 * math.pi / v
            if wl < orig / hi:
                out.append(v)
            elif wl > orig / lo:
                out.append(v / fac)
            else:
                s = (orig / wl - lo) / (hi - lo)
                out.append((1.0 - s) * v / fac + s * v)
        f = out
    return torch.tensor(f, dtype=torch.float32)


def rotate(x, dims, freqs):
    """x [T, heads, n]: the first ``dims`` entries of every head rotated, entry i paired
    with entry i + dims/2, by the angle position * f_i."""
    T = x.shape[0]
    ang = torch.arange(T, dtype=torch.float32)[:, None] * freqs[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    half = dims // 2
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def sigmoid_attention(P, p, m, u, eps):
    """Windowed attention without softmax: weight = sigmoid(score - distance bias + pb)."""
    T = u.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = u @ P[p + "q"].T + P[p + "q.b"]
    k = u @ P[p + "k"].T + P[p + "k.b"]
    v = u @ P[p + "v"].T + P[p + "v.b"]
    q = unit_rms(q, eps) * P[p + "q.norm"]
    k = unit_rms(k, eps) * P[p + "k.norm"]
    q, k, v = q.view(T, H, dk), k.view(T, G, dk), v.view(T, G, dv)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).float()
    vis = band(T, m["mask"]["size"])
    out = torch.zeros(T, H, dv)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * m["scale"]
        s = s - P[p + "r1"][h] * torch.log(1.0 + P[p + "r2"][h] * dist.clamp_min(0.0))
        w = torch.sigmoid(s + P[p + "pb"][h]) * vis
        out[:, h] = w @ v[:, g]
    return out.reshape(T, H * dv) @ P[p + "o"].T


def differential_attention(P, p, m, u, eps):
    """Two softmax maps per head over shared values, o = a1 - lambda a2, unit rms per
    head, times (1 - diff), times a per-head sigmoid gate of the input."""
    T = u.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (u @ P[p + "q"].T).view(T, H * 2, dk)
    k = (u @ P[p + "k"].T).view(T, G * 2, dk)
    v = (u @ P[p + "v"].T).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, rot["dims"], f), rotate(k, rot["dims"], f)
    vis = band(T, m["mask"]["size"])
    diff = m["diff"]
    lam = torch.exp((P[p + "lq1"] * P[p + "lk1"]).sum()) - torch.exp((P[p + "lq2"] * P[p + "lk2"]).sum()) + diff
    gate = torch.sigmoid(u @ P[p + "g"].T)                       # [T, H]
    out = torch.zeros(T, H, dv)
    for h in range(H):
        g = h // (H // G)
        maps = []
        for t in range(2):
            s = (q[:, 2 * h + t] @ k[:, 2 * g + t].T) * m["scale"]
            s = s.masked_fill(~vis, float("-inf"))
            maps.append(torch.softmax(s, -1) @ v[:, g])
        o = maps[0] - lam * maps[1]
        o = unit_rms(o, eps) * (1.0 - diff)
        out[:, h] = o * gate[:, h:h + 1]
    return out.reshape(T, H * dv) @ P[p + "o"].T


def mamba2(P, p, m, u, eps):
    """Selective state space layer, token by token."""
    T = u.shape[0]
    H, dv, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * dv
    zxbcdt = u @ P[p + "in"].T
    z = zxbcdt[:, :inner]
    xbc = zxbcdt[:, inner:2 * inner + 2 * G * N]
    dt = zxbcdt[:, 2 * inner + 2 * G * N:]
    # causal convolution per channel, zeros before the start; the last tap is the current token
    w, b = P[p + "conv"], P[p + "conv.b"]
    pad = torch.cat([torch.zeros(taps - 1, xbc.shape[1]), xbc], 0)
    conv = torch.stack([(pad[t:t + taps] * w.T).sum(0) for t in range(T)]) + b
    xbc = silu(conv)
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + P[p + "dt_bias"], threshold=1e9)
    rate = torch.exp(P[p + "A_log"])
    S = torch.zeros(H, N, dv)
    y = torch.zeros(T, H, dv)
    grp = torch.arange(H) // (H // G)            # head h reads group floor(h / (H / G))
    for t in range(T):
        Bt, Ct = B[t, grp], C[t, grp]            # [H, N]
        decay = torch.exp(-rate * dt[t])
        S = decay[:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * x[t][:, None, :]
        y[t] = (S * Ct[:, :, None]).sum(1) + P[p + "D"][:, None] * x[t]
    y = y.view(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).view(T, inner) * P[p + "norm"]
    return y @ P[p + "o"].T


def feed_forward(P, p, u):
    return (gelu_tanh(u @ P[p + "gate"].T) * (u @ P[p + "up"].T)) @ P[p + "down"].T


MIXERS = {"attention": sigmoid_attention, "attention_2": differential_attention, "mamba2": mamba2}


def forward(cfg, P, tokens, taps=None):
    """fp32 logits [T, vocab] of a whole sequence; ``taps``: list that receives the
    residual after every layer."""
    eps = cfg["norm"]["eps"]
    x = P["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, l in enumerate(cfg["layers"]):
        src = l.get("weights_of", i)
        p = f"l{src}."
        norm = lambda name, v: unit_rms(v, eps) * P[p + name]   # noqa: E731
        y = MIXERS[l["type"]](P, p + "mix.", l["mixer"], norm("norm1", x), eps)
        x = x + norm("norm1b", y)
        if l.get("mlp") is not None:
            y = feed_forward(P, p + "mlp.", norm("norm2", x))
            x = x + norm("norm2b", y)
        if taps is not None:
            taps.append(x.clone())
    return (unit_rms(x, eps) * P["final.norm"]) @ P["head"].T
