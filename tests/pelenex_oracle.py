"""Plain, slow restatement of the Pelenex design in float64 PyTorch: one function per mechanism,
token by token where the design is a recurrence, no code shared with the package.  ``forward``
runs a whole token list through a checkpoint dictionary (name -> tensor) and a configuration
dictionary (the parsed ``config.json``) and returns the logits of every position and the
residual stream after every layer.

Notation: W width, H heads, G key/value heads, D key size, E value size, t token index.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def lin(w, x):
    return x @ w.to(F64).t()


def silu(z):
    return z * torch.sigmoid(z)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sinusoid(position: int, width: int):
    out = torch.zeros(width, dtype=F64)
    for i in range(width // 2):
        a = position * 10000.0 ** (-2.0 * i / width)
        out[2 * i], out[2 * i + 1] = math.sin(a), math.cos(a)
    return out


def group_norm(x, w, groups, eps):
    """x [..., W] split into ``groups`` consecutive parts, each divided by its own rms."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    return rms(parts, eps).reshape(x.shape) * w.to(F64)


def capped(z, cap):
    return cap * torch.tanh(z / cap)


# ------------------------------------------------------------------ mixers (h: [T, W])
def mlstm(h, p, m, eps):
    H, D, E, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    T = h.shape[0]
    q = (lin(p["q"], h) * D ** -0.5).view(T, H, D)
    k = lin(p["k"], h).view(T, H, D)
    v = lin(p["v"], h).view(T, H, E)
    ig = capped(lin(p["i"], h) + p["i.b"].to(F64), cap)
    fg = torch.nn.functional.logsigmoid(capped(lin(p["f"], h) + p["f.b"].to(F64), cap))
    S = torch.zeros(H, D, E, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    mx = torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, E, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hde,hd->he", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    y = rms(out, eps).reshape(T, H * E) * p["norm"].to(F64) * torch.sigmoid(lin(p["g"], h))
    return lin(p["o"], y)


def window_attention(h, p, m, eps):
    """Softmax attention whose values are the keys before their norm; sliding window with kept
    first tokens; a per-head penalty proportional to the distance."""
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    size, keep = m["mask"]["size"], m["mask"]["keep_first"]
    T = h.shape[0]
    q = lin(p["q"], h).view(T, H, D)
    kraw = lin(p["k"], h).view(T, G, D)
    qn, kn = rms(q, eps), rms(kraw, eps)
    out = torch.zeros(T, H, D, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        slope = 2.0 ** (-8.0 * (hh + 1) / H)
        for i in range(T):
            js = [j for j in range(i + 1) if i - j < size or j < keep]
            s = torch.stack([(qn[i, hh] * kn[j, g]).sum() * m["scale"] - slope * (i - j) for j in js])
            w = torch.softmax(s, 0)
            out[i, hh] = (w[:, None] * kraw[js, g]).sum(0)
    return lin(p["o"], out.reshape(T, H * D))


def gated_linear_attention(h, p, m, eps):
    H, D, E, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    T = h.shape[0]
    q = (lin(p["q"], h) * D ** -0.5).view(T, H, D)
    k = lin(p["k"], h).view(T, H, D)
    v = lin(p["v"], h).view(T, H, E)
    z = lin(p["a2"], lin(p["a1"], h)) + p["a2.b"].to(F64)
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).view(T, H, D)
    S = torch.zeros(H, D, E, dtype=F64)
    out = torch.zeros(T, H, E, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    y = (rms(out, eps) * p["norm"].to(F64)).reshape(T, H * E) * silu(lin(p["g"], h))
    return lin(p["o"], y)


def parallel_mixer(h, p, m, eps):
    left = window_attention(h, {k[5:]: v for k, v in p.items() if k.startswith("left.")
                                and k != "left.out"}, m["left"], eps)
    right = gated_linear_attention(h, {k[6:]: v for k, v in p.items() if k.startswith("right.")
                                       and k != "right.out"}, m["right"], eps)
    return 0.5 * (rms(left, eps) * p["left.out"].to(F64) + rms(right, eps) * p["right.out"].to(F64))


def short_conv(x, w):
    """x [T, C], w [C, taps] (last column: the current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                y[t] += x[s] * w[:, j].to(F64)
    return y


def channel_delta(h, p, m, eps):
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_conv(lin(p["q"], h), p["q.conv"])).view(T, G, D)
    k = silu(short_conv(lin(p["k"], h), p["k.conv"])).view(T, G, D)
    v = silu(short_conv(lin(p["v"], h), p["v.conv"])).view(T, H, E)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(lin(p["b"], h))
    z = lin(p["a2"], lin(p["a1"], h)) + p["dt_bias"].to(F64)
    rate = torch.exp(p["A_log"].to(F64))[None, :, None]
    decay = torch.exp(-rate * torch.nn.functional.softplus(z).view(T, H, D))
    S = torch.zeros(H, D, E, dtype=F64)
    out = torch.zeros(T, H, E, dtype=F64)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            Sh = decay[t, hh][:, None] * S[hh]
            u = beta[t, hh] * (v[t, hh] - Sh.t() @ k[t, g])
            Sh = Sh + k[t, g][:, None] * u[None, :]
            out[t, hh] = Sh.t() @ q[t, g]
            S[hh] = Sh
    gate = torch.sigmoid(lin(p["g2"], lin(p["g1"], h)))
    y = (rms(out, eps) * p["norm"].to(F64)).reshape(T, H * E) * gate
    return lin(p["o"], y)


# ------------------------------------------------------------------ feed-forward
def gated_ff(x, p):
    return lin(p["down"], silu(lin(p["gate"], x)) * lin(p["up"], x))


def feed_forward(h, p, f, margins=None):
    """``margins`` (a list of length T): lowered to the gap between the last chosen and the best
    rejected router logit of every token (how close the routing decision is)."""
    if f["kind"] == "dense":
        return gated_ff(h, p)
    n, top = f["router"]["experts"], f["router"]["top"]
    z = lin(p["router"], h)
    s = torch.sigmoid(z)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        ranked = sorted(range(n), key=lambda e: (-float(s[t, e]), e))
        order = ranked[:top]
        if margins is not None and top < n:
            margins[t] = min(margins[t], float(z[t, ranked[top - 1]] - z[t, ranked[top]]))
        for e in order:
            pe = {k[len(f"e{e}."):]: v for k, v in p.items() if k.startswith(f"e{e}.")}
            out[t] += gated_ff(s[t, e] * h[t], pe)
    if f.get("shared"):
        out = out + gated_ff(h, {k[7:]: v for k, v in p.items() if k.startswith("shared.")})
    return out


# ------------------------------------------------------------------ the model
MIXERS = {"mlstm": mlstm, "parallel": parallel_mixer, "channel_delta": channel_delta}


def forward(cfg: dict, ckpt: dict, tokens, margins=None):
    """Returns (logits [T, vocab], stream after every layer [layers, T, W]), float64.  ``margins``:
    see ``feed_forward``."""
    W, eps, groups = cfg["width"], float(cfg["norm"]["eps"]), cfg["norm"]["groups"]
    T = len(tokens)
    x = ckpt["embed"].to(F64)[torch.tensor(tokens)] + torch.stack([sinusoid(t, W) for t in range(T)])
    streams = []
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        p = {k[len(pre):]: v for k, v in ckpt.items() if k.startswith(pre)}
        h = group_norm(x, p["norm1"], groups, eps)
        y = MIXERS[L["type"]](h, {k[4:]: v for k, v in p.items() if k.startswith("mix.")},
                              L["mixer"], eps)
        if L.get("mlp"):
            y = y + feed_forward(h, {k[4:]: v for k, v in p.items() if k.startswith("mlp.")}, L["mlp"],
                                 margins)
        x = x + y
        streams.append(x.clone())
    z = lin(ckpt["head"], group_norm(x, ckpt["final.norm"], groups, eps))
    cap = cfg.get("logit_softcap")
    if cap:
        z = capped(z, float(cap))
    return z, torch.stack(streams) if streams else torch.zeros(0, T, W, dtype=F64)
