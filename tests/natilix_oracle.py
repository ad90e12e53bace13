"""Plain, slow re-statement of the Natilix decoder, one function per mechanism, in float64 by
default.  It shares no code with ``minivllm_amd``: the tests compare the framework against it.

Notation: T tokens, W model width, H query heads, G key/value heads, D query/key head size,
E value head size.  All functions work on ONE sequence, token after token where the mechanism
is recurrent, and return any state they carry so that a caller can cut a sequence anywhere.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ------------------------------------------------------------------ small pieces
def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ------------------------------------------------------------------ embedding
def bigram_rows(tokens: List[int], prev: Optional[int], mul_prev: int, mul_cur: int, buckets: int):
    """Row of the bigram table for each token; ``prev`` is the token before ``tokens[0]`` or
    None at the start of a sequence (which uses the extra last row)."""
    rows = []
    for t in tokens:
        rows.append(buckets if prev is None else (prev * mul_prev + t * mul_cur) % buckets)
        prev = t
    return rows


# ------------------------------------------------------------------ rotary
def rope_frequencies(dims: int, base: float, scaling: Optional[dict]) -> torch.Tensor:
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    if scaling:
        factor, low, high, orig = (scaling["factor"], scaling["low"], scaling["high"],
                                   scaling["original"])
        out = []
        for fi in f.tolist():
            wl = 2 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=torch.float64)
    return f


def rope_pairs(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, dims: int):
    """x [T, heads, D]: neighbours (2i, 2i+1) of the first ``dims`` entries are rotated by
    position * freqs[i]; angles are formed in float32 as a serving engine would."""
    ang = (positions.to(torch.float32)[:, None] * freqs.to(torch.float32)[None, :]).to(torch.float64)
    c, s = torch.cos(ang)[:, None, :].to(x.dtype), torch.sin(ang)[:, None, :].to(x.dtype)
    out = x.clone()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ------------------------------------------------------------------ attention with a sink
def sink_attention(q, k, v, scale: float, sink: torch.Tensor, q_start: int = 0):
    """q [Tq, H, D], k [Tk, G, D], v [Tk, G, E]; query i sits at position q_start + i and sees
    keys 0 .. q_start + i.  The softmax denominator has one more term exp(sink[h])."""
    Tq, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(Tq, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(Tq):
            n = q_start + i + 1
            s = (k[:n, g] @ q[i, h]) * scale
            m = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[:n, g]).sum(0) / (e.sum() + torch.exp(sink[h] - m))
    return out


# ------------------------------------------------------------------ short causal convolution
def short_conv(x: torch.Tensor, w: torch.Tensor, tail: Optional[torch.Tensor]):
    """x [T, C], w [C, taps] (last column = current token), tail [taps-1, C] = the inputs
    before x (zeros at a sequence's start).  Returns (y [T, C], new tail)."""
    taps = w.shape[1]
    if tail is None:
        tail = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype)
    full = torch.cat([tail, x], 0)
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        y[t] = (full[t:t + taps] * w.t()).sum(0)
    return y, full[full.shape[0] - (taps - 1):].clone()


# ------------------------------------------------------------------ gated delta rule
def gated_delta_rule(q, k, v, beta, g, S: Optional[torch.Tensor]):
    """q, k [T, H, D] (already per query head), v [T, H, E], beta, g [T, H]; S [H, D, E].
    Per token: decay, delta-rule write, then read (the read sees the token's own write)."""
    T, H, D = q.shape
    E = v.shape[-1]
    if S is None:
        S = torch.zeros(H, D, E, dtype=q.dtype)
    S = S.clone()
    o = torch.zeros(T, H, E, dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            S[h] = g[t, h] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].t() @ k[t, h])
            S[h] = S[h] + torch.outer(k[t, h], u)
            o[t, h] = S[h].t() @ q[t, h]
    return o, S


# ------------------------------------------------------------------ routed feed-forward
def grouped_top_experts(z: torch.Tensor, top: int, groups: int, keep: int):
    """z [E] router logits -> (expert ids, weights): softmax over all experts, only experts of
    the ``keep`` groups with the largest best score are eligible, weights are the raw scores."""
    s = torch.softmax(z, -1)
    E = s.shape[0]
    per = E // groups
    best = s.view(groups, per).max(-1).values
    kept = torch.topk(best, keep).indices.tolist()
    masked = torch.full_like(s, -1.0)
    for gi in kept:
        masked[gi * per:(gi + 1) * per] = s[gi * per:(gi + 1) * per]
    ids = torch.topk(masked, top).indices
    return ids.tolist(), s[ids]


def routing_margin(z: torch.Tensor, top: int, groups: int, keep: int) -> float:
    """How far the routing decision for logits z is from flipping, in logit units: the smallest
    gap between a kept and a dropped group's best logit, or between a chosen and an eligible
    unchosen logit (scores are a monotone function of the logits)."""
    per = z.shape[0] // groups
    gbest = z.view(groups, per).max(-1).values
    best = gbest.sort(descending=True).values
    m = float(best[keep - 1] - best[keep]) if keep < groups else float("inf")
    ids, _ = grouped_top_experts(z, top, groups, keep)
    kept = torch.topk(gbest, keep).indices.tolist()
    rest = [float(z[e]) for gi in kept for e in range(gi * per, (gi + 1) * per) if e not in ids]
    if rest:
        m = min(m, float(z[ids].min()) - max(rest))
    return m


def routed_ffn(h: torch.Tensor, router, ups, downs, top, groups, keep, margins=None):
    out = torch.zeros(h.shape[0], downs[0].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        if margins is not None:
            margins[t] = min(margins[t], routing_margin(router @ h[t], top, groups, keep))
        ids, w = grouped_top_experts(router @ h[t], top, groups, keep)
        for e, we in zip(ids, w):
            out[t] += we * (downs[e] @ gelu_erf(ups[e] @ h[t]))
    return out


# ------------------------------------------------------------------ the whole decoder
class Oracle:
    """Runs a model given as (config dict, {name: tensor}); ``feed`` takes the next tokens of
    one sequence and returns logits for all of them; everything a sequence carries is in
    ``self.state``."""

    def __init__(self, cfg: dict, weights: Dict[str, torch.Tensor], dtype=torch.float64):
        self.cfg, self.dtype = cfg, dtype
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
        self.eps = cfg["norm"]["eps"]
        self.reset()

    def reset(self):
        self.state = {"n": 0, "prev": None, "layers": [dict() for _ in self.cfg["layers"]]}
        self.trace = []

    def _attention(self, i, m, h, st, pos, shared):
        w, p = self.w, f"l{i}.mix."
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        T = h.shape[0]
        q = (h @ w[p + "q"].t()).view(T, H, D)
        k = (h @ w[p + "k"].t()).view(T, G, D)
        v = (h @ w[p + "v"].t()).view(T, G, E)
        rot = m.get("rot")
        if rot:
            f = rope_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
            q, k = rope_pairs(q, pos, f, rot["dims"]), rope_pairs(k, pos, f, rot["dims"])
        if m.get("v_mix"):
            if "v_first" in shared:
                lam = w[p + "vmix"]
                v = (1 - lam) * v + lam * shared["v_first"]
            else:
                shared["v_first"] = v
        K = torch.cat([st["k"], k], 0) if "k" in st else k
        V = torch.cat([st["v"], v], 0) if "v" in st else v
        st["k"], st["v"] = K, V
        o = sink_attention(q, K, V, m["scale"], w[p + "sink"], q_start=K.shape[0] - T)
        gate = torch.sigmoid(h @ w[p + "g"].t())                   # [T, H]
        o = o * gate[:, :, None]
        return o.reshape(T, H * E) @ w[p + "o"].t()

    def _delta(self, i, m, h, st):
        w, p = self.w, f"l{i}.mix."
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        T = h.shape[0]
        q, st["cq"] = short_conv(h @ w[p + "q"].t(), w[p + "q.conv"], st.get("cq"))
        k, st["ck"] = short_conv(h @ w[p + "k"].t(), w[p + "k.conv"], st.get("ck"))
        v, st["cv"] = short_conv(h @ w[p + "v"].t(), w[p + "v.conv"], st.get("cv"))
        q, k, v = silu(q).view(T, G, D), silu(k).view(T, G, D), silu(v).view(T, H, E)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        rep = H // G
        q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
        beta = torch.sigmoid(h @ w[p + "b"].t())
        g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].t() + w[p + "dt_bias"]))
        o, st["S"] = gated_delta_rule(q, k, v, beta, g, st.get("S"))
        o = rms_unit(o, self.eps) * w[p + "norm"]
        o = o * silu(h @ w[p + "g"].t()).view(T, H, E)
        return o.reshape(T, H * E) @ w[p + "o"].t()

    def feed(self, tokens: List[int]) -> torch.Tensor:
        cfg, w, st = self.cfg, self.w, self.state
        T = len(tokens)
        x = w["embed"][tokens]
        bg = (cfg.get("embedding") or {}).get("bigram")
        if bg:
            rows = bigram_rows(tokens, st["prev"], bg["mul_prev"], bg["mul_cur"], bg["buckets"])
            x = x + w["bigram"][rows]
        pos = torch.arange(st["n"], st["n"] + T)
        shared = {}
        self.trace = []
        self.margin = [float('inf')] * T          # per token: the closest routing decision of any layer
        for i, layer in enumerate(cfg["layers"]):
            p, ls, m = f"l{i}.", st["layers"][i], layer["mixer"]
            h = norm_around_zero(x, w[p + "norm1"], self.eps)
            y = self._attention(i, m, h, ls, pos, shared) if layer["type"] == "attention" \
                else self._delta(i, m, h, ls)
            x = x + norm_around_zero(y, w[p + "norm1b"], self.eps)
            if layer.get("mlp"):
                r = layer["mlp"]["router"]
                E = r["experts"]
                h = norm_around_zero(x, w[p + "norm2"], self.eps)
                y = routed_ffn(h, w[p + "mlp.router"], [w[f"{p}mlp.e{e}.up"] for e in range(E)],
                               [w[f"{p}mlp.e{e}.down"] for e in range(E)], r["top"],
                               r["groups"]["count"], r["groups"]["keep"], margins=self.margin)
                x = x + norm_around_zero(y, w[p + "norm2b"], self.eps)
            self.trace.append(x.clone())
        st["n"] += T
        st["prev"] = tokens[-1]
        return norm_around_zero(x, w["final.norm"], self.eps) @ w["head"].t()
