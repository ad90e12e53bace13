"""Small Natilix configurations and random checkpoints for the tests (made here, from the
tensor names and shapes the family's checkpoints use; nothing is read from outside)."""
from __future__ import annotations

import json
import os

import torch


def attention(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=12, base=100.0, scaling=True,
              scale=0.21, v_mix=True, original=32):
    rot = None
    if rot_dims:
        rot = {"base": base, "dims": rot_dims,
               "scaling": ({"factor": 3.0, "low": 1.0, "high": 2.5, "original": original}
                           if scaling else None)}
    return {"type": "attention", "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads,
                                           "vdim": vdim, "rot": rot, "scale": scale, "v_mix": v_mix}}


def delta(heads=4, kv_heads=2, dim=12, vdim=20, conv=3):
    return {"type": "delta", "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads,
                                       "vdim": vdim, "conv": conv}}


def moe(ff=24, experts=6, top=2, groups=3, keep=2):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def config(layers, width=40, vocab=89, eps=1e-5, bigram=(53, 7, 11)):
    """``layers``: list of (mixer dict, mlp dict or None)."""
    c = {"architecture": "Natilix", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "layers": [dict(m, mlp=f) for m, f in layers]}
    if bigram:
        c["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return c


def default_config():
    return config([(delta(), moe()), (attention(), moe(experts=4, top=1, groups=1, keep=1)),
                   (delta(heads=2, kv_heads=2, dim=8, vdim=8, conv=2), None),
                   (attention(heads=2, kv_heads=1, rot_dims=16, scaling=False, v_mix=False), moe()),
                   (attention(heads=6, kv_heads=2, dim=10, rot_dims=0), None)])


def shapes(c):
    W, V = c["width"], c["vocab"]
    yield "embed", (V, W)
    if c.get("embedding"):
        yield "bigram", (c["embedding"]["bigram"]["buckets"] + 1, W)
    for i, L in enumerate(c["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        yield p + "norm1", (W,)
        yield p + "norm1b", (W,)
        if L["type"] == "attention":
            for n, r in (("q", H * D), ("k", G * D), ("v", G * E), ("g", H)):
                yield p + "mix." + n, (r, W)
            yield p + "mix.vmix", ()
            yield p + "mix.sink", (H,)
        else:
            for n, r in (("q", G * D), ("k", G * D), ("v", H * E)):
                yield p + "mix." + n, (r, W)
                yield p + "mix." + n + ".conv", (r, m["conv"])
            for n, s in (("b", (H, W)), ("a", (H, W)), ("g", (H * E, W)), ("A_log", (H,)),
                         ("dt_bias", (H,)), ("norm", (E,))):
                yield p + "mix." + n, s
        yield p + "mix.o", (W, H * E)
        if L["mlp"]:
            yield p + "norm2", (W,)
            yield p + "norm2b", (W,)
            f = L["mlp"]
            for j in range(f["router"]["experts"]):
                yield f"{p}mlp.e{j}.up", (f["expert"]["ff"], W)
                yield f"{p}mlp.e{j}.down", (W, f["expert"]["ff"])
            yield p + "mlp.router", (f["router"]["experts"], W)
    yield "final.norm", (W,)
    yield "head", (V, W)


def weights(c, seed=0, qk_gain=3.0):
    """Random tensors, rounded to bfloat16 (what a checkpoint holds); queries, keys and the
    router are scaled up so that softmaxes are peaked and routing decisions are not close."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in shapes(c):
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if leaf.startswith("norm") and leaf != "norm" or name == "final.norm":
            t = 0.2 * r
        elif leaf == "norm":
            t = 1.0 + 0.2 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf == "vmix":
            t = torch.tensor(0.35)
        elif leaf in ("sink", "dt_bias"):
            t = r
        elif leaf == "A_log":
            t = -1.0 + 0.5 * r
        elif name in ("embed", "bigram"):
            t = r
        else:
            gain = qk_gain if leaf in ("q", "k") else 2 * qk_gain if leaf == "router" else 1.0
            t = r * shape[-1] ** -0.5 * gain
        out[name] = t.to(torch.bfloat16)
    return out


def save_checkpoint(folder, c, w):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(c, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    return folder
