"""Small Pelenex configurations and random checkpoints for the tests (made here, from the tensor
names and shapes the family's checkpoints use; nothing is read from outside)."""
from __future__ import annotations

import json
import os

import torch


def mlstm(heads=3, dim=12, vdim=20, cap=6.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def parallel(heads=4, kv_heads=2, dim=16, size=9, keep=3, scale=0.6, rheads=2, rdim=12, rvdim=20, tau=5.0):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                 "mask": {"size": size, "keep_first": keep}},
        "right": {"heads": rheads, "dim": rdim, "vdim": rvdim, "tau": tau}}}


def delta(heads=4, kv_heads=2, dim=12, vdim=20, conv=3):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                                               "vdim": vdim, "conv": conv}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(ff=24, experts=6, top=2, shared=40):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers, width=40, vocab=89, eps=1e-5, groups=4, softcap=12.0):
    """``layers``: list of (mixer dict, mlp dict or None)."""
    return {"architecture": "Pelenex", "vocab": vocab, "width": width,
            "norm": {"eps": eps, "groups": groups}, "logit_softcap": softcap,
            "layers": [dict(m, mlp=f) for m, f in layers]}


def default_config():
    return config([(parallel(), moe()), (mlstm(), dense()), (delta(), moe(experts=4, top=1, shared=0)),
                   (parallel(heads=2, kv_heads=1, dim=24, size=17, keep=0, rheads=1), None),
                   (mlstm(heads=1, dim=8, vdim=8), moe(top=3)), (delta(heads=2, kv_heads=2, conv=2), dense(16))])


def mixer_shapes(kind, m, W, rank):
    if kind == "mlstm":
        H, D, E = m["heads"], m["dim"], m["vdim"]
        return [("q", (H * D, W)), ("k", (H * D, W)), ("v", (H * E, W)), ("g", (H * E, W)),
                ("o", (W, H * E)), ("norm", (H * E,)), ("i", (H, W)), ("i.b", (H,)), ("f", (H, W)),
                ("f.b", (H,))]
    if kind == "parallel":
        l, r = m["left"], m["right"]
        H, G, D = l["heads"], l["kv_heads"], l["dim"]
        Hr, Dr, Er = r["heads"], r["dim"], r["vdim"]
        return [("left.q", (H * D, W)), ("left.k", (G * D, W)), ("left.o", (W, H * D)),
                ("right.q", (Hr * Dr, W)), ("right.k", (Hr * Dr, W)), ("right.v", (Hr * Er, W)),
                ("right.g", (Hr * Er, W)), ("right.o", (W, Hr * Er)), ("right.norm", (Er,)),
                ("right.a1", (rank, W)), ("right.a2", (Hr * Dr, rank)), ("right.a2.b", (Hr * Dr,)),
                ("left.out", (W,)), ("right.out", (W,))]
    H, G, D, E, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    out = []
    for k, n in (("q", G * D), ("k", G * D), ("v", H * E)):
        out += [(k, (n, W)), (k + ".conv", (n, taps))]
    return out + [("b", (H, W)), ("A_log", (H,)), ("norm", (E,)), ("a1", (rank, W)),
                  ("a2", (H * D, rank)), ("dt_bias", (H * D,)), ("g1", (rank + 1, W)),
                  ("g2", (H * E, rank + 1)), ("o", (W, H * E))]


def shapes(c, rank=5):
    W, V = c["width"], c["vocab"]
    yield "embed", (V, W)
    for i, L in enumerate(c["layers"]):
        p = f"l{i}."
        yield p + "norm1", (W,)
        for n, s in mixer_shapes(L["type"], L["mixer"], W, rank):
            yield p + "mix." + n, s
        f = L["mlp"]
        if f and f["kind"] == "dense":
            for n, s in (("gate", (f["ff"], W)), ("up", (f["ff"], W)), ("down", (W, f["ff"]))):
                yield p + "mlp." + n, s
        elif f:
            names = [(f"e{j}.", f["expert"]["ff"]) for j in range(f["router"]["experts"])]
            if f.get("shared"):
                names.append(("shared.", f["shared"]["ff"]))
            for e, ff in names:
                for n, s in (("gate", (ff, W)), ("up", (ff, W)), ("down", (W, ff))):
                    yield p + "mlp." + e + n, s
            yield p + "mlp.router", (f["router"]["experts"], W)
    yield "final.norm", (W,)
    yield "head", (V, W)


def weights(c, seed=0, qk_gain=2.0, rank=5):
    """Random tensors, rounded to bfloat16 (what a checkpoint holds); queries, keys, gates and the
    router are scaled up so that softmaxes are peaked, gates reach their cap and routing
    decisions are not close."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in shapes(c, rank):
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm", "out") or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif len(shape) == 1 and leaf in ("b", "dt_bias"):
            t = r
        elif leaf == "A_log":
            t = -1.0 + 0.5 * r
        elif name == "embed":
            t = r
        else:
            gain = qk_gain if leaf in ("q", "k", "i", "f") else 2 * qk_gain if leaf == "router" else 1.0
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
