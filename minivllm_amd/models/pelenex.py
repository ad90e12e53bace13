"""Pelenex: a decoder whose layers are *parallel* - one grouped RMS norm feeds a sequence mixer
and a feed-forward side by side, x <- x + mixer(h) + ff(h) - around a fp32 residual stream, with
three kinds of mixer in whatever order the configuration lists them:

* ``mlstm``          matrix memory with exponential gating (``layers.linear_attention.MatrixLSTM``);
* ``parallel``       two mixers on the same input, each RMS-normalised over the width with its own
                     weight, averaged: softmax attention over a sliding window that keeps the first
                     tokens, with unit-RMS q / k, a distance penalty per head and the un-normalised
                     keys as values (``layers.attention.SinkAttention`` without its sink), next to
                     gated linear attention with a low-rank decay projection
                     (``layers.linear_attention.GatedLinearAttention``);
* ``channel_delta``  gated delta rule with one decay per head and key channel and low-rank decay
                     and gate projections (``layers.delta_rule.GatedDeltaRule``).

Feed-forward: dense gated (silu), or sigmoid-routed experts whose weight scales the expert's
input, plus a shared expert (``layers.moe.RoutedGatedExperts`` for all three).  Embedding: token
row + sinusoidal position vector.  Output: the grouped norm, an untied head and a tanh soft cap.

Everything that reads a layer's normed input is ONE projection: the mixer's q / k / v / gates /
low-rank first stages and the feed-forward's gate and up rows are stacked into ``in_proj``.

``PelenexConfig.from_dict`` reads the family's ``config.json``; sizes the file does not name (the
ranks of the low-rank projections) come from the checkpoint's tensor shapes, so the fused
parameters are built when the weights arrive (``load_weights``).  Single rank only.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from minivllm_amd import ops
from minivllm_amd.layers.attention import SinkAttention
from minivllm_amd.layers.delta_rule import GatedDeltaRule
from minivllm_amd.layers.embedding_head import SinusoidalEmbedding
from minivllm_amd.layers.layernorm import GroupRMSNorm
from minivllm_amd.layers.linear_attention import GatedLinearAttention, MatrixLSTM
from minivllm_amd.layers.moe import RoutedGatedExperts
from minivllm_amd.utils.context import get_context

MIXER_TYPES = ("mlstm", "parallel", "channel_delta")


# ------------------------------------------------------------------ configuration
@dataclass
class PelenexLayerSpec:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@dataclass
class PelenexConfig:
    vocab_size: int
    hidden_size: int
    layers: List[PelenexLayerSpec] = field(default_factory=list)
    rms_norm_epsilon: float = 1e-6
    norm_groups: int = 1
    logit_softcap: float = 0.0
    max_position: int = 8192
    name: str = "pelenex"
    architecture: str = "pelenex"
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, c: dict, name: str = "pelenex") -> "PelenexConfig":
        layers = []
        for L in c["layers"]:
            if L["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown layer type {L['type']!r}")
            f = L.get("mlp")
            if f and f.get("kind") not in ("dense", "moe"):
                raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
            layers.append(PelenexLayerSpec(L["type"], L["mixer"], f or None))
        return cls(vocab_size=c["vocab"], hidden_size=c["width"], layers=layers,
                   rms_norm_epsilon=float(c["norm"]["eps"]), norm_groups=int(c["norm"].get("groups", 1)),
                   logit_softcap=float(c.get("logit_softcap") or 0.0),
                   max_position=int(c.get("max_position", 8192)), name=name)

    def validate_engine(self, engine_cfg) -> None:
        if engine_cfg.tp_degree != 1:
            raise ValueError("Pelenex runs on one rank (its mixers are not sharded)")
        if self.hidden_size % self.norm_groups or self.hidden_size % 2:
            raise ValueError("the width must be even and a multiple of the norm's groups")
        for L in self.layers:
            for m in ([L.mixer["left"]] if L.type == "parallel" else [L.mixer]):
                if m["heads"] % m.get("kv_heads", m["heads"]):
                    raise ValueError("heads must be a multiple of kv_heads")
            if L.type == "parallel" and L.mixer["left"].get("vdim", L.mixer["left"]["dim"]) != L.mixer["left"]["dim"]:
                raise ValueError("attention whose values are its keys needs vdim == dim")


def _param(t: torch.Tensor, like: torch.Tensor, dtype=None) -> nn.Parameter:
    return nn.Parameter(t.to(device=like.device, dtype=dtype or like.dtype).contiguous(),
                        requires_grad=False)


def _take(w: dict, key: str, shape, where: str) -> torch.Tensor:
    if key not in w:
        raise KeyError(f"checkpoint lacks {where}{key}")
    t = w.pop(key)
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"shape mismatch for {where}{key}: expected {tuple(shape)}, checkpoint "
                         f"has {tuple(t.shape)}")
    return t


# ------------------------------------------------------------------ mixers
class PelenexMLSTMMixer(nn.Module):
    def __init__(self, W: int, m: dict, eps: float):
        super().__init__()
        self.W = W
        self.core = MatrixLSTM(m["heads"], m["dim"], m.get("vdim", m["dim"]), m["gate_cap"], eps)
        self.in_rows = sum(self.core.split_sizes())
        self.o_proj = nn.Parameter(torch.zeros(W, m["heads"] * m.get("vdim", m["dim"])), requires_grad=False)

    def state_cores(self):
        return [self.core]

    def attention_cores(self):
        return []

    def forward(self, proj, x, out_dtype):
        """proj: this mixer's columns of the layer's fused projection.  Returns what is added to
        the stream (or adds to ``x`` itself and returns None)."""
        return F.linear(self.core(proj, out_dtype), self.o_proj)

    def load(self, w: dict, where: str, like) -> List[torch.Tensor]:
        c, W = self.core, self.W
        H, D, E = c.num_heads, c.head_dim, c.v_head_dim
        rows = [_take(w, k, (n, W), where) for k, n in
                (("q", H * D), ("k", H * D), ("v", H * E), ("g", H * E), ("i", H), ("f", H))]
        self.o_proj = _param(_take(w, "o", (W, H * E), where), like)
        c.norm_weight.copy_(_take(w, "norm", (H * E,), where))
        c.i_bias.copy_(_take(w, "i.b", (H,), where))
        c.f_bias.copy_(_take(w, "f.b", (H,), where))
        return rows

    @staticmethod
    def shapes(W, m, rank):
        H, D, E = m["heads"], m["dim"], m.get("vdim", m["dim"])
        return [("q", (H * D, W)), ("k", (H * D, W)), ("v", (H * E, W)), ("g", (H * E, W)),
                ("o", (W, H * E)), ("norm", (H * E,)), ("i", (H, W)), ("i.b", (H,)),
                ("f", (H, W)), ("f.b", (H,))]


class PelenexParallelMixer(nn.Module):
    """Windowed softmax attention (left) and gated linear attention (right) on the same input;
    result = (rmsnorm(left) * w_left + rmsnorm(right) * w_right) / 2, added to the stream by one
    kernel."""

    def __init__(self, W: int, m: dict, eps: float):
        super().__init__()
        self.W, self.eps = W, eps
        l, r = m["left"], m["right"]
        H, G, D = l["heads"], l.get("kv_heads", l["heads"]), l["dim"]
        slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float32)
        mask = l.get("mask") or {}
        self.attn = SinkAttention(H, G, D, D, float(l["scale"]), sink=False,
                                  window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)),
                                  distance_slopes=slopes)
        self.gla = GatedLinearAttention(r["heads"], r["dim"], r.get("vdim", r["dim"]), r["tau"], eps)
        self.left_sizes = [H * D, G * D]
        self.right_rows = sum(self.gla.split_sizes())
        self.rank = 0
        f32 = dict(dtype=torch.float32)
        self.left_out = nn.Parameter(torch.ones(W, **f32), requires_grad=False)
        self.right_out = nn.Parameter(torch.ones(W, **f32), requires_grad=False)
        self.left_o = nn.Parameter(torch.zeros(W, H * D), requires_grad=False)
        self.right_o = nn.Parameter(torch.zeros(W, r["heads"] * r.get("vdim", r["dim"])), requires_grad=False)
        self.decay_up = nn.Parameter(torch.zeros(r["heads"] * r["dim"], 1), requires_grad=False)
        self.in_rows = 0

    def state_cores(self):
        return [self.gla]

    def attention_cores(self):
        return [self.attn]

    def forward(self, proj, x, out_dtype):
        a = self.attn
        T = proj.shape[0]
        H, G, D = a.num_heads, a.num_kv_heads, a.head_dim
        nl = sum(self.left_sizes)
        q, k = proj[:, :nl].split(self.left_sizes, dim=-1)
        q, k = q.view(T, H, D), k.view(T, G, D)
        ops.unit_norm_store(q, k, self.eps, a.k_cache, a.v_cache, get_context().slot_mapping)
        left = F.linear(a(q, None), self.left_o)
        right_in = proj[:, nl:nl + self.right_rows]
        low = proj[:, nl + self.right_rows:nl + self.right_rows + self.rank]
        right = F.linear(self.gla(right_in, F.linear(low, self.decay_up), out_dtype), self.right_o)
        ops.add_normed_mean(x, [(left, self.left_out), (right, self.right_out)], self.eps)
        return None

    def load(self, w: dict, where: str, like) -> List[torch.Tensor]:
        W, a, g = self.W, self.attn, self.gla
        H, G, D = a.num_heads, a.num_kv_heads, a.head_dim
        Hr, Dr, Er = g.num_heads, g.head_dim, g.v_head_dim
        rows = [_take(w, "left.q", (H * D, W), where), _take(w, "left.k", (G * D, W), where)]
        rows += [_take(w, "right." + k, (n, W), where) for k, n in
                 (("q", Hr * Dr), ("k", Hr * Dr), ("v", Hr * Er), ("g", Hr * Er))]
        a1 = _take(w, "right.a1", None, where)
        self.rank = a1.shape[0]
        rows.append(a1)
        self.decay_up = _param(_take(w, "right.a2", (Hr * Dr, self.rank), where), like)
        g.decay_bias.copy_(_take(w, "right.a2.b", (Hr * Dr,), where))
        g.norm_weight.copy_(_take(w, "right.norm", (Er,), where))
        self.left_o = _param(_take(w, "left.o", (W, H * D), where), like)
        self.right_o = _param(_take(w, "right.o", (W, Hr * Er), where), like)
        self.left_out.copy_(_take(w, "left.out", (W,), where))
        self.right_out.copy_(_take(w, "right.out", (W,), where))
        return rows

    @staticmethod
    def shapes(W, m, rank):
        l, r = m["left"], m["right"]
        H, G, D = l["heads"], l.get("kv_heads", l["heads"]), l["dim"]
        Hr, Dr, Er = r["heads"], r["dim"], r.get("vdim", r["dim"])
        return [("left.q", (H * D, W)), ("left.k", (G * D, W)), ("left.o", (W, H * D)),
                ("right.q", (Hr * Dr, W)), ("right.k", (Hr * Dr, W)), ("right.v", (Hr * Er, W)),
                ("right.g", (Hr * Er, W)), ("right.o", (W, Hr * Er)), ("right.norm", (Er,)),
                ("right.a1", (rank, W)), ("right.a2", (Hr * Dr, rank)), ("right.a2.b", (Hr * Dr,)),
                ("left.out", (W,)), ("right.out", (W,))]


class PelenexDeltaMixer(nn.Module):
    def __init__(self, W: int, m: dict, eps: float):
        super().__init__()
        self.W = W
        H, G, D, E = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
        self.core = GatedDeltaRule(H, G, D, E, int(m.get("conv", 1)), eps, channel_decay=True,
                                   gate_act="sigmoid")
        self.base_rows = sum(self.core.split_sizes())
        self.rank_a = self.rank_g = 0
        self.o_proj = nn.Parameter(torch.zeros(W, H * E), requires_grad=False)
        self.decay_up = nn.Parameter(torch.zeros(H * D, 1), requires_grad=False)
        self.gate_up = nn.Parameter(torch.zeros(H * E, 1), requires_grad=False)
        self.in_rows = 0

    def state_cores(self):
        return [self.core]

    def attention_cores(self):
        return []

    def forward(self, proj, x, out_dtype):
        n = self.base_rows
        a = F.linear(proj[:, n:n + self.rank_a], self.decay_up)
        gate = F.linear(proj[:, n + self.rank_a:n + self.rank_a + self.rank_g], self.gate_up)
        return F.linear(self.core(proj, out_dtype, a=a, gate=gate), self.o_proj)

    def load(self, w: dict, where: str, like) -> List[torch.Tensor]:
        c, W = self.core, self.W
        H, G, D, E = c.num_heads, c.num_kv_heads, c.head_dim, c.v_head_dim
        sizes = (("q", G * D), ("k", G * D), ("v", H * E))
        rows = [_take(w, k, (n, W), where) for k, n in sizes] + [_take(w, "b", (H, W), where)]
        convs = [_take(w, k + ".conv", (n, c.taps), where) for k, n in sizes]
        c.conv_weight.copy_(torch.cat(convs, 0))
        a1, g1 = _take(w, "a1", None, where), _take(w, "g1", None, where)
        self.rank_a, self.rank_g = a1.shape[0], g1.shape[0]
        rows += [a1, g1]
        self.decay_up = _param(_take(w, "a2", (H * D, self.rank_a), where), like)
        self.gate_up = _param(_take(w, "g2", (H * E, self.rank_g), where), like)
        c.A_log.copy_(_take(w, "A_log", (H,), where))
        c.dt_bias.copy_(_take(w, "dt_bias", (H * D,), where))
        c.norm_weight.copy_(_take(w, "norm", (E,), where))
        self.o_proj = _param(_take(w, "o", (W, H * E), where), like)
        return rows

    @staticmethod
    def shapes(W, m, rank):
        H, G, D, E = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
        taps = int(m.get("conv", 1))
        out = []
        for k, n in (("q", G * D), ("k", G * D), ("v", H * E)):
            out += [(k, (n, W)), (k + ".conv", (n, taps))]
        return out + [("b", (H, W)), ("A_log", (H,)), ("norm", (E,)), ("a1", (rank, W)),
                      ("a2", (H * D, rank)), ("dt_bias", (H * D,)), ("g1", (rank, W)),
                      ("g2", (H * E, rank)), ("o", (W, H * E))]


_MIXERS = {"mlstm": PelenexMLSTMMixer, "parallel": PelenexParallelMixer,
           "channel_delta": PelenexDeltaMixer}


def _ff_sizes(f: Optional[dict]):
    """(expert ff, experts, top, shared ff) of a feed-forward entry of the configuration."""
    if not f:
        return None
    if f["kind"] == "dense":
        return 0, 0, 0, int(f["ff"])
    shared = f.get("shared") or {}
    return int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]), int(shared.get("ff", 0))


class PelenexLayer(nn.Module):
    def __init__(self, cfg: PelenexConfig, spec: PelenexLayerSpec):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.rms_norm_epsilon
        self.kind = spec.type
        self.norm1 = GroupRMSNorm(W, cfg.norm_groups, eps)
        self.mix = _MIXERS[spec.type](W, spec.mixer, eps)
        sizes = _ff_sizes(spec.mlp)
        self.mlp = RoutedGatedExperts(W, *sizes) if sizes else None
        self.in_proj = nn.Parameter(torch.zeros(1, W), requires_grad=False)
        self.mix_rows = 0

    def forward(self, h, x, out_dtype):
        """h: the layer's normed input; x: the fp32 stream.  Returns the tensors still to be
        added to the stream."""
        proj = F.linear(h, self.in_proj)
        ys = []
        y = self.mix(proj[:, :self.mix_rows], x, out_dtype)
        if y is not None:
            ys.append(y)
        if self.mlp is not None:
            ys.append(self.mlp(h, gu=proj[:, self.mix_rows:]))
        return ys

    def load(self, w: dict, where: str, like) -> None:
        W = self.norm1.weight.shape[0]
        self.norm1.weight.copy_(_take(w, "norm1", (W,), where))
        mw = {k[4:]: w.pop(k) for k in [k for k in w if k.startswith("mix.")]}
        rows = self.mix.load(mw, where + "mix.", like)
        if mw:
            raise KeyError(f"checkpoint tensor {where}mix.{next(iter(mw))} has no parameter")
        self.mix_rows = sum(r.shape[0] for r in rows)
        f = self.mlp
        if f is not None:
            fw = {k[4:]: w.pop(k) for k in [k for k in w if k.startswith("mlp.")]}
            names = [f"e{j}." for j in range(f.experts)] + (["shared."] if f.shared_ff else [])
            if not f.experts:
                names = [""]                         # a dense layer's tensors carry no expert name
            sizes = [f.ff] * f.experts + ([f.shared_ff] if f.shared_ff else [])
            rows += [_take(fw, n + "gate", (s, W), where + "mlp.") for n, s in zip(names, sizes)]
            rows += [_take(fw, n + "up", (s, W), where + "mlp.") for n, s in zip(names, sizes)]
            f.down = _param(torch.cat([_take(fw, n + "down", (W, s), where + "mlp.")
                                       for n, s in zip(names, sizes)], 1), like)
            if f.experts:
                f.router.copy_(_take(fw, "router", (f.experts, W), where + "mlp."))
            f.gate_up = None                          # its rows live in the layer's projection
            if fw:
                raise KeyError(f"checkpoint tensor {where}mlp.{next(iter(fw))} has no parameter")
        if w:
            raise KeyError(f"checkpoint tensor {where}{next(iter(w))} has no parameter")
        self.in_proj = _param(torch.cat(rows, 0), like)


class PelenexModel(nn.Module):
    def __init__(self, cfg: PelenexConfig):
        super().__init__()
        self.embed = SinusoidalEmbedding(cfg.vocab_size, cfg.hidden_size)
        self.layers = nn.ModuleList([PelenexLayer(cfg, s) for s in cfg.layers])
        self.eps, self.groups = cfg.rms_norm_epsilon, cfg.norm_groups
        self.act_dtype = self.embed.weight.dtype
        # observers for tests: called with (layer index, fp32 stream) after every layer
        self.layer_hook = None

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the fp32 residual stream [T, W] after the last layer (the final norm belongs
        to the head: only the rows whose logits are wanted go through it)."""
        dt = self.act_dtype
        x = self.embed(input_ids, positions)
        n = len(self.layers)
        h = self.layers[0].norm1(x, dt) if n else None
        for i, layer in enumerate(self.layers):
            ys = layer(h, x, dt)
            nxt = self.layers[i + 1].norm1.weight if i + 1 < n else None
            h = ops.residual_group_norm(x, ys, nxt, self.groups, self.eps, dt)
            if self.layer_hook is not None:
                self.layer_hook(i, x)
        return x


class CappedNormedHead(nn.Module):
    """Final grouped norm + untied output projection + tanh soft cap, applied to the rows a step
    wants (each sequence's last row, or the context's ``logit_rows``)."""

    def __init__(self, vocab_size: int, hidden_size: int, groups: int, eps: float, cap: float):
        super().__init__()
        self.norm = GroupRMSNorm(hidden_size, groups, eps)
        self.weight = nn.Parameter(torch.zeros(vocab_size, hidden_size), requires_grad=False)
        self.cap = float(cap)
        self.num_embeddings = vocab_size
        self.vocab_start = 0

    def select_last(self, hidden: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        if ctx.logit_rows is not None:
            return hidden.index_select(0, ctx.logit_rows.long())
        if ctx.is_prefill and ctx.cu_seqlens_q is not None:
            return hidden.index_select(0, (ctx.cu_seqlens_q[1:] - 1).long())
        return hidden

    def local_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        rows = self.select_last(hidden)
        z = F.linear(self.norm(rows, self.weight.dtype), self.weight)
        return ops.tanh_cap_(z, self.cap) if self.cap > 0 else z

    def forward(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.local_logits(hidden)


class PelenexForCausalLM(nn.Module):
    has_recurrent_state = True
    needs_aux_rows = False

    def __init__(self, config: PelenexConfig):
        super().__init__()
        self.config = config
        self.model = PelenexModel(config)
        self.lm_head = CappedNormedHead(config.vocab_size, config.hidden_size, config.norm_groups,
                                        config.rms_norm_epsilon, config.logit_softcap)

    def forward(self, input_ids, positions=None):
        if positions is None:
            positions = get_context().positions
        return self.model(input_ids, positions)

    def compute_logits(self, hidden):
        return self.lm_head(hidden)

    def compute_local_logits(self, hidden):
        return self.lm_head.local_logits(hidden)

    # ---- what the engine needs to know about caches and state ---------------------------
    def attention_layers(self):
        return [a for l in self.model.layers for a in l.mix.attention_cores()]

    def state_layers(self):
        return [c for l in self.model.layers for c in l.mix.state_cores()]

    # ---- weights -----------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, items) -> int:
        """``items``: iterable of (checkpoint name, tensor).  The tensors of a layer are collected
        and then stacked into its fused parameters (whose sizes follow the tensors' shapes where
        the configuration names none); unknown or missing names raise."""
        like = self.model.embed.weight
        per_layer: List[dict] = [dict() for _ in self.model.layers]
        top = {"embed": self.model.embed.weight, "head": self.lm_head.weight,
               "final.norm": self.lm_head.norm.weight}
        n, seen = 0, set()
        for name, t in items:
            n += 1
            if name in top:
                if tuple(top[name].shape) != tuple(t.shape):
                    raise ValueError(f"shape mismatch for {name}: expected {tuple(top[name].shape)}, "
                                     f"checkpoint has {tuple(t.shape)}")
                top[name].copy_(t.to(top[name].dtype))
                seen.add(name)
                continue
            li, _, rest = name.partition(".")
            if not (li.startswith("l") and li[1:].isdigit()) or int(li[1:]) >= len(per_layer):
                raise KeyError(f"checkpoint tensor {name!r} has no parameter")
            per_layer[int(li[1:])][rest] = t
        for k in top:
            if k not in seen:
                raise KeyError(f"checkpoint lacks {k}")
        for i, (layer, w) in enumerate(zip(self.model.layers, per_layer)):
            layer.load(w, f"l{i}.", like)
        return n

    def checkpoint_shapes(self, rank: int = 8):
        """(name, shape) of every tensor a checkpoint of this configuration holds; ``rank``: the
        inner size of the low-rank projections (a checkpoint's own shapes decide when loading)."""
        c = self.config
        W = c.hidden_size
        yield "embed", (c.vocab_size, W)
        for i, L in enumerate(c.layers):
            p = f"l{i}."
            yield p + "norm1", (W,)
            for nm, shape in _MIXERS[L.type].shapes(W, L.mixer, rank):
                yield p + "mix." + nm, shape
            sizes = _ff_sizes(L.mlp)
            if sizes:
                ff, ne, _, sff = sizes
                names = [(f"e{j}.", ff) for j in range(ne)] + ([("shared.", sff)] if ne and sff else [])
                if not ne:
                    names = [("", sff)]
                for nm, s in names:
                    yield p + "mlp." + nm + "gate", (s, W)
                    yield p + "mlp." + nm + "up", (s, W)
                    yield p + "mlp." + nm + "down", (W, s)
                if ne:
                    yield p + "mlp.router", (ne, W)
        yield "final.norm", (W,)
        yield "head", (c.vocab_size, W)

    def random_checkpoint(self, seed: int = 0, rank: int = 8):
        """Seeded random tensors (values exactly representable in bfloat16) of every checkpoint
        name, scaled so that activations stay O(1) through the stack."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        for name, shape in self.checkpoint_shapes(rank):
            leaf = name.rsplit(".", 1)[-1]
            r = torch.randn(shape, generator=g)
            if leaf in ("norm1", "norm", "out") or name == "final.norm":
                t = 1.0 + 0.1 * r
            elif leaf == "conv":
                t = 0.5 * r
            elif leaf in ("dt_bias",):
                t = r
            elif leaf == "b" and len(shape) == 1:
                t = 1.0 + r                              # gate and decay biases
            elif leaf == "A_log":
                t = -1.0 + 0.5 * r
            elif name == "embed":
                t = r
            else:
                t = r * (shape[-1] ** -0.5) * (2.0 if leaf in ("q", "k", "router", "i", "f") else 1.0)
            out[name] = t.to(torch.bfloat16)
        return out

    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        self.load_weights(self.random_checkpoint(seed).items())
