"""Natilix: a hybrid decoder whose layers alternate (in any order the configuration lists)
between softmax attention and a gated delta-rule recurrence, each followed by an optional
mixture-of-experts feed-forward, around a fp32 residual stream.

* embedding: token row + a hashed bigram row (``HashedBigramEmbedding``);
* every sublayer sits between two zero-centred RMS norms: x <- x + norm_b(f(norm_a(x)));
* attention (``SinkAttention``): grouped query heads, key/query size D and value size E,
  rotation of neighbouring pairs on the first ``rot.dims`` entries with Llama-3.1-style
  frequency scaling, an explicit score scale, a learned sink in the softmax denominator,
  values mixed with those of the first value-mixing layer of the same token before they are
  cached, a sigmoid gate per head on the output;
* delta rule (``GatedDeltaRule``);
* feed-forward (``GroupedRoutedExperts``);
* final norm + untied head.

``NatilixConfig.from_dict`` reads the family's ``config.json``; tensor names follow its
checkpoints (``l<i>.mix.q``, ``l<i>.mlp.e<j>.up``, ...) and are packed into fused parameters by
``load_weights``.  Single rank only (no tensor-parallel sharding of the new mixers yet).
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
from minivllm_amd.layers.embedding_head import HashedBigramEmbedding
from minivllm_amd.layers.layernorm import OffsetRMSNorm
from minivllm_amd.layers.moe import GroupedRoutedExperts
from minivllm_amd.layers.rotary_embedding import PairRotaryEmbedding
from minivllm_amd.utils.context import get_context


# ------------------------------------------------------------------ configuration
@dataclass
class MixerSpec:
    kind: str                       # "attention" | "delta"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float = 1.0              # attention
    rot: Optional[Dict[str, Any]] = None
    v_mix: bool = False
    conv: int = 1                   # delta: taps of the short convolution


@dataclass
class ExpertsSpec:
    ff: int
    experts: int
    top: int
    groups: int
    keep: int


@dataclass
class LayerSpec:
    mixer: MixerSpec
    mlp: Optional[ExpertsSpec]


@dataclass
class NatilixConfig:
    vocab_size: int
    hidden_size: int
    layers: List[LayerSpec] = field(default_factory=list)
    rms_norm_epsilon: float = 1e-6
    bigram: Optional[Dict[str, int]] = None      # buckets, mul_prev, mul_cur
    max_position: int = 8192
    name: str = "natilix"
    architecture: str = "natilix"
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, c: dict, name: str = "natilix") -> "NatilixConfig":
        layers = []
        for L in c["layers"]:
            m = L["mixer"]
            kind = L["type"]
            if kind not in ("attention", "delta"):
                raise ValueError(f"unknown layer type {kind!r}")
            spec = MixerSpec(kind=kind, heads=m["heads"], kv_heads=m.get("kv_heads", m["heads"]),
                             dim=m["dim"], vdim=m.get("vdim", m["dim"]),
                             scale=float(m.get("scale", 1.0)), rot=m.get("rot"),
                             v_mix=bool(m.get("v_mix", False)), conv=int(m.get("conv", 1)))
            f = L.get("mlp")
            mlp = None
            if f:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
                r = f["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                mlp = ExpertsSpec(ff=f["expert"]["ff"], experts=r["experts"], top=r["top"],
                                  groups=g["count"], keep=g["keep"])
            layers.append(LayerSpec(spec, mlp))
        return cls(vocab_size=c["vocab"], hidden_size=c["width"], layers=layers,
                   rms_norm_epsilon=float(c["norm"]["eps"]),
                   bigram=(c.get("embedding") or {}).get("bigram"),
                   max_position=int(c.get("max_position", 8192)), name=name)

    def validate_engine(self, engine_cfg) -> None:
        if engine_cfg.tp_degree != 1:
            raise ValueError("Natilix runs on one rank (its mixers are not sharded)")
        for L in self.layers:
            m = L.mixer
            if m.heads % m.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
        mixes = [(L.mixer.kv_heads, L.mixer.vdim) for L in self.layers
                 if L.mixer.kind == "attention" and L.mixer.v_mix]
        if len(set(mixes)) > 1:
            raise ValueError("value-mixing layers must share kv_heads and vdim")


# ------------------------------------------------------------------ modules
class NatilixAttentionMixer(nn.Module):
    def __init__(self, W: int, m: MixerSpec, max_position: int, mix_role: int):
        """``mix_role``: 0 no value mixing, 1 the first value-mixing layer (publishes its
        values), 2 a later one (blends them in)."""
        super().__init__()
        H, G, D, E = m.heads, m.kv_heads, m.dim, m.vdim
        self.sizes = [H * D, G * D, G * E, H]                      # q, k, v, gate
        self.in_proj = nn.Parameter(torch.zeros(sum(self.sizes), W), requires_grad=False)
        self.o_proj = nn.Parameter(torch.zeros(W, H * E), requires_grad=False)
        self.vmix = nn.Parameter(torch.zeros((), dtype=torch.float32), requires_grad=False)
        self.mix_role = mix_role
        self.rot_dims = int(m.rot["dims"]) if m.rot else 0
        self.rope = (PairRotaryEmbedding(self.rot_dims, max_position, float(m.rot["base"]),
                                         m.rot.get("scaling")) if m.rot else None)
        self.attn = SinkAttention(H, G, D, E, m.scale)
        self.shape = (H, G, D, E)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, shared: dict) -> torch.Tensor:
        H, G, D, E = self.shape
        T = h.shape[0]
        proj = F.linear(h, self.in_proj)
        q, k, v, gate = proj.split(self.sizes, dim=-1)
        q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, E)
        ctx = get_context()
        if self.mix_role == 1:
            shared["v_first"] = torch.empty((T, G, E), dtype=proj.dtype, device=proj.device)
        ops.pair_rope_mix_store(q, k, v, positions,
                                self.rope.cos_sin_cache if self.rope is not None else None,
                                self.rot_dims, shared.get("v_first"), self.vmix, self.mix_role,
                                self.attn.k_cache, self.attn.v_cache, ctx.slot_mapping)
        return F.linear(self.attn(q, gate), self.o_proj)


class NatilixDeltaMixer(nn.Module):
    def __init__(self, W: int, m: MixerSpec, eps: float):
        super().__init__()
        self.core = GatedDeltaRule(m.heads, m.kv_heads, m.dim, m.vdim, m.conv, eps)
        self.in_proj = nn.Parameter(torch.zeros(sum(self.core.split_sizes()), W), requires_grad=False)
        self.o_proj = nn.Parameter(torch.zeros(W, m.heads * m.vdim), requires_grad=False)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, shared: dict) -> torch.Tensor:
        return F.linear(self.core(F.linear(h, self.in_proj), h.dtype), self.o_proj)


class NatilixLayer(nn.Module):
    def __init__(self, cfg: NatilixConfig, spec: LayerSpec, mix_role: int):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.rms_norm_epsilon
        self.kind = spec.mixer.kind
        self.norm1, self.norm1b = OffsetRMSNorm(W, eps), OffsetRMSNorm(W, eps)
        self.mix = (NatilixAttentionMixer(W, spec.mixer, cfg.max_position, mix_role)
                    if self.kind == "attention" else NatilixDeltaMixer(W, spec.mixer, eps))
        self.mlp = None
        if spec.mlp is not None:
            f = spec.mlp
            self.norm2, self.norm2b = OffsetRMSNorm(W, eps), OffsetRMSNorm(W, eps)
            self.mlp = GroupedRoutedExperts(W, f.ff, f.experts, f.top, f.groups, f.keep)


class NatilixModel(nn.Module):
    def __init__(self, cfg: NatilixConfig):
        super().__init__()
        W = cfg.hidden_size
        self.embed = nn.Parameter(torch.zeros(cfg.vocab_size, W), requires_grad=False)
        b = cfg.bigram
        self.bigram = HashedBigramEmbedding(b["buckets"], W, b["mul_prev"], b["mul_cur"]) if b else None
        layers, seen_mix = [], False
        for spec in cfg.layers:
            role = 0
            if spec.mixer.kind == "attention" and spec.mixer.v_mix:
                role, seen_mix = (2 if seen_mix else 1), True
            layers.append(NatilixLayer(cfg, spec, role))
        self.layers = nn.ModuleList(layers)
        self.eps = cfg.rms_norm_epsilon
        self.act_dtype = self.embed.dtype
        # observers for tests: called with (layer index, fp32 stream) after every layer
        self.layer_hook = None

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the fp32 residual stream [T, W] after the last layer (the final norm belongs
        to the head: only the rows whose logits are wanted go through it)."""
        ctx = get_context()
        dt, eps = self.act_dtype, self.eps
        x = ops.embed_sum(input_ids, ctx.aux_rows, self.embed,
                          self.bigram.weight if self.bigram is not None else None)
        shared: dict = {}
        n = len(self.layers)
        h = self.layers[0].norm1(x, dt) if n else None
        for i, layer in enumerate(self.layers):
            y = layer.mix(h, positions, shared)
            nxt = self.layers[i + 1].norm1.weight if i + 1 < n else None
            if layer.mlp is not None:
                h = ops.post_norm_residual(y, layer.norm1b.weight, x, eps, layer.norm2.weight, dt)
                y = layer.mlp(h)
                h = ops.post_norm_residual(y, layer.norm2b.weight, x, eps, nxt, dt)
            else:
                h = ops.post_norm_residual(y, layer.norm1b.weight, x, eps, nxt, dt)
            if self.layer_hook is not None:
                self.layer_hook(i, x)
        return x


class NormedHead(nn.Module):
    """Final zero-centred norm + untied output projection, applied to the rows a step wants
    (each sequence's last row, or the context's ``logit_rows``)."""

    def __init__(self, vocab_size: int, hidden_size: int, eps: float):
        super().__init__()
        self.norm = OffsetRMSNorm(hidden_size, eps)
        self.weight = nn.Parameter(torch.zeros(vocab_size, hidden_size), requires_grad=False)
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
        return F.linear(self.norm(rows, self.weight.dtype), self.weight)

    def forward(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.local_logits(hidden)


class NatilixForCausalLM(nn.Module):
    has_recurrent_state = True

    def __init__(self, config: NatilixConfig):
        super().__init__()
        self.config = config
        self.model = NatilixModel(config)
        self.lm_head = NormedHead(config.vocab_size, config.hidden_size, config.rms_norm_epsilon)

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
        return [l.mix.attn for l in self.model.layers if l.kind == "attention"]

    def state_layers(self):
        return [l.mix.core for l in self.model.layers if l.kind == "delta"]

    @property
    def needs_aux_rows(self) -> bool:
        """The batch must carry a row of the second embedding table for every token."""
        return self.model.bigram is not None

    def aux_embedding_rows(self, tokens, prev_tokens):
        return self.model.bigram.rows_for(tokens, prev_tokens)

    # ---- weights -----------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, items) -> int:
        """``items``: iterable of (checkpoint name, tensor).  Stacks the per-projection and
        per-expert tensors into the fused parameters; unknown names raise."""
        n = 0
        top = {"embed": self.model.embed, "head": self.lm_head.weight,
               "final.norm": self.lm_head.norm.weight}
        if self.model.bigram is not None:
            top["bigram"] = self.model.bigram.weight
        for name, t in items:
            n += 1
            if name in top:
                _put(top[name], t)
                continue
            li, _, rest = name.partition(".")
            if not (li.startswith("l") and li[1:].isdigit()) or int(li[1:]) >= len(self.model.layers):
                raise KeyError(f"checkpoint tensor {name!r} has no parameter")
            layer = self.model.layers[int(li[1:])]
            if rest in ("norm1", "norm1b", "norm2", "norm2b"):
                _put(getattr(layer, rest).weight, t)
            elif rest.startswith("mix."):
                self._load_mixer(layer, rest[4:], t, name)
            elif rest.startswith("mlp.") and layer.mlp is not None:
                self._load_mlp(layer.mlp, rest[4:], t, name)
            else:
                raise KeyError(f"checkpoint tensor {name!r} has no parameter")
        return n

    @staticmethod
    def _load_mixer(layer, key, t, name):
        mix = layer.mix
        if key == "o":
            return _put(mix.o_proj, t)
        if layer.kind == "attention":
            order = ["q", "k", "v", "g"]
            if key in order:
                return _put_rows(mix.in_proj, mix.sizes, order.index(key), t)
            if key == "sink":
                return _put(mix.attn.sink, t)
            if key == "vmix":
                return _put(mix.vmix, t)
        else:
            core, order = mix.core, ["q", "k", "v", "g", "b", "a"]
            if key in order:
                return _put_rows(mix.in_proj, core.split_sizes(), order.index(key), t)
            convs = ["q.conv", "k.conv", "v.conv"]
            if key in convs:
                return _put_rows(core.conv_weight, core.split_sizes()[:3], convs.index(key), t)
            simple = {"A_log": core.A_log, "dt_bias": core.dt_bias, "norm": core.norm_weight}
            if key in simple:
                return _put(simple[key], t)
        raise KeyError(f"checkpoint tensor {name!r} has no parameter")

    @staticmethod
    def _load_mlp(mlp, key, t, name):
        if key == "router":
            return _put(mlp.router, t)
        e, _, which = key.partition(".")
        if e.startswith("e") and e[1:].isdigit() and int(e[1:]) < mlp.experts:
            j, ff = int(e[1:]), mlp.ff
            if which == "up":
                return _put(mlp.up[j * ff:(j + 1) * ff], t)
            if which == "down":
                return _put(mlp.down[:, j * ff:(j + 1) * ff], t)
        raise KeyError(f"checkpoint tensor {name!r} has no parameter")

    def checkpoint_shapes(self):
        """(name, shape) of every tensor a checkpoint of this configuration holds."""
        c = self.config
        W = c.hidden_size
        yield "embed", (c.vocab_size, W)
        if c.bigram:
            yield "bigram", (c.bigram["buckets"] + 1, W)
        for i, L in enumerate(c.layers):
            p, m = f"l{i}.", L.mixer
            H, G, D, E = m.heads, m.kv_heads, m.dim, m.vdim
            for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if L.mlp else ()):
                yield p + nm, (W,)
            if m.kind == "attention":
                for nm, rows in (("q", H * D), ("k", G * D), ("v", G * E), ("g", H)):
                    yield p + "mix." + nm, (rows, W)
                yield p + "mix.vmix", ()
                yield p + "mix.sink", (H,)
            else:
                for nm, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
                    yield p + "mix." + nm, (rows, W)
                    yield p + "mix." + nm + ".conv", (rows, m.conv)
                for nm, shape in (("b", (H, W)), ("a", (H, W)), ("g", (H * E, W)), ("A_log", (H,)),
                                  ("dt_bias", (H,)), ("norm", (E,))):
                    yield p + "mix." + nm, shape
            yield p + "mix.o", (W, H * E)
            if L.mlp:
                for j in range(L.mlp.experts):
                    yield f"{p}mlp.e{j}.up", (L.mlp.ff, W)
                    yield f"{p}mlp.e{j}.down", (W, L.mlp.ff)
                yield p + "mlp.router", (L.mlp.experts, W)
        yield "final.norm", (W,)
        yield "head", (c.vocab_size, W)

    def random_checkpoint(self, seed: int = 0):
        """Seeded random tensors (values exactly representable in bfloat16) of every checkpoint
        name: scales chosen so that activations stay O(1) through the stack."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        for name, shape in self.checkpoint_shapes():
            leaf = name.rsplit(".", 1)[-1]
            r = torch.randn(shape, generator=g)
            if leaf in ("norm1", "norm1b", "norm2", "norm2b") or name == "final.norm":
                t = 0.1 * r
            elif leaf == "norm":
                t = 1.0 + 0.1 * r
            elif leaf == "conv":
                t = 0.5 * r
            elif leaf == "vmix":
                t = torch.sigmoid(r)
            elif leaf in ("sink", "dt_bias"):
                t = r
            elif leaf == "A_log":
                t = -1.0 + 0.5 * r
            elif name in ("embed", "bigram"):
                t = r
            else:
                t = r * (shape[-1] ** -0.5) * (3.0 if leaf in ("q", "k", "router") else 1.0)
            out[name] = t.to(torch.bfloat16)
        return out

    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        self.load_weights(self.random_checkpoint(seed).items())


def _put(param, t):
    if tuple(param.shape) != tuple(t.shape):
        raise ValueError(f"shape mismatch: parameter {tuple(param.shape)} vs checkpoint {tuple(t.shape)}")
    param.copy_(t.to(param.dtype))


def _put_rows(param, sizes, idx, t):
    lo = sum(sizes[:idx])
    _put(param[lo:lo + sizes[idx]], t)
