"""Linear-attention mixers with a per-sequence matrix state S [D, E] per head, fp32, carried from
token to token in the engine's state slots (a sequence that starts at position 0 starts from
zeros whatever its slot held).  Both take the raw projections of a step's rows and leave the
activation of their gates, which is fp32 work, to the scan kernel.

``MatrixLSTM``: exponential input gate and sigmoid forget gate in the log domain, both soft-capped,
stabilised by a running maximum m that starts at 0:

    i = cap tanh((z_i + b_i) / cap);   f = logsigmoid(cap tanh((z_f + b_f) / cap))
    m' = max(f + m, i);  S <- e^(f+m-m') S + e^(i-m') k v^T;  n <- e^(f+m-m') n + e^(i-m') k
    o = S^T q / (max(|n . q|, e^(-m')) + 1e-6),   q scaled by D^-1/2

then each head's o divided by its root mean square, times a weight over all heads' outputs,
times sigmoid of a gate projection.  (The recurrence is the mLSTM of "xLSTM: Extended Long
Short-Term Memory", Beck et al., 2024.)

``GatedLinearAttention``: a decay per key channel,

    alpha = sigmoid(z_a + b_a)^(1/tau);   S <- diag(alpha) S + k v^T;   o = S^T q

q scaled by D^-1/2, each head's o RMS-normalised with a weight shared by the heads, times silu of
a gate projection.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from minivllm_amd import ops
from minivllm_amd.utils.context import get_context


def _layout(ctx):
    return (ctx.cu_seqlens_q if ctx.is_prefill else None, ctx.positions, ctx.state_slots)


class MatrixLSTM(nn.Module):
    def __init__(self, num_heads: int, head_dim: int, v_head_dim: int, gate_cap: float, eps: float):
        super().__init__()
        H, D, E = num_heads, head_dim, v_head_dim
        self.num_heads, self.head_dim, self.v_head_dim = H, D, E
        self.gate_cap, self.eps = float(gate_cap), eps
        f32 = dict(dtype=torch.float32)
        self.i_bias = nn.Parameter(torch.zeros(H, **f32), requires_grad=False)
        self.f_bias = nn.Parameter(torch.zeros(H, **f32), requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(H * E, **f32), requires_grad=False)
        self.state: Optional[torch.Tensor] = None          # [slots, H, D, E]
        self.norm_state: Optional[torch.Tensor] = None     # [slots, H, Z, D], Z = ceil(E / 16) copies
        self.max_state: Optional[torch.Tensor] = None      # [slots, H, Z]

    def state_spec(self):
        """n and m are kept once per 16 value columns: the scan kernel's workgroups (one per block
        of columns of a head) each read and write their own copy, so none sees another's update."""
        H, D, E = self.num_heads, self.head_dim, self.v_head_dim
        Z = (E + 15) // 16
        return [("state", (H, D, E)), ("norm_state", (H, Z, D)), ("max_state", (H, Z))]

    def split_sizes(self):
        """Column blocks of the fused input projection: q, k, v, output gate, input gate, forget gate."""
        H, D, E = self.num_heads, self.head_dim, self.v_head_dim
        return [H * D, H * D, H * E, H * E, H, H]

    def forward(self, proj: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """proj [T, sum(split_sizes)] -> [T, H*E] (input of the output projection)."""
        if self.state is None:
            raise RuntimeError("the matrix memory needs allocated state slots")
        T = proj.shape[0]
        H, D, E = self.num_heads, self.head_dim, self.v_head_dim
        q, k, v, gate, ig, fg = proj.split(self.split_sizes(), dim=-1)
        o = ops.mlstm_scan(q.view(T, H, D), k.view(T, H, D), v.view(T, H, E), ig, fg, self.i_bias,
                           self.f_bias, self.gate_cap, self.state, self.norm_state, self.max_state,
                           *_layout(get_context()))
        return ops.gated_head_norm(o, self.norm_weight, gate, self.eps, out_dtype,
                                   "sigmoid").view(T, H * E)


class GatedLinearAttention(nn.Module):
    def __init__(self, num_heads: int, head_dim: int, v_head_dim: int, tau: float, eps: float):
        super().__init__()
        H, D, E = num_heads, head_dim, v_head_dim
        self.num_heads, self.head_dim, self.v_head_dim = H, D, E
        self.tau, self.eps = float(tau), eps
        f32 = dict(dtype=torch.float32)
        self.decay_bias = nn.Parameter(torch.zeros(H * D, **f32), requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(E, **f32), requires_grad=False)
        self.state: Optional[torch.Tensor] = None          # [slots, H, D, E]

    def state_spec(self):
        return [("state", (self.num_heads, self.head_dim, self.v_head_dim))]

    def split_sizes(self):
        """Column blocks of the fused input projection: q, k, v, output gate."""
        H, D, E = self.num_heads, self.head_dim, self.v_head_dim
        return [H * D, H * D, H * E, H * E]

    def forward(self, proj: torch.Tensor, decay_raw: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """proj [T, >= sum(split_sizes)] (further columns are the caller's), decay_raw [T, H*D]
        (the decay's pre-activation without its bias) -> [T, H*E]."""
        if self.state is None:
            raise RuntimeError("linear attention needs allocated state slots")
        T = proj.shape[0]
        H, D, E = self.num_heads, self.head_dim, self.v_head_dim
        q, k, v, gate = proj[:, :sum(self.split_sizes())].split(self.split_sizes(), dim=-1)
        o = ops.gla_scan(q.view(T, H, D), k.view(T, H, D), v.view(T, H, E), decay_raw,
                         self.decay_bias, self.tau, self.state, *_layout(get_context()))
        return ops.gated_head_norm(o, self.norm_weight, gate, self.eps, out_dtype,
                                   "silu").view(T, H * E)
