"""Gated delta rule: a linear-attention mixer whose per-head state S [D, E] is decayed, corrected
towards the new value along the new key, and read out, token after token:

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

with q, k unit vectors (q scaled by D^-1/2) that went through a short causal convolution and
silu, beta = sigmoid(.), g = exp(-exp(A_log) softplus(. + dt_bias)), and the read-out divided
by its root mean square over E, scaled by a shared weight and gated by silu of a projection.
State (S in fp32 and the convolutions' last taps-1 inputs) lives in per-sequence slots handed
out by the scheduler; a sequence that starts at position 0 starts from zeros whatever its slot
held.  Every constant (heads, sizes, taps) is a constructor argument.

``channel_decay``: g is a vector over the key channels of a head (it scales the rows of S),
``dt_bias`` then has H * D entries and the decay's pre-activation arrives as its own tensor
(the caller's low-rank projection) instead of as a column block of the fused projection; so
does the output gate.  ``gate_act``: "silu" or "sigmoid".
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from minivllm_amd import ops
from minivllm_amd.utils.context import get_context


class GatedDeltaRule(nn.Module):
    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 conv_taps: int, eps: float, channel_decay: bool = False, gate_act: str = "silu"):
        super().__init__()
        H, G, D, E = num_heads, num_kv_heads, head_dim, v_head_dim
        self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim = H, G, D, E
        self.taps, self.eps = conv_taps, eps
        self.channel_decay, self.gate_act = channel_decay, gate_act
        f32 = dict(dtype=torch.float32)
        # taps of the q, k and v channels stacked in that order (last column = current token)
        self.conv_weight = nn.Parameter(torch.zeros(2 * G * D + H * E, conv_taps, **f32),
                                        requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(H, **f32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(H * D if channel_decay else H, **f32),
                                    requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(E, **f32), requires_grad=False)
        # [slots, H, D, E] and [slots, taps-1, 2GD + HE], attached by the runner
        self.state: Optional[torch.Tensor] = None
        self.conv_state: Optional[torch.Tensor] = None

    @property
    def conv_channels(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.v_head_dim

    def state_spec(self):
        """(attribute, shape of one slot's row): what the engine allocates per state slot, fp32."""
        H, D, E = self.num_heads, self.head_dim, self.v_head_dim
        return [("state", (H, D, E)), ("conv_state", (max(self.taps - 1, 0), self.conv_channels))]

    def split_sizes(self):
        """Column blocks of the fused input projection: q, k, v, gate, beta, decay (with
        ``channel_decay``: q, k, v, beta; decay and gate come as arguments of ``forward``)."""
        H, G, D, E = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        if self.channel_decay:
            return [G * D, G * D, H * E, H]
        return [G * D, G * D, H * E, H * E, H, H]

    def forward(self, proj: torch.Tensor, out_dtype: torch.dtype,
                a: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
        """proj [T, >= sum(split_sizes)] (further columns are the caller's) -> [T, H*E] (input of
        the output projection).  ``a`` [T, H*D] and ``gate`` [T, H*E]: with ``channel_decay``."""
        ctx = get_context()
        if self.state is None:
            raise RuntimeError("the delta rule needs allocated state slots")
        T = proj.shape[0]
        H, G, D, E = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        n = sum(self.split_sizes())
        if self.channel_decay:
            q, k, v, b = proj[:, :n].split(self.split_sizes(), dim=-1)
        else:
            q, k, v, gate, b, a = proj[:, :n].split(self.split_sizes(), dim=-1)
        cu_q = ctx.cu_seqlens_q if ctx.is_prefill else None
        lay = (cu_q, ctx.positions, ctx.state_slots)
        qn, kn, vv, beta, decay = ops.delta_prepare(
            q.view(T, G, D), k.view(T, G, D), v.view(T, H, E), b, a, self.conv_weight,
            self.A_log, self.dt_bias, self.conv_state, *lay, row_seq=ctx.row_seq)
        o = ops.delta_scan(qn, kn, vv, beta, decay, self.state, *lay)
        return ops.gated_head_norm(o, self.norm_weight, gate, self.eps, out_dtype,
                                   self.gate_act).view(T, H * E)
