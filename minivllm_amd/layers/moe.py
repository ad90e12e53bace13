"""Mixture of small feed-forward experts behind a grouped top-k router.

Router: softmax over all experts (fp32), experts in ``groups`` equal runs of neighbours, a
group scored by its best expert, only the ``keep`` best groups eligible, the ``top`` largest
eligible scores chosen and used as weights without renormalising.  Experts: down(act(up h)),
no biases, act = erf gelu.

Execution: the experts' up projections are one stacked weight [experts*ff, W] and their down
projections one [W, experts*ff]; a step computes ``down_all @ (route ⊙ gelu(up_all h))`` where
``route`` holds each token's weight for the expert a column belongs to and exactly zero for
experts it did not choose.  Two dense GEMMs and one fused activation kernel, no token
permutation, no host synchronisation (so the step can be captured into a graph); the price is
experts/top times the arithmetic of a gathered execution.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from minivllm_amd import ops


class GroupedRoutedExperts(nn.Module):
    def __init__(self, hidden_size: int, ff: int, experts: int, top: int, groups: int, keep: int):
        super().__init__()
        if experts % groups or not (0 < keep <= groups) or top > experts // groups * keep:
            raise ValueError("router: groups must divide experts and the kept groups must hold "
                             "at least `top` experts")
        self.ff, self.experts, self.top, self.groups, self.keep = ff, experts, top, groups, keep
        self.router = nn.Parameter(torch.zeros(experts, hidden_size, dtype=torch.float32),
                                   requires_grad=False)
        self.up = nn.Parameter(torch.zeros(experts * ff, hidden_size), requires_grad=False)
        self.down = nn.Parameter(torch.zeros(hidden_size, experts * ff), requires_grad=False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        route = ops.grouped_route(h, self.router, self.top, self.groups, self.keep)
        act = ops.gelu_route_scale(F.linear(h, self.up), route, self.ff, h.dtype)
        return F.linear(act, self.down)
