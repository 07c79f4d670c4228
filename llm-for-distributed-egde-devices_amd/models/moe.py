"""Mixture-of-experts feed-forward for layer-spec models.

Router: softmax over all experts in fp32, the ``top`` largest scores renormalised and scaled, or
sigmoid scores taken as they are, or the ``top`` largest logits (with a bias) and a softmax over those
alone (``ops.seqmix.moe_route``).  Experts: clamped or plain silu
gated-linear units, the router's weight on their output or on their input, weights stacked per layer as
``w_gu`` [E, 2 ff, W] (gate rows, then up rows) and ``w_down`` [E, W, ff]; decode-sized steps read
only the chosen experts' rows, prompt-sized steps sort (token, choice) pairs by expert
(``ops.seqmix.moe_experts``).  The shared expert is a dense unit of the same form.  ``forward``
returns the shared expert's output and the chosen experts' outputs with their weights apart: the
layer's output norm adds them up in fp32 in one kernel with the residual add.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from ..ops import seqmix
from .configs import MoESpec
from .layers import Linear


class MoEFeedForward(nn.Module):
    def __init__(self, spec: MoESpec, width: int, dtype, device):
        super().__init__()
        self.spec = spec
        s = spec
        self.router = nn.Parameter(torch.zeros(s.experts, width, dtype=torch.float32, device=device), requires_grad=False)
        self.router_b = nn.Parameter(torch.zeros(s.experts, dtype=torch.float32, device=device), requires_grad=False) \
            if s.router_bias else None
        self.w_gu = nn.Parameter(torch.zeros(s.experts, 2 * s.ff, width, dtype=dtype, device=device), requires_grad=False)
        self.w_down = nn.Parameter(torch.zeros(s.experts, width, s.ff, dtype=dtype, device=device), requires_grad=False)
        if s.shared_ff:
            self.shared_gu = Linear(width, 2 * s.shared_ff, False, dtype, device)
            self.shared_down = Linear(s.shared_ff, width, False, dtype, device)

    def forward(self, h: torch.Tensor):
        """h [T, W] -> (shared expert's output [T, W] or None, expert outputs [T, top, W], weights fp32
        [T, top] still to be applied to them, or None when the experts ran on weighted inputs)."""
        s = self.spec
        idx, wts = seqmix.moe_route(h, self.router, s.top, s.scale, s.router, self.router_b)
        on_input = s.weight_on == "input"
        parts = seqmix.moe_experts(h, idx, self.w_gu, self.w_down, s.limit, s.act, wts if on_input else None)
        if on_input:
            wts = None
        shared = None
        if s.shared_ff:
            shared = self.shared_down(seqmix.glu_clamp(self.shared_gu(h), s.shared_ff, s.shared_limit))
        return shared, parts, wts
