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


class RoutedGatedExperts(nn.Module):
    """Gated feed-forward experts down(silu(gate x) * (up x)) behind a sigmoid router, plus an
    optional shared expert that every token uses; with ``experts`` = 0 it is a plain dense gated
    feed-forward of size ``shared_ff``.

    Router: s = sigmoid(W_r h) in fp32, the ``top`` largest scores chosen (ties to the lower
    index) and used as weights as they are.  An expert is fed its weight times the row:
    out = sum_j expert_j(s_j h) + shared(h).

    Execution: one stacked gate+up weight [2 C, W], C = experts * ff + shared_ff (all gate rows,
    then all up rows) and one stacked down weight [W, C].  Because the two input projections are
    linear, scaling the input by s_j is scaling their outputs, which the activation kernel does
    (``ops.swiglu_route_scale``; exactly zero for experts a token did not choose): two dense
    GEMMs and one elementwise kernel for routed experts, shared expert and dense layer alike,
    no token permutation, no host synchronisation."""

    def __init__(self, hidden_size: int, ff: int, experts: int, top: int, shared_ff: int = 0):
        super().__init__()
        if experts and not 0 < top <= experts:
            raise ValueError("router: `top` must lie in 1 .. experts")
        self.ff, self.experts, self.top, self.shared_ff = ff, experts, top, shared_ff
        self.columns = experts * ff + shared_ff
        self.router = (nn.Parameter(torch.zeros(experts, hidden_size, dtype=torch.float32),
                                    requires_grad=False) if experts else None)
        self.gate_up = nn.Parameter(torch.zeros(2 * self.columns, hidden_size), requires_grad=False)
        self.down = nn.Parameter(torch.zeros(hidden_size, self.columns), requires_grad=False)

    def column_range(self, expert: int):
        """Columns of expert ``expert`` (-1: the shared one) among the stacked C."""
        if expert < 0:
            return self.experts * self.ff, self.columns
        return expert * self.ff, (expert + 1) * self.ff

    def forward(self, h: torch.Tensor, gu: torch.Tensor = None) -> torch.Tensor:
        """``gu``: the stacked gate+up projection of h when the caller has computed it already
        (as columns of a wider fused projection)."""
        route = (ops.grouped_route(h, self.router, self.top, 1, 1, "sigmoid")
                 if self.experts else None)
        if gu is None:
            gu = F.linear(h, self.gate_up)
        act = ops.swiglu_route_scale(gu, route, self.ff, self.shared_ff, h.dtype)
        return F.linear(act, self.down)


class CappedRoutedExperts(nn.Module):
    """Gated experts with clamped pre-activations behind a router that renormalises over what it
    chose, plus an optional shared expert with a per-token gate.

    Router: z = W_r h + b in fp32; the ``top`` largest logits are chosen (ties to the lower
    index) and their weights are the softmax over those logits alone.  Expert: g = min(gate h, L),
    u = clamp(up h, -L, L), down(g sigmoid(``slope`` g) (u + 1)), no biases; the routing weight
    scales the expert's OUTPUT (the down projection is linear, so it is applied to the
    activation).  Shared expert: the same form with its own size and limit, for every token,
    times sigmoid(w_s . h); w_s is one more row of the router matrix, so its logit comes out of
    the same fp32 pass (``ops.grouped_route(..., gates=1)``).

    Execution as for the other routed layers here: one stacked gate+up weight [2 C, W], C =
    experts * ff + shared_ff (all gate rows, then all up rows), one stacked down weight [W, C],
    the activation exactly zero for experts a token did not choose: two dense GEMMs and one
    elementwise kernel, no permutation, no host synchronisation."""

    def __init__(self, hidden_size: int, ff: int, experts: int, top: int, limit: float,
                 shared_ff: int = 0, shared_limit: float = 0.0, shared_gate: bool = True,
                 slope: float = 1.702):
        super().__init__()
        self.slope = float(slope)
        if not 0 < top <= experts:
            raise ValueError("router: `top` must lie in 1 .. experts")
        self.ff, self.experts, self.top, self.shared_ff = ff, experts, top, shared_ff
        self.limit, self.shared_limit = float(limit), float(shared_limit)
        self.gates = 1 if (shared_ff and shared_gate) else 0
        self.columns = experts * ff + shared_ff
        f32 = dict(dtype=torch.float32)
        self.router = nn.Parameter(torch.zeros(experts + self.gates, hidden_size, **f32), requires_grad=False)
        self.router_bias = nn.Parameter(torch.zeros(experts + self.gates, **f32), requires_grad=False)
        self.gate_up = nn.Parameter(torch.zeros(2 * self.columns, hidden_size), requires_grad=False)
        self.down = nn.Parameter(torch.zeros(hidden_size, self.columns), requires_grad=False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        route = ops.grouped_route(h, self.router, self.top, 1, 1, "chosen", self.router_bias, self.gates)
        act = ops.capped_glu_route_scale(F.linear(h, self.gate_up), route, self.ff, self.shared_ff,
                                         self.limit, self.shared_limit, h.dtype, self.slope)
        return F.linear(act, self.down)
