"""Real-gated linear recurrent unit (the recurrent block of Griffin: De, Smith et al., "Griffin:
Mixing Gated Linear Recurrences with Local Attention for Efficient Language Models").

Two branches of C channels come out of one projection of the layer's input: y (through a tanh
gelu) and x, which passes a short causal convolution per channel (bias, no activation): u.  The
channels are cut into ``blocks`` equal parts; part k has two square matrices that give the gates
    r = sigmoid(R_k u_k + r_k),   i = sigmoid(I_k u_k + i_k),
and per channel, token after token,
    d = exp(-sharp r softplus(lam)),   S <- d S + sqrt(1 - d^2) (i u),
from S = 0 at a sequence's first token.  The mixer's output is S * y (before its output
projection).  Gates, decay and state are fp32; the two gate matrices of a part are ONE batched
fp32 product [blocks, T, c] x [blocks, c, 2c] (``gate_weight``: R_k^T beside I_k^T).

A pass of the layer keeps per sequence the state S [C] and the convolution's last taps-1 inputs
(``StateSlots``); a layer that runs several times per token with the same weights has one per
pass.  ``sharp`` is the constant in the decay's exponent (8 in Griffin).
"""
from __future__ import annotations

from typing import List

import torch
import torch.nn as nn

from minivllm_amd import ops
from minivllm_amd.layers.state_space import StateSlots
from minivllm_amd.utils.context import get_context


class RealGatedLRU(nn.Module):
    def __init__(self, channels: int, blocks: int, conv_taps: int, sharp: float = 8.0, passes: int = 1):
        super().__init__()
        if blocks < 1 or channels % blocks:
            raise ValueError("the gate blocks must divide the recurrent width")
        self.channels, self.blocks, self.taps, self.sharp = channels, blocks, int(conv_taps), float(sharp)
        c = channels // blocks
        f32 = dict(dtype=torch.float32)
        self.conv_weight = nn.Parameter(torch.zeros(channels, self.taps, **f32), requires_grad=False)
        self.conv_bias = nn.Parameter(torch.zeros(channels, **f32), requires_grad=False)
        self.gate_weight = nn.Parameter(torch.zeros(blocks, c, 2 * c, **f32), requires_grad=False)
        self.gate_bias = nn.Parameter(torch.zeros(blocks, 2 * c, **f32), requires_grad=False)
        self.lam = nn.Parameter(torch.zeros(channels, **f32), requires_grad=False)
        spec = [("state", (channels,)), ("conv_state", (max(self.taps - 1, 0), channels))]
        self.slots: List[StateSlots] = [StateSlots(spec) for _ in range(passes)]

    @torch.no_grad()
    def load_gates(self, ra, ra_b, ri, ri_b) -> None:
        """ra / ri [blocks, c, c] stored [out, in]; biases [blocks, c]."""
        self.gate_weight.copy_(torch.cat([ra.float().transpose(1, 2), ri.float().transpose(1, 2)], 2))
        self.gate_bias.copy_(torch.cat([ra_b.float(), ri_b.float()], 1))

    def forward(self, x: torch.Tensor, y: torch.Tensor, out_dtype: torch.dtype, which: int = 0) -> torch.Tensor:
        """x, y [T, C]: the two branches' projections (bias added; column blocks of one
        projection output will do) -> S * gelu_tanh(y) [T, C]; ``which``: the pass whose state is
        read and advanced."""
        ctx = get_context()
        st = self.slots[which]
        if st.state is None:
            raise RuntimeError("the recurrent unit needs allocated state slots")
        T, C = x.shape
        cu_q = ctx.cu_seqlens_q if ctx.is_prefill else None
        lay = (cu_q, ctx.positions, ctx.state_slots)
        u = ops.short_conv(x, self.conv_weight, self.conv_bias, st.conv_state, *lay,
                           row_seq=ctx.row_seq if ctx.is_prefill else None)
        gates = torch.bmm(u.view(T, self.blocks, C // self.blocks).transpose(0, 1), self.gate_weight)
        return ops.rglru_scan(u, gates, self.gate_bias, self.lam, y, st.state, *lay, self.sharp, out_dtype)
