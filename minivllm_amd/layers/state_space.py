"""State-space mixer in its dual (linear-attention) form, as in Mamba-2: per head a matrix state
S [N, E] with ONE scalar decay per token,

    dt = softplus(z_dt + dt_bias);   S <- exp(-exp(A_log) dt) S + dt B x^T;   y = S^T C + D x

x [H, E], B and C [G, N] (head h reads group h / (H/G)) come out of one short causal convolution
with bias, then silu; y of all heads is multiplied by silu of a gate projection, cut into
``norm_groups`` equal parts that are each divided by their own root mean square, and weighted.
It is the gated outer-product recurrence of ``layers.delta_rule`` without the correction term
(k = B, q = C, v = x, beta = dt), so it runs through the same two ops with ``ssd`` / ``correct``
set.  Step sizes, decays, the state and the norm are fp32.

A pass of the layer keeps its state (S and the convolution's last taps-1 inputs) in a
``StateSlots`` object; a layer that runs several times per token with the same weights has one
per pass.  A sequence that starts at position 0 starts from zeros whatever its slot held.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn

from minivllm_amd import ops
from minivllm_amd.utils.context import get_context


class StateSlots:
    """What one pass of a recurrent layer keeps per sequence: ``spec`` = [(attribute, shape of one
    slot's fp32 row)]; the engine allocates [slots, *shape] for each and sets the attribute."""

    def __init__(self, spec):
        self._spec = list(spec)
        for name, _ in self._spec:
            setattr(self, name, None)

    def state_spec(self):
        return self._spec


class StateSpaceDuality(nn.Module):
    def __init__(self, num_heads: int, groups: int, state_size: int, v_head_dim: int,
                 conv_taps: int, norm_groups: int, eps: float, passes: int = 1):
        super().__init__()
        H, G, N, E = num_heads, groups, state_size, v_head_dim
        if H % G or (H * E) % norm_groups:
            raise ValueError("heads must be a multiple of groups, and norm_groups must divide heads * vdim")
        self.num_heads, self.groups, self.state_size, self.v_head_dim = H, G, N, E
        self.taps, self.norm_groups, self.eps = int(conv_taps), int(norm_groups), eps
        f32 = dict(dtype=torch.float32)
        C = 2 * G * N + H * E
        # channels in the order the recurrence reads them: C (its q), B (its k), x (its v)
        self.conv_weight = nn.Parameter(torch.zeros(C, self.taps, **f32), requires_grad=False)
        self.conv_bias = nn.Parameter(torch.zeros(C, **f32), requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(H, **f32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(H, **f32), requires_grad=False)
        self.skip = nn.Parameter(torch.zeros(H, **f32), requires_grad=False)
        self.norm_weight = nn.Parameter(torch.ones(H * E, **f32), requires_grad=False)
        spec = [("state", (H, N, E)), ("conv_state", (max(self.taps - 1, 0), C))]
        self.slots: List[StateSlots] = [StateSlots(spec) for _ in range(passes)]

    def split_sizes(self):
        """Column blocks of the fused input projection in the order this module reads them:
        C, B, x (the convolved channels), the gate z, the step size's pre-activation."""
        H, G, N, E = self.num_heads, self.groups, self.state_size, self.v_head_dim
        return [G * N, G * N, H * E, H * E, H]

    def forward(self, proj: torch.Tensor, out_dtype: torch.dtype, which: int = 0) -> torch.Tensor:
        """proj [T, >= sum(split_sizes)] -> [T, H*E] (input of the output projection);
        ``which``: the pass whose state is read and advanced."""
        ctx = get_context()
        st = self.slots[which]
        if st.state is None:
            raise RuntimeError("the state-space mixer needs allocated state slots")
        T = proj.shape[0]
        H, G, N, E = self.num_heads, self.groups, self.state_size, self.v_head_dim
        q, k, v, z, dt = proj[:, :sum(self.split_sizes())].split(self.split_sizes(), dim=-1)
        cu_q = ctx.cu_seqlens_q if ctx.is_prefill else None
        lay = (cu_q, ctx.positions, ctx.state_slots)
        qn, kn, vv, step, decay = ops.delta_prepare(
            q.view(T, G, N), k.view(T, G, N), v.view(T, H, E), None, dt, self.conv_weight,
            self.A_log, self.dt_bias, st.conv_state, *lay, row_seq=ctx.row_seq,
            conv_bias=self.conv_bias, ssd=True)
        o = ops.delta_scan(qn, kn, vv, step, decay, st.state, *lay, correct=False)
        return ops.gated_group_norm(o, vv, self.skip, z, self.norm_weight, self.norm_groups,
                                    self.eps, out_dtype)
