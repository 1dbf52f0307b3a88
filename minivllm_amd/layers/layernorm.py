"""RMSNorm with an optional fused residual add.

Same math as the reference's ``LayerNorm`` module (reference:
src/myvllm/layers/layernorm.py:3-28), which despite its name is an RMSNorm.  Here
the scale is a learnable parameter named ``weight`` (checkpoint compatible) and
``eps`` comes from the model configuration; the reference uses a fixed 1e-5 and a
non-learnable buffer of ones.
"""
from __future__ import annotations

from typing import Optional, Tuple, Union

import torch
import torch.nn as nn

from minivllm_amd import ops


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size), requires_grad=False)
        # True once the scale vector has been multiplied into the weights of the projection
        # that consumes this norm's output (``weight`` is all ones from then on)
        self.folded = False

    @torch.no_grad()
    def fold_into(self, *linear_weights: torch.Tensor) -> None:
        """``norm(x) * g @ W.T == norm(x) @ (W * g).T``: move the scale vector into ``W`` (shape
        [out, in]) so that the normalisation left in front of the GEMM is a per-row scalar."""
        if self.folded:
            return
        g = self.weight.float()
        for w in linear_weights:
            w.copy_((w.float() * g[None, :]).to(w.dtype))
        self.weight.fill_(1.0)
        self.folded = True

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None
                ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        # ``x`` may be a projection's pending work (ops.partials): ops takes it over
        if residual is None:
            return ops.rms_norm(x, self.weight, self.eps)
        return ops.add_rms_norm(x, residual, self.weight, self.eps)


LayerNorm = RMSNorm      # the reference's class name


class OffsetRMSNorm(nn.Module):
    """RMS norm whose stored weight is an offset from one: ``x / rms(x) * (1 + weight)``.  The
    weight stays fp32 whatever the activation dtype is; the op that applies it is chosen by the
    caller (``ops.offset_rms_norm`` alone, or ``ops.post_norm_residual`` when the result is added
    to a fp32 residual stream and the next sublayer's norm follows at once)."""

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.zeros(hidden_size, dtype=torch.float32), requires_grad=False)

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.offset_rms_norm(x, self.weight, self.eps, out_dtype or x.dtype)


class GroupRMSNorm(nn.Module):
    """RMS norm in groups: the vector is cut into ``groups`` equal consecutive parts, each
    divided by its own root mean square (eps inside the root), the whole multiplied by a plain
    fp32 weight.  ``groups`` = 1 is the ordinary RMS norm.  Applied alone (``ops.group_rms_norm``)
    or fused with the update of a fp32 residual stream (``ops.residual_group_norm``)."""

    def __init__(self, hidden_size: int, groups: int = 1, eps: float = 1e-6):
        super().__init__()
        if groups < 1 or hidden_size % groups:
            raise ValueError("the norm's groups must divide the width")
        self.eps, self.groups = eps, groups
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float32), requires_grad=False)

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.group_rms_norm(x, self.weight, self.groups, self.eps, out_dtype or x.dtype)


class ScalarRMSNorm(nn.Module):
    """RMS norm whose gain is ONE number for all coordinates: ``x / rms(x) * gain`` (eps inside
    the root).  The gain is kept as a host float besides the parameter, so that the fused form
    (``ops.residual_sum_norm``: update of the fp32 stream + this norm) takes it as a kernel
    argument.  Applied alone it normalises the rows it is given."""

    def __init__(self, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones((), dtype=torch.float32), requires_grad=False)
        self.gain = 1.0

    @torch.no_grad()
    def load(self, t: torch.Tensor) -> None:
        if t.numel() != 1:
            raise ValueError(f"a scalar norm takes one number, got shape {tuple(t.shape)}")
        self.weight.copy_(t.reshape(()).to(torch.float32))
        self.gain = float(t.reshape(()).float())

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.residual_sum_norm(x, (), (), self.gain, self.eps, out_dtype or x.dtype)
