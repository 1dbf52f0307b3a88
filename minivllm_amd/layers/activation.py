"""SwiGLU gate: ``silu(x[..., :I]) * x[..., I:]`` (reference:
src/myvllm/layers/activation.py:6-18, there a torch.compile'd function; here one
vectorised HIP kernel on GPU)."""
import torch
import torch.nn as nn

from minivllm_amd import ops


class SiluAndMul(nn.Module):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.silu_and_mul(x)


class XIELU(nn.Module):
    """xIELU with two learned numbers p, q: ``softplus(p) z^2 + z/2`` for z > 0 and
    ``(1/2 + softplus(q)) (e^z - 1 - z) + z/2`` otherwise.  The two coefficients are worked out
    once, when the numbers are loaded, and handed to the kernel as arguments."""

    def __init__(self):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(2, dtype=torch.float32), requires_grad=False)
        self.load(torch.zeros(2))

    @torch.no_grad()
    def load(self, t: torch.Tensor) -> None:
        if tuple(t.shape) != (2,):
            raise ValueError(f"xIELU takes two numbers, got shape {tuple(t.shape)}")
        self.weight.copy_(t.to(torch.float32))
        sp = torch.nn.functional.softplus(t.double())
        self.above, self.below = float(sp[0]), float(0.5 + sp[1])

    def forward(self, u: torch.Tensor, out_dtype=None) -> torch.Tensor:
        return ops.xielu(u, self.above, self.below, out_dtype or u.dtype)
