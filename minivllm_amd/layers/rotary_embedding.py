"""Rotary position embedding table (NeoX / half-split convention).

The reference precomputes ``cos_sin_cache[max_position, head_dim]`` and applies
the rotation in a torch.compile'd function (reference:
src/myvllm/layers/rotary_embedding.py:48-83).  Here the module only owns the fp32
table; the rotation itself is fused with the per-head q/k RMSNorm and the KV-cache
store in one kernel (``ops.qk_norm_rope_store``).  ``forward`` keeps the
reference's standalone ``(positions, q, k) -> (q, k)`` behaviour.
"""
from __future__ import annotations

from functools import lru_cache

import torch
import torch.nn as nn

from minivllm_amd.ops import torch_ref


class RotaryEmbedding(nn.Module):
    def __init__(self, head_size: int, rotary_dim: int, max_position: int, base: float,
                 rope_scaling=None):
        """``rope_scaling``: HF-style dict (``rope_type`` linear / llama3) or None."""
        super().__init__()
        if rotary_dim != head_size:
            raise ValueError("partial rotary is not supported")
        self.head_size = head_size
        self.max_position = max_position
        self.base = base
        self.register_buffer("cos_sin_cache",
                             torch_ref.build_cos_sin_cache(head_size, max_position, base,
                                                           rope_scaling=rope_scaling),
                             persistent=False)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor):
        """query [T,Hq,D] / key [T,Hkv,D] -> rotated copies."""
        cs = self.cos_sin_cache[positions.long()].float()
        cos, sin = cs.chunk(2, dim=-1)
        q = torch_ref.apply_rope(query.float(), cos, sin).to(query.dtype)
        k = torch_ref.apply_rope(key.float(), cos, sin).to(key.dtype)
        return q, k


@lru_cache(maxsize=4)
def get_rope(head_size: int, rotary_dim: int, max_position: int, base: float) -> RotaryEmbedding:
    return RotaryEmbedding(head_size, rotary_dim, max_position, base)


class PairRotaryEmbedding(nn.Module):
    """Rotation of neighbouring pairs (2i, 2i+1) of the first ``rotary_dim`` entries of a head
    (the interleaved convention), the rest passing unchanged.  ``scaling``: None or a dict with
    ``factor / low / high / original`` (the Llama 3.1 rule: wavelengths below original/high
    keep their frequency, above original/low divide it by factor, a linear blend between).
    Owns the fp32 table [max_position, rotary_dim] (cos, then sin) whose angles are formed in
    fp32; the rotation itself happens in ``ops.pair_rope_mix_store``."""

    def __init__(self, rotary_dim: int, max_position: int, base: float, scaling=None):
        super().__init__()
        if rotary_dim % 2:
            raise ValueError("rotary_dim must be even")
        self.rotary_dim = rotary_dim
        from minivllm_amd.ops import torch_seqmix
        self.register_buffer("cos_sin_cache",
                             torch_seqmix.pair_cos_sin_table(rotary_dim, max_position, base, scaling),
                             persistent=False)


class HalfRotation(nn.Module):
    """Rotation in the half-split layout on the first ``rotary_dim`` entries of a vector: entry i
    is paired with entry i + rotary_dim/2 and the pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2i / rotary_dim); later entries pass
    unchanged.  Owns only the fp32 frequencies (rounded from float64); the angle is the fp32
    product of position and frequency, formed where the rotation is applied
    (``ops.latent_rope_store``), so no table and no maximal position."""

    def __init__(self, rotary_dim: int, base: float):
        super().__init__()
        if rotary_dim % 2:
            raise ValueError("rotary_dim must be even")
        self.rotary_dim, self.base = int(rotary_dim), float(base)
        i = torch.arange(rotary_dim // 2, dtype=torch.float64)
        self.register_buffer("inv_freq", (self.base ** (-2.0 * i / max(rotary_dim, 1))).float(),
                             persistent=False)
