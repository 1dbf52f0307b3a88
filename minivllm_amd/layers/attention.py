"""Attention layer over a paged KV cache, plus the three kernel entry points the
reference exposes.

Reference (src/myvllm/layers/attention.py:67-108, 212-280, 418-473, 476-557):
``store_kvcache`` scatters new K/V rows into the cache, prefill runs a varlen
causal flash-attention over the *new* tokens only (so a cached prefix is silently
ignored), decode runs one-query paged attention with a ``block_size`` that is
never wired to the engine's.  Here the cache tensor itself defines the block
size, prefill attends through the block table whenever a cache is attached
(``q_len <= k_len``, so prefix-cache hits and re-prefill after preemption are
exact), and K/V are written by the fused norm+RoPE+store kernel upstream, not by
this layer.

Cache tensors are logically ``[num_blocks, block_size, num_kv_heads, head_dim]``;
the engine allocates them with a head-major physical order so that one
(block, kv-head) pair is one contiguous slab for the decode kernel.
"""
from __future__ import annotations

import math
import os
from typing import Optional

import torch
import torch.nn as nn

from minivllm_amd import ops
from minivllm_amd.utils.context import get_context


# ----------------------------------------------- reference-signature functions
def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                  block_size: Optional[int] = None) -> None:
    if block_size is not None and block_size != k_cache.shape[1]:
        raise ValueError(f"block_size={block_size} does not match the cache ({k_cache.shape[1]})")
    ops.store_kvcache(key, value, k_cache, v_cache, slot_mapping)


def flash_attention_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                            cu_seqlens: torch.Tensor, scale: float,
                            num_heads: Optional[int] = None, num_kv_heads: Optional[int] = None,
                            head_dim: Optional[int] = None,
                            max_seqlen: Optional[int] = None) -> torch.Tensor:
    """q [T,Hq,D], k/v [T,Hkv,D], causal, packed by ``cu_seqlens``.  ``scale`` is the
    full softmax scale (1/sqrt(D) already included)."""
    return ops.flash_attention_prefill(q, k, v, cu_seqlens, scale, max_seqlen)


def paged_attention_decode(query: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_tables: torch.Tensor, context_lens: torch.Tensor, scale: float,
                           num_heads: Optional[int] = None, num_kv_heads: Optional[int] = None,
                           head_dim: Optional[int] = None, block_size: Optional[int] = None,
                           max_context_len: Optional[int] = None) -> torch.Tensor:
    if block_size is not None and block_size != k_cache.shape[1]:
        raise ValueError(f"block_size={block_size} does not match the cache ({k_cache.shape[1]})")
    return ops.paged_attention_decode(query, k_cache, v_cache, block_tables, context_lens, scale,
                                      max_context_len)


# --------------------------------------------------------------------- layer
# MINIVLLM_NO_Q_FUSE=1: q-norm + RoPE of the Q rows stay in the store kernel (for A/B timing)
_FUSE_Q_ROPE = os.environ.get("MINIVLLM_NO_Q_FUSE", "0") != "1"
# MINIVLLM_NO_DECODE_FUSE=1: decode steps keep the stand-alone norm + rotate + store kernel
_FUSE_DECODE_STORE = os.environ.get("MINIVLLM_NO_DECODE_FUSE", "0") != "1"


class Attention(nn.Module):
    def __init__(self, num_heads: int, head_dim: int, scale: float = 1.0,
                 num_kv_heads: Optional[int] = None, block_size: Optional[int] = None):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.num_kv_heads = num_kv_heads or num_heads
        # like the reference, ``scale`` multiplies 1/sqrt(head_dim) (attention.py:512)
        self.scale = scale / math.sqrt(head_dim)
        self.block_size = block_size
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None

    @staticmethod
    def fuses_q_rope(ctx, q: torch.Tensor) -> bool:
        """True for the steps whose attention transforms raw Q rows itself (``q_rope``): pure
        prefill steps on the GPU.  Decode rows (decode steps, the riders of a mixed step) go
        through the decode kernel, which expects finished queries."""
        return bool(_FUSE_Q_ROPE and ctx.is_prefill and not ctx.num_decode_seqs and q.is_cuda)

    def fuses_decode_store(self, ctx, qkv: torch.Tensor) -> bool:
        """True for the steps whose attention takes the raw q / k / v projections and does the
        norm, the rotation and the cache write itself (``new_kv``): pure decode steps on the GPU
        with a 16-bit cache whose positions are ``context_lens - 1`` (the engine's are)."""
        return bool(_FUSE_DECODE_STORE and not ctx.is_prefill and qkv.is_cuda
                    and ctx.positions_in_context and self.k_cache is not None
                    and self.k_cache.dtype != torch.float8_e4m3fn and self.head_dim in (64, 128))

    def reads_k_from_cache(self, ctx) -> bool:
        """True for prefill steps whose attention goes through the block table of a 16-bit cache
        (the freshly projected ``k`` / ``v`` arguments of ``forward`` are then never read)."""
        return bool(ctx.is_prefill and self.k_cache is not None and ctx.block_tables is not None
                    and ctx.slot_mapping is not None and self.k_cache.dtype != torch.float8_e4m3fn)

    def forward(self, q: torch.Tensor, k: Optional[torch.Tensor] = None,
                v: Optional[torch.Tensor] = None, q_rope=None, new_kv=None) -> torch.Tensor:
        """q [T,Hq,D] (rows may be strided); k/v [T,Hkv,D] are only read when no cache
        is attached.  ``q_rope`` (prefill steps only): q holds the raw projection, see
        ``ops.flash_attention_prefill``.  ``new_kv`` = (cos_sin, q_norm weight, k_norm weight,
        eps) (decode steps only, ``fuses_decode_store``): q, k and v are raw projections, see
        ``ops.paged_attention_decode``.  Returns [T, Hq*D]."""
        ctx = get_context()
        T = q.shape[0]
        assert q_rope is None or self.fuses_q_rope(ctx, q)
        assert new_kv is None or self.fuses_decode_store(ctx, q)
        if ctx.is_prefill and ctx.num_decode_seqs:
            return self._mixed(q, ctx)
        if ctx.is_prefill:
            paged = self.k_cache is not None and ctx.block_tables is not None
            if paged and self.k_cache.dtype == torch.float8_e4m3fn and not ctx.has_prefix \
                    and k is not None:
                paged = False       # nothing cached yet: attend to the exact K/V just projected
            if paged:
                o = ops.paged_attention_prefill(q, self.k_cache, self.v_cache, ctx.cu_seqlens_q,
                                                ctx.cu_seqlens_k, ctx.block_tables, self.scale,
                                                ctx.max_seqlen_q, max_seqlen_k=ctx.max_seqlen_k,
                                                total_k=ctx.total_k_tokens, q_rope=q_rope,
                                                work_items=ctx.prefill_items,
                                                positions_in_context=ctx.positions_in_context)
            else:
                o = ops.flash_attention_prefill(q, k, v, ctx.cu_seqlens_q, self.scale,
                                                ctx.max_seqlen_q, q_rope=q_rope)
        else:
            if self.k_cache is None:
                raise RuntimeError("decode needs an allocated KV cache")
            o = ops.paged_attention_decode(q, self.k_cache, self.v_cache, ctx.block_tables,
                                           ctx.context_lens, self.scale, ctx.max_context_len,
                                           new_kv=(k, v) + tuple(new_kv) if new_kv is not None else None)
        return o.reshape(T, self.num_heads * self.head_dim)

    def _mixed(self, q: torch.Tensor, ctx) -> torch.Tensor:
        """The decode rows (the first ``num_decode_seqs`` rows and sequence slots) through the
        decode kernel, the prompt rows behind them through the prefill kernel (a one-row query
        in the prefill kernel would stream the KV of its sequence once per query head and fill
        1 of 128 tile rows), one output buffer.  Rows that belong to no sequence (padding of the
        token bucket, unused slots of a captured step) are left as they are."""
        if self.k_cache is None or ctx.block_tables is None:
            raise RuntimeError("a mixed prefill + decode step needs an allocated KV cache")
        T = q.shape[0]
        Bd = ctx.num_decode_seqs
        o = q.new_empty((T, self.num_heads, self.head_dim)) if q.is_cuda \
            else q.new_zeros((T, self.num_heads, self.head_dim))
        if ctx.num_seqs > Bd:
            # cu_seqlens hold absolute rows, so q and o go in whole
            ops.paged_attention_prefill(q, self.k_cache, self.v_cache,
                                        ctx.cu_seqlens_q[Bd:], ctx.cu_seqlens_k[Bd:],
                                        ctx.block_tables[Bd:], self.scale, ctx.max_seqlen_q,
                                        out=o, max_seqlen_k=ctx.max_seqlen_k,
                                        total_k=ctx.total_k_tokens, work_items=ctx.prefill_items)
        ops.paged_attention_decode(q[:Bd], self.k_cache, self.v_cache,
                                   ctx.block_tables[:Bd], ctx.context_lens, self.scale,
                                   ctx.max_context_len, out=o[:Bd])
        return o.reshape(T, self.num_heads * self.head_dim)


class SinkAttention(nn.Module):
    """Causal attention over a paged cache whose softmax denominator carries one extra term
    ``exp(sink_h)`` per query head (no key, no value), with key and value heads of different
    sizes (K cache [blocks, block, G, D], V cache [blocks, block, G, E]) and an optional
    per-head output gate ``sigmoid(gate_h)`` applied inside the kernel.  ``scale`` is the full
    score multiplier.  Scores, weights and the weighted sum are fp32 in every implementation.

    Options, each a constructor argument: ``sink=False`` - an ordinary softmax (no extra term);
    ``window`` > 0 - a query at position i sees key j <= i only when i - j < window or
    j < keep_first (the first tokens stay visible at their true positions); ``distance_slopes``
    [H] - slope_h * (i - j) is taken off the score of key j; ``value_in_key`` - a token's value is
    the leading ``v_head_dim`` entries of its key row, so the engine allocates no V cache and
    ``v_cache`` is a view into ``k_cache``; ``head_temps`` - a learned multiplier per query head
    on the scaled score (``temps`` [H] fp32); ``softcap`` > 0 - score <- softcap tanh(score /
    softcap) after scale and temperature; ``pool`` > 0 (needs a window) - besides the window's
    tokens a query at position i sees ONE key and value for every block of ``pool`` tokens that
    has passed out of its window as a whole (b pool + pool - 1 <= i - window): the means of the
    block's cached keys and values, kept in ``k_pool`` / ``v_pool`` [pages, rows, G, D|E] that the engine
    allocates next to the token caches (``block_cache_spec``) and ``update_pools`` fills once the
    step's tokens are cached; block rows and token rows are weighed in the same softmax."""

    def __init__(self, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, sink: bool = True, window: int = 0, keep_first: int = 0,
                 distance_slopes: Optional[torch.Tensor] = None, value_in_key: bool = False,
                 head_temps: bool = False, softcap: float = 0.0, pool: int = 0):
        super().__init__()
        if pool and (not window or keep_first or value_in_key or distance_slopes is not None):
            raise ValueError("pooled blocks need a window and combine with neither kept first "
                             "tokens, a distance penalty nor values inside the key rows")
        self.softcap, self.pool = float(softcap), int(pool) if window else 0
        self.temps = (nn.Parameter(torch.ones(num_heads, dtype=torch.float32), requires_grad=False)
                      if head_temps else None)
        self.k_pool: Optional[torch.Tensor] = None
        self.v_pool: Optional[torch.Tensor] = None
        if value_in_key and v_head_dim > head_dim:
            raise ValueError("values inside the key rows cannot be longer than the keys")
        self.value_in_key = bool(value_in_key)
        self.num_heads, self.num_kv_heads = num_heads, num_kv_heads
        self.head_dim, self.v_head_dim, self.scale = head_dim, v_head_dim, scale
        self.window, self.keep_first = int(window), int(keep_first)
        self.sink = (nn.Parameter(torch.zeros(num_heads, dtype=torch.float32), requires_grad=False)
                     if sink else None)
        if distance_slopes is not None:
            self.register_buffer("slopes", distance_slopes.to(torch.float32), persistent=False)
        else:
            self.slopes = None
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None

    def block_cache_spec(self, block_size: int):
        """Further per-page allocations next to the K / V caches: [(attribute, which cache it
        follows in memory, (rows per page, G, d))].  A pooled row's address is its page's, so
        rows * pool covers a page of tokens; the engine places each behind the cache named, in
        ONE allocation, and the kernels reach pooled rows as further rows of that cache."""
        if not self.pool:
            return []
        rows = -(-block_size // self.pool)
        return [("k_pool", "k_cache", (rows, self.num_kv_heads, self.head_dim)),
                ("v_pool", "v_cache", (rows, self.num_kv_heads, self.v_head_dim))]

    def update_pools(self) -> None:
        """After the step's keys and values are cached: the block means of every block that a
        token of this step completes."""
        if not self.pool:
            return
        ctx = get_context()
        ops.pool_block_means(self.k_cache, self.v_cache, self.k_pool, self.v_pool, self.pool,
                             ctx.positions, ctx.block_tables,
                             ctx.row_seq if ctx.is_prefill else None, ctx.slot_mapping)

    def forward(self, q: torch.Tensor, gate: Optional[torch.Tensor]) -> torch.Tensor:
        """q [T,H,D] (rotated; rows may be strided), gate [T,H] raw or None; K/V of every token
        of the step are in the cache already.  Returns [T, H*E]."""
        ctx = get_context()
        if self.k_cache is None:
            raise RuntimeError("attention needs an allocated KV cache")
        T = q.shape[0]
        out = torch.zeros((T, self.num_heads, self.v_head_dim), dtype=q.dtype, device=q.device)
        a = (self.k_cache, self.v_cache)
        opt = dict(window=self.window, keep_first=self.keep_first, slopes=self.slopes)
        if self.temps is not None or self.softcap or self.pool:
            opt.update(temps=self.temps, softcap=self.softcap, pool=self.pool, k_pool=self.k_pool,
                       v_pool=self.v_pool)
        if not ctx.is_prefill:
            ops.sink_attention_decode(q, *a, ctx.block_tables, ctx.context_lens, self.scale,
                                      self.sink, gate, out, ctx.max_context_len or None, **opt)
        else:
            # prompt portions through the prefill kernel, the single next tokens that ride along
            # (the first num_decode_seqs rows and sequences) through the decode kernel
            Bd = ctx.num_decode_seqs
            if ctx.num_seqs > Bd:
                ops.sink_attention_prefill(q, *a, ctx.cu_seqlens_q[Bd:], ctx.cu_seqlens_k[Bd:],
                                           ctx.block_tables[Bd:], self.scale, self.sink, gate, out,
                                           positions=ctx.positions, max_q=ctx.max_seqlen_q or None,
                                           row_seq=ctx.row_seq, first_seq=Bd, **opt)
            if Bd:
                ops.sink_attention_decode(q[:Bd], *a, ctx.block_tables[:Bd], ctx.context_lens,
                                          self.scale, self.sink,
                                          None if gate is None else gate[:Bd], out[:Bd],
                                          ctx.max_context_len or None, **opt)
        return out.view(T, self.num_heads * self.v_head_dim)


class LatentAttention(nn.Module):
    """Attention whose keys and values are expansions of one cached latent per token: key of
    head h = [W_uk_h c | r], value = W_uv_h c, with c the RMS-normed latent (R numbers) and r one
    rotated key part (P numbers) shared by all heads.  Only c and r are cached, and the
    expansions are never formed: with a_h = W_uk_h^T q_h the score is (a_h . c + q_rot_h . r) *
    scale, and the weighted sum of values is W_uv_h applied to the weighted sum of latents.  So
    this is attention with ONE key/value head whose key row is [c | r] (R + P) and whose value row
    is c (R), run by ``SinkAttention`` (no sink; its window and kernels), between two batched
    products per head.  ``up_k`` [H, D, R] and ``up_v`` [H, E, R] are the per-head expansion
    matrices; ``rotation``: a ``HalfRotation`` over the first entries of the P-part.  Only c and r
    are cached, once: the values are read from the key rows (``value_in_key``)."""

    def __init__(self, num_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, kv_rank: int,
                 scale: float, window: int, rotation, eps: float):
        super().__init__()
        H, D, P, E, R = num_heads, head_dim, rot_dim, v_head_dim, kv_rank
        self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank = H, D, P, E, R
        self.eps, self.rotation = eps, rotation
        if rotation.rotary_dim > P:
            raise ValueError("the rotation covers more entries than the rotated part has")
        self.core = self.make_core(H, P, R, scale, window)
        self.latent_norm = nn.Parameter(torch.ones(R, dtype=torch.float32), requires_grad=False)
        self.up_k = nn.Parameter(torch.zeros(H, D, R), requires_grad=False)
        self.up_v = nn.Parameter(torch.zeros(H, E, R), requires_grad=False)

    @staticmethod
    def make_core(num_heads: int, rot_dim: int, kv_rank: int, scale: float, window: int) -> SinkAttention:
        """A cache holder of this attention (one per pass of a layer that runs several times):
        one KV head, key rows [c | r], values = the leading R entries of the key rows."""
        return SinkAttention(num_heads, 1, kv_rank + rot_dim, kv_rank, scale, sink=False,
                             window=window, value_in_key=True)

    def forward(self, q: torch.Tensor, dkv: torch.Tensor, core: Optional[SinkAttention] = None
                ) -> torch.Tensor:
        """q [T, H, D + P] (the rotated part last), dkv [T, R + P] raw -> [T, H, E] as a
        transposed view of [H, T, E].  ``core``: the cache holder of this pass (default: the
        module's own)."""
        ctx = get_context()
        core = core or self.core
        T = q.shape[0]
        H, D, R = self.num_heads, self.head_dim, self.kv_rank
        q_abs = torch.bmm(q[:, :, :D].transpose(0, 1), self.up_k)                    # [H, T, R]
        rot = self.rotation
        qf = ops.latent_rope_store(q_abs, q, dkv, self.latent_norm, self.eps, ctx.positions,
                                   rot.inv_freq, rot.rotary_dim, core.k_cache,
                                   None if core.value_in_key else core.v_cache, ctx.slot_mapping)
        o = core(qf, None).view(T, H, R)
        return torch.bmm(o.transpose(0, 1), self.up_v.transpose(1, 2)).transpose(0, 1)   # [T, H, E]
