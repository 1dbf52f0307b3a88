"""ctypes bindings for ``_hip_hybrid.so`` (``csrc/hybrid``): the gfx950 kernels of hybrid
decoders.  Same conventions as ``ops.hip``: raw device pointers, element strides, the current
HIP stream (so calls made during graph capture become graph nodes), no PyTorch fallback.  The
library is built on first use when it is missing (a few seconds, hipcc only).  Tensors are
bfloat16 or float32 (``dt`` 0 / 2); fp32 tensors (stream, state, router, norm weights) are always
fp32.  Function signatures mirror ``ops.torch_seqmix``.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                         "_hip_hybrid.so")
if not os.path.exists(_LIB_PATH):
    from minivllm_amd import build as _build
    _build.build_hip_group("hybrid", verbose=False)
_lib = ctypes.CDLL(_LIB_PATH)

_L, _I, _F, _P = ctypes.c_long, ctypes.c_int, ctypes.c_float, ctypes.c_void_p


def _sig(name, *argtypes):
    f = getattr(_lib, name)
    f.argtypes = list(argtypes)
    f.restype = ctypes.c_int
    return f


_embed = _sig("hyb_embed_sum", _P, _P, _P, _P, _P, _L, _I, _F, _I, _P)
_norm = _sig("hyb_offset_rms_norm", _P, _P, _P, _L, _I, _F, _I, _P)
_post = _sig("hyb_post_norm_residual", _P, _L, _P, _P, _P, _P, _L, _I, _F, _I, _P)
_rope = _sig("hyb_pair_rope_mix_store", _P, _P, _P, _L, _P, _P, _I, _P, _P, _I, _P, _P, _P, _L,
             _I, _I, _I, _I, _I, _P)
_ghn = _sig("hyb_gated_head_norm", _P, _P, _P, _L, _P, _L, _I, _I, _F, _I, _I, _I, _P)
_route = _sig("hyb_grouped_route", _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _I, _P)
_gelu = _sig("hyb_gelu_route_scale", _P, _P, _P, _L, _I, _I, _I, _P)
_POOL = (_P, _F, _I, _I, _L)        # head temperatures, soft cap, pool, pooled rows per page, first pooled row
_attn = _sig("hyb_sink_attention_rows", _P, _L, _L, _P, _P, _P, _I, _I, _P, _P, _I, _P, _P, _L, _P,
             _F, _L, _I, _I, _I, _I, _I, _I, _I, _P, _I, *_POOL, _I, _P)
_tiles = _sig("hyb_sink_attention_tiles", _P, _L, _L, _P, _P, _P, _I, _I, _P, _P, _P, _P, _L, _P, _F,
              _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _I, *_POOL, _I, _P)
_tiles_ok = _lib.hyb_sink_attention_tiles_ok
_tiles_ok.argtypes = [_I, _I]
_tiles_ok.restype = _I
_split = _sig("hyb_sink_attention_split", _P, _L, _L, _P, _P, _P, _I, _I, _P, _P, _P, _L, _P, _P, _F,
              _I, _I, _I, _I, _I, _I, _I, _I, _P, _I, *_POOL, _I, _P)
_split_ok = _lib.hyb_sink_attention_split_ok
_split_ok.argtypes = [_I, _I]
_split_ok.restype = _I
_prep = _sig("hyb_delta_prepare", _P, _L, _I, _P, _L, _I, _P, _I, _P, _I, _P, _P, _P, _P, _P, _P, _P,
             _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _I, _P)
_scan = _sig("hyb_delta_scan", _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P)
_cscan = _sig("hyb_channel_delta_scan", _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P)
_gla = _sig("hyb_gla_scan", _P, _P, _P, _L, _L, _L, _P, _L, _P, _F, _P, _P, _P, _P, _P, _I, _I, _I, _I,
            _I, _P)
_mlstm = _sig("hyb_mlstm_scan", _P, _P, _P, _L, _L, _L, _P, _P, _L, _P, _P, _F, _P, _P, _P, _P, _P, _P,
              _P, _I, _I, _I, _I, _I, _P)
_esin = _sig("hyb_embed_sinusoid", _P, _P, _P, _P, _P, _L, _I, _I, _P)
_rgn = _sig("hyb_residual_group_norm", _P, _P, _L, _P, _L, _P, _P, _L, _I, _I, _F, _I, _P)
_anm = _sig("hyb_add_normed_mean", _P, _P, _L, _P, _P, _L, _P, _L, _I, _F, _I, _P)
_uns = _sig("hyb_unit_norm_store", _P, _P, _L, _F, _P, _P, _P, _L, _I, _I, _I, _I, _P)
_swi = _sig("hyb_swiglu_route_scale", _P, _L, _P, _P, _L, _I, _I, _I, _I, _P)
_cap = _sig("hyb_tanh_cap", _P, _L, _F, _I, _P)
_rsn = _sig("hyb_residual_sum_norm", _P, _P, _P, _P, _I, _F, _P, _L, _I, _F, _I, _P)
_rnr = _sig("hyb_rms_norm_rows", _P, _L, _P, _P, _L, _I, _F, _I, _P)
_rns = _sig("hyb_row_norm_store", _P, _P, _P, _L, _P, _P, _F, _P, _P, _P, _L, _I, _I, _I, _I, _P)
_lrs = _sig("hyb_latent_rope_store", _P, _P, _L, _P, _L, _P, _F, _P, _P, _I, _P, _P, _P, _P, _L, _I,
            _I, _I, _I, _I, _P)
_xie = _sig("hyb_xielu", _P, _L, _P, _L, _I, _F, _F, _I, _P)
_ggn = _sig("hyb_gated_group_norm", _P, _P, _P, _P, _L, _P, _P, _L, _I, _I, _I, _F, _I, _P)
_sgt = _sig("hyb_sigmoid_gate", _P, _L, _L, _P, _L, _P, _L, _I, _I, _I, _P)
_hrs = _sig("hyb_half_rope_store", _P, _P, _P, _L, _P, _P, _I, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P)
_pbm = _sig("hyb_pool_block_means", _P, _P, _P, _P, _P, _P, _P, _I, _P, _L, _I, _I, _I, _I, _I, _I, _I, _P)
_utg = _sig("hyb_unturn_gate", _P, _L, _L, _P, _P, _P, _L, _P, _L, _I, _I, _I, _P)
_scv = _sig("hyb_short_conv", _P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _P)
_lru = _sig("hyb_rglru_scan", _P, _P, _P, _P, _P, _L, _P, _P, _P, _P, _P, _L, _I, _I, _I, _F, _I, _I, _P)
_crt = _sig("hyb_chosen_route", _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P)
_cgl = _sig("hyb_capped_glu_route_scale", _P, _L, _P, _P, _L, _I, _I, _I, _I, _F, _F, _F, _I, _P)

_DT = {torch.bfloat16: 0, torch.float32: 2}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"hybrid kernels take bfloat16 / float32 activations, got {t.dtype}")


def _stream() -> int:
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _check(rc: int, name: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{name} failed (code {rc}): shape outside the kernel's range or a "
                           f"HIP launch error")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _f32(t: torch.Tensor) -> torch.Tensor:
    assert t.dtype == torch.float32 and t.is_contiguous(), "fp32 contiguous tensor expected"
    return t


def _i32(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None:
        return None
    assert t.dtype == torch.int32 and t.is_contiguous()
    return t


def _rows(t: torch.Tensor) -> int:
    """Row stride (elements) of a [T, ...] view whose trailing dims are dense."""
    assert t.stride(-1) == 1
    return t.stride(0) if t.shape[0] > 1 else int(t.stride(0) or t[0].numel())


# ------------------------------------------------------------------ embedding + norms
def embed_sum(ids, aux_rows, table, aux_table, scale=1.0):
    T, W = ids.shape[0], table.shape[1]
    x = torch.empty((T, W), dtype=torch.float32, device=table.device)
    _check(_embed(_ptr(_i32(ids)), _ptr(_i32(aux_rows)) if aux_table is not None else None,
                  table.data_ptr(), _ptr(aux_table), x.data_ptr(), T, W, float(scale), _dt(table), _stream()),
           "embed_sum")
    return x


def offset_rms_norm(x, w, eps, out_dtype):
    x = _f32(x)
    T, W = x.shape
    out = torch.empty((T, W), dtype=out_dtype, device=x.device)
    _check(_norm(x.data_ptr(), _f32(w).data_ptr(), out.data_ptr(), T, W, eps, _dt(out), _stream()),
           "offset_rms_norm")
    return out


def post_norm_residual(y, wb, x, eps, w_next, out_dtype):
    x = _f32(x)
    T, W = x.shape
    assert y.shape == x.shape and y.stride(-1) == 1 and y.dtype == out_dtype
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if w_next is not None else None
    _check(_post(y.data_ptr(), y.stride(0), _f32(wb).data_ptr(), x.data_ptr(),
                 _ptr(w_next), _ptr(h), T, W, eps, _dt(y), _stream()), "post_norm_residual")
    return h


# ------------------------------------------------------------------ rotation, value mix, store
def pair_rope_mix_store(q, k, v, positions, cos_sin, rot_dims, v_first, lam, v_mode,
                        k_cache, v_cache, slot_mapping):
    T, H, D = q.shape
    G, E = v.shape[1], v.shape[2]
    rs = q.stride(0)
    assert (T == 1 or (k.stride(0) == rs and v.stride(0) == rs)) and q.stride(1) == D \
        and k.stride(1) == D and v.stride(1) == E and q.stride(2) == 1, \
        "q / k / v must be views of one projection output"
    if k_cache is not None:
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype
    if rot_dims:
        assert cos_sin.shape[1] == rot_dims and cos_sin.dtype == torch.float32
    if v_mode:
        assert v_first is not None and v_first.is_contiguous() and v_first.dtype == q.dtype \
            and v_first.numel() == T * G * E
    _check(_rope(q.data_ptr(), k.data_ptr(), v.data_ptr(), rs, _i32(positions).data_ptr(),
                 _ptr(cos_sin) if rot_dims else None, rot_dims, _ptr(v_first) if v_mode else None,
                 _f32(lam).data_ptr(), v_mode, _ptr(k_cache), _ptr(v_cache), _ptr(_i32(slot_mapping)),
                 T, H, G, D, E, _dt(q), _stream()), "pair_rope_mix_store")


# ------------------------------------------------------------------ attention with a sink
def _slopes(slopes, H):
    if slopes is None:
        return None
    assert slopes.dtype == torch.float32 and slopes.is_contiguous() and slopes.numel() == H
    return slopes.data_ptr()


def _value_rows(k_cache, v_cache):
    """Elements from one (slot, KV head) value row to the next.  The V cache is a dense tensor
    [blocks, block, G, E] or, when the values are stored inside the key rows, a view
    [blocks, block, G, E] of the leading E entries of each wider row."""
    n, bs, G, E = v_cache.shape
    vs = v_cache.stride(2) if G > 1 else v_cache.stride(1)
    assert v_cache.stride(3) == 1 and vs >= E and v_cache.stride(1) == G * vs \
        and (n == 1 or v_cache.stride(0) == bs * G * vs), "value rows must be evenly spaced"
    assert v_cache.dtype == k_cache.dtype and v_cache.shape[:3] == k_cache.shape[:3]
    return vs


def _pool_args(k_cache, v_cache, vs, H, temps, softcap, pool, k_pool, v_pool):
    """(temps, softcap, pool, pooled rows per page, first pooled row) for the attention kernels.
    The pooled caches lie behind the token caches in the same allocations, the same number of
    rows behind both."""
    tp = None
    if temps is not None:
        assert temps.dtype == torch.float32 and temps.is_contiguous() and temps.numel() == H
        tp = temps.data_ptr()
    if not pool:
        return tp, float(softcap), 0, 0, 0
    n, bs, G, D = k_cache.shape
    es = k_cache.element_size()
    assert k_pool.is_contiguous() and v_pool.is_contiguous() and k_pool.shape[0] == n \
        and k_pool.shape[2:] == (G, D) and v_pool.shape[:3] == k_pool.shape[:3] \
        and k_pool.shape[1] * pool >= bs and k_pool.dtype == k_cache.dtype
    base = (k_pool.data_ptr() - k_cache.data_ptr()) // (G * D * es)
    assert base > 0 and k_cache.data_ptr() + base * G * D * es == k_pool.data_ptr() \
        and v_cache.data_ptr() + base * G * vs * es == v_pool.data_ptr(), \
        "the pooled rows must follow their token cache in one allocation"
    return tp, float(softcap), int(pool), int(k_pool.shape[1]), int(base)


def _attention_rows(q, k_cache, v_cache, block_tables, row_seq, lens, len_add, scale, sink, gate, out,
                    seq_base=0, window=0, keep_first=0, slopes=None, temps=None, softcap=0.0, pool=0,
                    k_pool=None, v_pool=None):
    T, H, D = q.shape
    G, E = k_cache.shape[2], v_cache.shape[3]
    assert q.stride(2) == 1 and out.is_contiguous() and out.shape == (T, H, E) and out.dtype == q.dtype
    assert k_cache.is_contiguous() and k_cache.dtype == q.dtype
    vs = _value_rows(k_cache, v_cache)
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    if gate is not None:
        assert gate.stride(1) == 1 and gate.dtype == q.dtype
    _check(_attn(q.data_ptr(), q.stride(0), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                 block_tables.data_ptr(), block_tables.stride(0), k_cache.shape[1],
                 _ptr(_i32(row_seq)), _i32(lens).data_ptr(), len_add,
                 _f32(sink).data_ptr() if sink is not None else None,
                 _ptr(gate), gate.stride(0) if gate is not None else 0, out.data_ptr(), scale, T,
                 H, G, D, E, seq_base, int(window), int(keep_first), _slopes(slopes, H), vs,
                 *_pool_args(k_cache, v_cache, vs, H, temps, softcap, pool, k_pool, v_pool), _dt(q),
                 _stream()), "sink_attention")
    return out


def sink_attention_step(q, k_cache, v_cache, block_tables, row_seq, positions, scale, sink, gate, out,
                        seq_base=0, window=0, keep_first=0, slopes=None, **pooled):
    """Rows of a prefill-form step, one workgroup per row: row t belongs to sequence
    ``row_seq[t]`` (< ``seq_base``: skipped), whose block table is row ``row_seq[t] - seq_base``
    of ``block_tables``, and sees ``positions[t] + 1`` keys."""
    return _attention_rows(q, k_cache, v_cache, block_tables, row_seq, positions, 1, scale, sink,
                           gate, out, seq_base, window, keep_first, slopes, **pooled)


def sink_attention_prefill(q, k_cache, v_cache, cu_q, cu_k, block_tables, scale, sink, gate, out,
                           positions=None, max_q=None, row_seq=None, first_seq=0,
                           window=0, keep_first=0, slopes=None, temps=None, softcap=0.0, pool=0,
                           k_pool=None, v_pool=None):
    """The prompt portions of a step: sequence b owns rows cu_q[b] .. cu_q[b+1] (absolute rows
    of q / out / positions) and block table row b.  Runs the matrix-core tile kernel (fp32
    scores, weights and sums); head sizes it has no instance for go row by row.  ``cu_k`` is
    not needed (a row's context is its position + 1)."""
    T, H, D = q.shape
    G, E = k_cache.shape[2], v_cache.shape[3]
    nseq = cu_q.shape[0] - 1
    assert positions is not None, "the GPU form takes the rows' positions"
    if not _tiles_ok(D, E):
        assert row_seq is not None
        # ``first_seq``: number of the step's sequences ahead of these (its decode riders)
        return sink_attention_step(q, k_cache, v_cache, block_tables, row_seq, positions, scale,
                                   sink, gate, out, seq_base=first_seq, window=window,
                                   keep_first=keep_first, slopes=slopes, temps=temps,
                                   softcap=softcap, pool=pool, k_pool=k_pool, v_pool=v_pool)
    if max_q is None:
        max_q = int((cu_q[1:] - cu_q[:-1]).max())
    assert q.stride(2) == 1 and out.is_contiguous() and out.shape == (T, H, E) and out.dtype == q.dtype
    assert k_cache.is_contiguous() and k_cache.dtype == q.dtype
    vs = _value_rows(k_cache, v_cache)
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    if gate is not None:
        assert gate.stride(1) == 1 and gate.dtype == q.dtype
    _check(_tiles(q.data_ptr(), q.stride(0), q.stride(1), k_cache.data_ptr(), v_cache.data_ptr(),
                  block_tables.data_ptr(), block_tables.stride(0), k_cache.shape[1],
                  _i32c(cu_q).data_ptr(), _i32(positions).data_ptr(),
                  _f32(sink).data_ptr() if sink is not None else None,
                  _ptr(gate), gate.stride(0) if gate is not None else 0, out.data_ptr(), scale,
                  nseq, 0, max_q, H, G, D, E, int(window), int(keep_first), _slopes(slopes, H), vs,
                  *_pool_args(k_cache, v_cache, vs, H, temps, softcap, pool, k_pool, v_pool),
                  _dt(q), _stream()), "sink_attention_prefill")
    return out


def _i32c(t):
    assert t.dtype == torch.int32 and t.stride(0) == 1
    return t


def decode_splits(batch: int, kv_heads: int, heads: int, max_context_len) -> int:
    """Workgroups per (sequence, KV head group) of the split decode kernel: enough to fill the
    256 CUs several times over, each with at least 128 keys of the longest context."""
    groups = kv_heads * -(-(heads // kv_heads) // 4)
    want = max(1, 2048 // max(batch * groups, 1))
    room = max(1, (int(max_context_len) + 127) // 128) if max_context_len else 8
    return max(1, min(16, want, room))


def sink_attention_decode(q, k_cache, v_cache, block_tables, context_lens, scale, sink, gate, out,
                          max_context_len=None, window=0, keep_first=0, slopes=None, temps=None,
                          softcap=0.0, pool=0, k_pool=None, v_pool=None):
    """Single next tokens: row b is sequence b with ``context_lens[b]`` keys.  Head sizes the
    split-context kernel has an instance for (D in 64 / 128 / 256, E in 64 / 128) stream K / V
    rows with coalesced 16-byte loads over several workgroups per sequence and are merged by a
    second small kernel; other sizes go through the row kernel."""
    B, H, D = q.shape
    G, E = k_cache.shape[2], v_cache.shape[3]
    es = q.element_size()
    vs = _value_rows(k_cache, v_cache)
    if (_split_ok(D, E) and q.stride(2) == 1 and q.stride(1) == D and q.data_ptr() % 16 == 0
            and (B == 1 or (q.stride(0) * es) % 16 == 0) and k_cache.is_contiguous()
            and vs % 8 == 0 and v_cache.data_ptr() % 16 == 0 and out.is_contiguous()):
        seen = max_context_len
        if window and seen:           # what a row can see bounds the useful splits
            seen = min(int(seen), int(window) + int(keep_first) + (int(seen) // pool if pool else 0))
        splits = decode_splits(B, G, H, seen)
        ws = torch.empty((B * H * splits * (E + 2),), dtype=torch.float32, device=q.device)
        if gate is not None:
            assert gate.stride(1) == 1 and gate.dtype == q.dtype
        _check(_split(q.data_ptr(), q.stride(0) if B > 1 else H * D, q.stride(1), k_cache.data_ptr(),
                      v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                      k_cache.shape[1], _i32c(context_lens).data_ptr(),
                      _f32(sink).data_ptr() if sink is not None else None,
                      _ptr(gate), gate.stride(0) if gate is not None else 0, out.data_ptr(),
                      ws.data_ptr(), scale, B, H, G, D, E, splits, int(window), int(keep_first),
                      _slopes(slopes, H), vs,
                      *_pool_args(k_cache, v_cache, vs, H, temps, softcap, pool, k_pool, v_pool),
                      _dt(q), _stream()),
               "sink_attention_decode")
        return out
    return _attention_rows(q, k_cache, v_cache, block_tables, None, context_lens, 0, scale, sink,
                           gate, out, 0, window, keep_first, slopes, temps, softcap, pool, k_pool, v_pool)


# ------------------------------------------------------------------ gated delta rule
def delta_prepare(q, k, v, b, a, conv_w, a_log, dt_bias, conv_state, cu_q, positions, slots,
                  row_seq, conv_bias=None, ssd=False):
    T, G, D = q.shape
    H, E = v.shape[1], v.shape[2]
    rs = q.stride(0)
    base = q.data_ptr()
    es = q.element_size()
    # q, k, v are the first three column blocks of one projection output, b a view of it; a is a
    # view of it too or a tensor of its own, [T, H] (a decay per head) or [T, H*D] (per key channel)
    assert k.data_ptr() == base + G * D * es and v.data_ptr() == base + 2 * G * D * es
    assert T == 1 or (k.stride(0) == rs and v.stride(0) == rs and (ssd or b.stride(0) == rs))
    assert a.dtype == q.dtype and a.stride(-1) == 1 and a.shape[-1] in (H, H * D)
    DC = a.shape[-1] // H
    assert dt_bias.numel() == H * DC and (not ssd or DC == 1)
    b_off = 0 if ssd else (b.data_ptr() - base) // es
    if conv_bias is not None:
        assert conv_bias.numel() == 2 * G * D + H * E
    dev = q.device
    taps = _f32(conv_w).shape[1]
    assert conv_w.shape[0] == 2 * G * D + H * E
    f = dict(dtype=torch.float32, device=dev)
    qn, kn = torch.empty((T, G, D), **f), torch.empty((T, G, D), **f)
    vv, beta = torch.empty((T, H, E), **f), torch.empty((T, H), **f)
    decay = torch.empty((T, H) if DC == 1 else (T, H, D), **f)
    if cu_q is not None:
        assert row_seq is not None, "prefill-form steps pass the sequence of each row"
    B = slots.shape[0]
    _check(_prep(base, rs if T > 1 else int(rs or 0), b_off, a.data_ptr(), a.stride(0), DC,
                 conv_w.data_ptr(), taps, _ptr(_f32(conv_bias)) if conv_bias is not None else None,
                 int(bool(ssd)), _f32(a_log).data_ptr(), _f32(dt_bias).data_ptr(), _f32(conv_state).data_ptr(), _ptr(_i32(cu_q)),
                 _i32(positions).data_ptr(), _i32(slots).data_ptr(),
                 _ptr(_i32(row_seq)) if cu_q is not None else None, qn.data_ptr(), kn.data_ptr(),
                 vv.data_ptr(), beta.data_ptr(), decay.data_ptr(), T, B, H, G, D, E, _dt(q),
                 _stream()), "delta_prepare")
    return qn, kn, vv, beta, decay


def delta_scan(qn, kn, vv, beta, decay, state, cu_q, positions, slots, correct=True):
    T, G, D = qn.shape
    H, E = vv.shape[1], vv.shape[2]
    assert state.shape[1:] == (H, D, E)
    o = torch.zeros((T, H, E), dtype=torch.float32, device=qn.device)
    if decay.dim() == 3:                 # a decay per head and key channel
        assert decay.shape == (T, H, D) and decay.is_contiguous() and correct
        _check(_cscan(qn.data_ptr(), kn.data_ptr(), vv.data_ptr(), beta.data_ptr(), decay.data_ptr(),
                      _f32(state).data_ptr(), _ptr(_i32(cu_q)), _i32(positions).data_ptr(),
                      _i32(slots).data_ptr(), o.data_ptr(), slots.shape[0], H, G, D, E, _stream()),
               "channel_delta_scan")
        return o
    _check(_scan(qn.data_ptr(), kn.data_ptr(), vv.data_ptr(), beta.data_ptr(), decay.data_ptr(),
                 _f32(state).data_ptr(), _ptr(_i32(cu_q)), _i32(positions).data_ptr(),
                 _i32(slots).data_ptr(), o.data_ptr(), slots.shape[0], H, G, D, E, int(bool(correct)),
                 _stream()), "delta_scan")
    return o


def gated_head_norm(o, w, gate, eps, out_dtype, act="silu"):
    T, H, E = o.shape
    assert gate.stride(-1) == 1 and gate.dtype == out_dtype and w.numel() in (E, H * E)
    assert act in ("silu", "sigmoid")
    out = torch.empty((T, H, E), dtype=out_dtype, device=o.device)
    _check(_ghn(_f32(o).data_ptr(), _f32(w).data_ptr(), gate.data_ptr(), gate.stride(0),
                out.data_ptr(), T, H, E, eps, int(w.numel() == H * E and H > 1), int(act == "sigmoid"),
                _dt(out), _stream()), "gated_head_norm")
    return out


# ------------------------------------------------------------------ grouped expert routing
def grouped_route(h, router_w, top, groups, keep, score="softmax", bias=None, gates=0):
    T, W = h.shape
    if score == "chosen":
        NR = router_w.shape[0]
        assert groups == 1 and keep == 1 and h.is_contiguous() and 0 <= gates < NR
        dense = torch.empty((T, NR), dtype=torch.float32, device=h.device)
        _check(_crt(h.data_ptr(), _f32(router_w).data_ptr(), _ptr(_f32(bias)) if bias is not None else None,
                    dense.data_ptr(), T, W, NR - gates, NR, top, _dt(h), _stream()), "chosen_route")
        return dense
    assert score in ("softmax", "sigmoid") and bias is None and not gates
    NE = router_w.shape[0]
    assert h.is_contiguous()
    dense = torch.empty((T, NE), dtype=torch.float32, device=h.device)
    _check(_route(h.data_ptr(), _f32(router_w).data_ptr(), dense.data_ptr(), T, W, NE, top, groups,
                  keep, int(score == "sigmoid"), _dt(h), _stream()), "grouped_route")
    return dense


def gelu_route_scale(up, dense, ff, out_dtype):
    T = up.shape[0]
    NE = dense.shape[1]
    assert up.is_contiguous() and up.dtype == out_dtype and up.shape[1] == NE * ff
    act = torch.empty_like(up)
    _check(_gelu(up.data_ptr(), _f32(dense).data_ptr(), act.data_ptr(), T, NE, ff, _dt(up),
                 _stream()), "gelu_route_scale")
    return act


def swiglu_route_scale(gu, dense, ff, shared_ff, out_dtype):
    T = gu.shape[0]
    C = gu.shape[1] // 2
    NE = dense.shape[1] if dense is not None else 0
    assert gu.stride(1) == 1 and gu.dtype == out_dtype and C == NE * ff + shared_ff
    act = torch.empty((T, C), dtype=out_dtype, device=gu.device)
    _check(_swi(gu.data_ptr(), _rows(gu), _ptr(_f32(dense)) if dense is not None else None,
                act.data_ptr(), T, NE, ff if NE else 1, shared_ff, _dt(gu), _stream()),
           "swiglu_route_scale")
    return act


# ------------------------------------------------------------------ positions, grouped norms
def embed_sinusoid(ids, positions, table, inv_freq):
    T, W = ids.shape[0], table.shape[1]
    assert table.is_contiguous() and inv_freq.numel() == W // 2
    x = torch.empty((T, W), dtype=torch.float32, device=table.device)
    _check(_esin(_i32(ids).data_ptr(), _i32(positions).data_ptr(), table.data_ptr(),
                 _f32(inv_freq).data_ptr(), x.data_ptr(), T, W, _dt(table), _stream()), "embed_sinusoid")
    return x


def group_rms_norm(x, w, groups, eps, out_dtype):
    return residual_group_norm(x, (), w, groups, eps, out_dtype)


def residual_group_norm(x, ys, w_next, groups, eps, out_dtype):
    x = _f32(x)
    T, W = x.shape
    ys = list(ys)
    assert len(ys) <= 2, "at most two branches are added per call"
    for y in ys:
        assert y.shape == x.shape and y.stride(1) == 1 and y.dtype == out_dtype
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if w_next is not None else None
    if h is None and not ys:
        return None
    y1 = ys[0] if ys else None
    y2 = ys[1] if len(ys) > 1 else None
    _check(_rgn(x.data_ptr(), _ptr(y1), _rows(y1) if y1 is not None else 0, _ptr(y2),
                _rows(y2) if y2 is not None else 0, _ptr(w_next), _ptr(h), T, W, groups, eps,
                _DT[out_dtype], _stream()), "residual_group_norm")
    return h


def add_normed_mean(x, parts, eps):
    x = _f32(x)
    T, W = x.shape
    assert 1 <= len(parts) <= 2
    (y1, w1), (y2, w2) = parts[0], (parts[1] if len(parts) > 1 else (None, None))
    for y in (y1, y2):
        assert y is None or (y.shape == x.shape and y.stride(1) == 1 and y.dtype == y1.dtype)
    _check(_anm(x.data_ptr(), y1.data_ptr(), _rows(y1), _f32(w1).data_ptr(), _ptr(y2),
                _rows(y2) if y2 is not None else 0, _f32(w2).data_ptr() if w2 is not None else None,
                T, W, eps, _dt(y1), _stream()), "add_normed_mean")


def unit_norm_store(q, k, eps, k_cache, v_cache, slot_mapping):
    T, H, D = q.shape
    G = k.shape[1]
    rs = q.stride(0)
    assert (T == 1 or k.stride(0) == rs) and q.stride(1) == D and k.stride(1) == D \
        and q.stride(2) == 1 and k.stride(2) == 1, "q / k must be views of one projection output"
    if k_cache is not None:
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype \
            and k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (G, D)
    _check(_uns(q.data_ptr(), k.data_ptr(), rs, eps, _ptr(k_cache), _ptr(v_cache),
                _ptr(_i32(slot_mapping)), T, H, G, D, _dt(q), _stream()), "unit_norm_store")


def tanh_cap_(z, cap):
    assert z.is_contiguous()
    _check(_cap(z.data_ptr(), z.numel(), cap, _dt(z), _stream()), "tanh_cap")
    return z


# ------------------------------------------------------------------ gated outer-product recurrences
def _heads_view(t, n):
    """Element stride per token of a [T, heads, n] view whose heads are dense."""
    assert t.stride(2) == 1 and t.stride(1) == n
    return _rows(t)


def mlstm_scan(q, k, v, i_raw, f_raw, i_bias, f_bias, cap, state, norm_state, max_state,
               cu_q, positions, slots):
    T, H, D = q.shape
    E = v.shape[2]
    ZG = (E + 15) // 16
    assert state.shape[1:] == (H, D, E) and norm_state.shape[1:] == (H, ZG, D) \
        and max_state.shape[1:] == (H, ZG)
    assert i_raw.shape == (T, H) and f_raw.shape == (T, H) and i_raw.stride(1) == 1 and f_raw.stride(1) == 1
    assert T == 1 or i_raw.stride(0) == f_raw.stride(0)
    assert k.dtype == q.dtype and v.dtype == q.dtype and i_raw.dtype == q.dtype and f_raw.dtype == q.dtype
    o = torch.zeros((T, H, E), dtype=torch.float32, device=q.device)
    _check(_mlstm(q.data_ptr(), k.data_ptr(), v.data_ptr(), _heads_view(q, D), _heads_view(k, D),
                  _heads_view(v, E), i_raw.data_ptr(), f_raw.data_ptr(), _rows(i_raw),
                  _f32(i_bias).data_ptr(), _f32(f_bias).data_ptr(), cap, _f32(state).data_ptr(),
                  _f32(norm_state).data_ptr(), _f32(max_state).data_ptr(), _ptr(_i32(cu_q)),
                  _i32(positions).data_ptr(), _i32(slots).data_ptr(), o.data_ptr(), slots.shape[0],
                  H, D, E, _dt(q), _stream()), "mlstm_scan")
    return o


def gla_scan(q, k, v, a_raw, a_bias, tau, state, cu_q, positions, slots):
    T, H, D = q.shape
    E = v.shape[2]
    assert state.shape[1:] == (H, D, E) and a_raw.shape == (T, H * D) and a_raw.stride(1) == 1
    assert k.dtype == q.dtype and v.dtype == q.dtype and a_raw.dtype == q.dtype
    assert a_bias.numel() == H * D
    o = torch.zeros((T, H, E), dtype=torch.float32, device=q.device)
    _check(_gla(q.data_ptr(), k.data_ptr(), v.data_ptr(), _heads_view(q, D), _heads_view(k, D),
                _heads_view(v, E), a_raw.data_ptr(), _rows(a_raw), _f32(a_bias).data_ptr(), tau,
                _f32(state).data_ptr(), _ptr(_i32(cu_q)), _i32(positions).data_ptr(),
                _i32(slots).data_ptr(), o.data_ptr(), slots.shape[0], H, D, E, _dt(q), _stream()),
           "gla_scan")
    return o


# ------------------------------------------------------------------ scaled branches, latent keys
def rms_norm_rows(x, w, eps, out_dtype):
    T, n = x.shape
    assert x.stride(1) == 1 and x.dtype == out_dtype and w.numel() == n
    out = torch.empty((T, n), dtype=out_dtype, device=x.device)
    _check(_rnr(x.data_ptr(), _rows(x), _f32(w).data_ptr(), out.data_ptr(), T, n, eps, _dt(x),
                _stream()), "rms_norm_rows")
    return out


def residual_sum_norm(x, ys, scales, gain, eps, out_dtype):
    x = _f32(x)
    T, W = x.shape
    ys = list(ys)
    assert len(ys) <= 4 and len(ys) == len(scales), "at most four branches are added per call"
    for y in ys:
        assert y.shape == x.shape and y.stride(1) == 1 and y.dtype == out_dtype
    h = torch.empty((T, W), dtype=out_dtype, device=x.device) if gain is not None else None
    if h is None and not ys:
        return None
    n = len(ys)
    ptrs = (ctypes.c_void_p * 4)(*[y.data_ptr() for y in ys], *([None] * (4 - n)))
    strides = (ctypes.c_long * 4)(*[_rows(y) for y in ys], *([0] * (4 - n)))
    sc = (ctypes.c_float * 4)(*[float(v) for v in scales], *([0.0] * (4 - n)))
    _check(_rsn(x.data_ptr(), ptrs, strides, sc, n, float(gain) if gain is not None else 0.0,
                _ptr(h), T, W, eps, _DT[out_dtype], _stream()), "residual_sum_norm")
    return h


def row_norm_store(q, k, v, qw, kw, eps, k_cache, v_cache, slot_mapping):
    T, H, D = q.shape
    G, E = v.shape[1], v.shape[2]
    rs = q.stride(0)
    assert (T == 1 or (k.stride(0) == rs and v.stride(0) == rs)) and q.stride(1) == D \
        and k.stride(1) == D and v.stride(1) == E and q.stride(2) == 1 and k.stride(2) == 1 \
        and v.stride(2) == 1, "q / k / v must be views of one projection output"
    assert (qw is None) == (kw is None)
    if qw is not None:
        assert qw.numel() == H * D and kw.numel() == G * D
    if k_cache is not None:
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype \
            and k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (G, E)
    _check(_rns(q.data_ptr(), k.data_ptr(), v.data_ptr(), rs, _ptr(_f32(qw)) if qw is not None else None,
                _ptr(_f32(kw)) if kw is not None else None, eps, _ptr(k_cache), _ptr(v_cache),
                _ptr(_i32(slot_mapping)), T, H * D, G * D, G * E, _dt(q), _stream()), "row_norm_store")


def latent_rope_store(q_abs, q, dkv, w, eps, positions, inv_freq, rot_dims, k_cache, v_cache,
                      slot_mapping):
    H, T, R = q_abs.shape
    P = dkv.shape[1] - R
    D = q.shape[2] - P
    assert q_abs.is_contiguous() and q_abs.dtype == q.dtype and dkv.dtype == q.dtype
    assert q.shape[:2] == (T, H) and q.stride(2) == 1 and q.stride(1) == D + P and dkv.stride(1) == 1
    assert w.numel() == R and inv_freq.numel() * 2 == rot_dims
    if k_cache is not None:
        assert k_cache.is_contiguous() and k_cache.dtype == q.dtype and k_cache.shape[2:] == (1, R + P)
        if v_cache is not None:          # None: the values are the leading part of the key rows
            assert v_cache.is_contiguous() and v_cache.shape[2:] == (1, R)
    out = torch.empty((T, H, R + P), dtype=q.dtype, device=q.device)
    _check(_lrs(q_abs.data_ptr(), q.data_ptr(), _rows(q), dkv.data_ptr(), _rows(dkv),
                _f32(w).data_ptr(), eps, _i32(positions).data_ptr(), _f32(inv_freq).data_ptr(),
                int(rot_dims), _ptr(k_cache), _ptr(v_cache), _ptr(_i32(slot_mapping)), out.data_ptr(),
                T, H, D, P, R, _dt(q), _stream()), "latent_rope_store")
    return out


def xielu(u, ap, aq, out_dtype):
    T, n = u.shape
    assert u.stride(1) == 1 and u.dtype == out_dtype
    act = torch.empty((T, n), dtype=out_dtype, device=u.device)
    _check(_xie(u.data_ptr(), _rows(u), act.data_ptr(), T, n, float(ap), float(aq), _dt(u),
                _stream()), "xielu")
    return act


def gated_group_norm(o, skip_x, skip_w, z, w, groups, eps, out_dtype):
    T, H, E = o.shape
    assert skip_x.shape == o.shape and z.shape == (T, H * E) and z.stride(1) == 1 \
        and z.dtype == out_dtype and w.numel() == H * E and skip_w.numel() == H
    out = torch.empty((T, H * E), dtype=out_dtype, device=o.device)
    _check(_ggn(_f32(o).data_ptr(), _f32(skip_x).data_ptr(), _f32(skip_w).data_ptr(), z.data_ptr(),
                _rows(z), _f32(w).data_ptr(), out.data_ptr(), T, H, E, int(groups), eps,
                _DT[out_dtype], _stream()), "gated_group_norm")
    return out


def sigmoid_gate(o, gate, out_dtype):
    T, H, E = o.shape
    assert o.stride(2) == 1 and gate.shape == (T, H * E) and gate.stride(1) == 1 \
        and o.dtype == out_dtype and gate.dtype == out_dtype
    out = torch.empty((T, H * E), dtype=out_dtype, device=o.device)
    _check(_sgt(o.data_ptr(), o.stride(0), o.stride(1), gate.data_ptr(), _rows(gate), out.data_ptr(),
                T, H, E, _dt(o), _stream()), "sigmoid_gate")
    return out


# ------------------------------------------------------------------ rotated values, pooled blocks
def half_rope_store(q, k, v, positions, inv_freq, rot_dims, v_inv_freq, k_cache, v_cache, slot_mapping):
    T, H, D = q.shape
    G, E = v.shape[1], v.shape[2]
    rs = q.stride(0)
    assert (T == 1 or (k.stride(0) == rs and v.stride(0) == rs)) and q.stride(1) == D \
        and k.stride(1) == D and v.stride(1) == E and q.stride(2) == 1, \
        "q / k / v must be views of one projection output"
    if k_cache is not None:
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype \
            and k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (G, E)
    if rot_dims:
        assert inv_freq.numel() * 2 == rot_dims
    if v_inv_freq is not None:
        assert v_inv_freq.numel() * 2 == E
    _check(_hrs(q.data_ptr(), k.data_ptr(), v.data_ptr(), rs if T > 1 else int(rs or 0),
                _i32(positions).data_ptr(), _ptr(_f32(inv_freq)) if rot_dims else None, int(rot_dims),
                _ptr(_f32(v_inv_freq)) if v_inv_freq is not None else None, _ptr(k_cache), _ptr(v_cache),
                _ptr(_i32(slot_mapping)), T, H, G, D, E, _dt(q), _stream()), "half_rope_store")


def pool_block_means(k_cache, v_cache, k_pool, v_pool, pool, positions, block_tables, row_seq,
                     slot_mapping):
    n, bs, G, D = k_cache.shape
    E = v_cache.shape[3]
    T = positions.shape[0] if row_seq is None else min(positions.shape[0], row_seq.shape[0])
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_pool.is_contiguous() \
        and v_pool.is_contiguous() and k_pool.dtype == k_cache.dtype and v_pool.dtype == k_cache.dtype
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    if row_seq is None:
        assert block_tables.shape[0] >= T
    _check(_pbm(k_cache.data_ptr(), v_cache.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(),
                _i32(positions).data_ptr(), _i32(slot_mapping).data_ptr(), block_tables.data_ptr(),
                block_tables.stride(0), _ptr(_i32(row_seq)), T, bs, int(pool), k_pool.shape[1], G, D, E,
                _dt(k_cache), _stream()), "pool_block_means")


def unturn_gate(o, positions, v_inv_freq, gate, out_dtype):
    T, H, E = o.shape
    assert o.stride(2) == 1 and o.dtype == out_dtype
    if gate is not None:
        assert gate.shape == (T, H * E) and gate.stride(1) == 1 and gate.dtype == out_dtype
    if v_inv_freq is not None:
        assert v_inv_freq.numel() * 2 == E
    out = torch.empty((T, H * E), dtype=out_dtype, device=o.device)
    _check(_utg(o.data_ptr(), o.stride(0), o.stride(1), _i32(positions).data_ptr(),
                _ptr(_f32(v_inv_freq)) if v_inv_freq is not None else None, _ptr(gate),
                _rows(gate) if gate is not None else 0, out.data_ptr(), T, H, E, _dt(o), _stream()),
           "unturn_gate")
    return out


# ------------------------------------------------------------------ real-gated diagonal recurrence
def short_conv(x, w, bias, conv_state, cu_q, positions, slots, row_seq):
    T, C = x.shape
    taps = _f32(w).shape[1]
    assert x.stride(1) == 1 and w.shape[0] == C
    if cu_q is not None:
        assert row_seq is not None, "prefill-form steps pass the sequence of each row"
    if taps > 1:
        assert _f32(conv_state).shape[1:] == (taps - 1, C)
    u = torch.empty((T, C), dtype=torch.float32, device=x.device)
    B = slots.shape[0]
    _check(_scv(x.data_ptr(), _rows(x), w.data_ptr(), _ptr(_f32(bias)) if bias is not None else None,
                _ptr(conv_state) if taps > 1 else None, _ptr(_i32(cu_q)), _i32(positions).data_ptr(),
                _i32(slots).data_ptr(), _ptr(_i32(row_seq)) if cu_q is not None else None,
                u.data_ptr(), T, B, C, taps, _dt(x), _stream()), "short_conv")
    return u


def scan_waves(rows: int, seqs: int, channels: int) -> int:
    """Parts a sequence's rows are cut into by the recurrence kernel (one wave each): enough
    workgroups x waves to fill the chip, parts of at least 32 rows."""
    per_seq = max(1, rows // max(seqs, 1))
    want = max(1, 4096 // max(seqs * ((channels + 63) // 64), 1))
    return max(1, min(16, want, per_seq // 32))


def rglru_scan(u, gates, gate_bias, lam, y, state, cu_q, positions, slots, sharp, out_dtype):
    T, C = u.shape
    nb = gates.shape[0]
    assert _f32(u) is u and _f32(gates).shape == (nb, T, 2 * (C // nb)) and _f32(gate_bias).shape == (nb, 2 * (C // nb))
    assert y.shape == (T, C) and y.stride(1) == 1 and y.dtype == out_dtype and _f32(state).shape[1] == C
    out = torch.empty((T, C), dtype=out_dtype, device=u.device)
    B = slots.shape[0]
    nw = scan_waves(T, B, C) if cu_q is not None else 1
    _check(_lru(u.data_ptr(), gates.data_ptr(), gate_bias.data_ptr(), _f32(lam).data_ptr(),
                y.data_ptr(), _rows(y), state.data_ptr(), _ptr(_i32(cu_q)), _i32(positions).data_ptr(),
                _i32(slots).data_ptr(), out.data_ptr(), T, B, C, nb, float(sharp), nw, _DT[out_dtype],
                _stream()), "rglru_scan")
    return out


def capped_glu_route_scale(gu, dense, ff, shared_ff, limit, shared_limit, out_dtype, slope=1.702):
    T = gu.shape[0]
    C = gu.shape[1] // 2
    NR = dense.shape[1]
    NE = (C - shared_ff) // ff
    assert gu.stride(1) == 1 and gu.dtype == out_dtype and C == NE * ff + shared_ff and NR in (NE, NE + 1)
    act = torch.empty((T, C), dtype=out_dtype, device=gu.device)
    _check(_cgl(gu.data_ptr(), _rows(gu), _f32(dense).data_ptr(), act.data_ptr(), T, NE, NR, ff,
                shared_ff, float(limit), float(shared_limit), float(slope), _dt(gu), _stream()),
           "capped_glu_route_scale")
    return act
