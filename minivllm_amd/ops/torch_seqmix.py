"""Plain PyTorch forms of the ops that hybrid decoders add to the dense ones: norms with a
zero-centred weight around a fp32 residual stream, rotation of neighbouring pairs with value
mixing, attention with a sink term and separate key / value head sizes (optionally windowed,
with kept first tokens and a distance penalty), the gated delta rule with its short
convolutions, routing over grouped experts; and, for decoders with parallel sublayers, grouped
norms, sinusoidal positions, gated linear attention, the matrix LSTM and sigmoid-routed gated
experts.  They run CPU tensors (the
engine's CPU mode) and serve as the shape-for-shape counterpart of the gfx950 kernels in
``csrc/hybrid`` (``ops.hip_hybrid``).  Everything a recurrence touches is fp32 here too.

Sequence layout arguments shared by the per-sequence ops (``SeqLayout``): ``cu_q`` [B+1] rows
of each sequence inside the step (None: row b is sequence b, one token each), ``positions`` [T]
(a sequence's first row holds the position where this step starts it), ``slots`` [B] state slot
per sequence (negative: an unused row of a padded batch).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from .torch_ref import _gather_paged


def _bounds(cu_q, positions, B):
    if cu_q is None:
        rows = list(range(B + 1))
    else:
        rows = cu_q.tolist()
    return rows


# ------------------------------------------------------------------ embedding + norms
def embed_sum(ids, aux_rows, table, aux_table, scale=1.0):
    """fp32 rows ``(table[ids] + aux_table[aux_rows]) * scale`` (``aux_table`` None: the first alone)."""
    x = table[ids.long()].float()
    if aux_table is not None:
        x = x + aux_table[aux_rows.long()].float()
    return x * scale if scale != 1.0 else x


def offset_rms_norm(x, w, eps, out_dtype):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w.float())).to(out_dtype)


def post_norm_residual(y, wb, x, eps, w_next, out_dtype):
    """``x += norm(y) * (1 + wb)`` in place on the fp32 stream ``x``; with ``w_next`` also returns
    ``norm(x) * (1 + w_next)`` (the input of the next sublayer)."""
    yf = y.float()
    x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + wb.float()))
    if w_next is None:
        return None
    return offset_rms_norm(x, w_next, eps, out_dtype)


# ------------------------------------------------------------------ rotation, value mix, store
def pair_cos_sin_table(rot_dims: int, max_position: int, base: float, scaling) -> torch.Tensor:
    """[max_position, rot_dims] fp32: cos of the rot_dims/2 angles, then their sin.  The angle
    position * f_i is formed in fp32 (f_i rounded to fp32 first), its cos / sin in fp64."""
    import math
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / rot_dims)
    if scaling:
        factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        orig = float(scaling["original"])
        wl = 2 * math.pi / f
        s = (orig / wl - low) / (high - low)
        mid = (1 - s) * f / factor + s * f
        f = torch.where(wl < orig / high, f, torch.where(wl > orig / low, f / factor, mid))
    ang = torch.arange(max_position, dtype=torch.float32)[:, None] * f.float()[None, :]
    ang = ang.double()
    return torch.cat([ang.cos(), ang.sin()], -1).float()


def _rotate_pairs(x, cs, rot_dims):
    """x [T, heads, D] fp32, cs [T, rot_dims] -> rotated copy."""
    if rot_dims == 0:
        return x
    half = rot_dims // 2
    c, s = cs[:, None, :half], cs[:, None, half:]
    a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
    out = x.clone()
    out[..., 0:rot_dims:2] = a * c - b * s
    out[..., 1:rot_dims:2] = b * c + a * s
    return out


def pair_rope_mix_store(q, k, v, positions, cos_sin, rot_dims, v_first, lam, v_mode,
                        k_cache, v_cache, slot_mapping):
    """q [T,H,D], k [T,G,D], v [T,G,E] views of a projection output.  Rotates q in place and k
    on its way into the cache; ``v_mode`` 1: copies v into ``v_first``; 2: v <- (1 - lam) v +
    lam v_first (fp32); the result goes into the cache.  Rows with slot < 0 store nothing."""
    cs = cos_sin[positions.long()] if rot_dims else None
    q.copy_(_rotate_pairs(q.float(), cs, rot_dims).to(q.dtype))
    kr = _rotate_pairs(k.float(), cs, rot_dims)
    vf = v.float()
    if v_mode == 1:
        v_first.copy_(v.reshape(v_first.shape))
    elif v_mode == 2:
        lf = lam.float()
        vf = (1.0 - lf) * vf + lf * v_first.float().reshape(vf.shape)
    if k_cache is not None and slot_mapping is not None:
        bs = k_cache.shape[1]
        slots = slot_mapping.long()
        keep = slots >= 0
        blk, off = torch.div(slots[keep], bs, rounding_mode="floor"), slots[keep] % bs
        k_cache[blk, off] = kr[keep].to(k_cache.dtype)
        v_cache[blk, off] = vf[keep].to(v_cache.dtype)


# ------------------------------------------------------------------ attention with a sink
def _sink_attend(q, k, v, scale, sink, gate, offset, window=0, keep_first=0, slopes=None,
                 temps=None, softcap=0.0, pool=0, kp=None, vp=None):
    """q [Lq,H,D], k [Lk,G,D], v [Lk,G,E], gate [Lq,H] -> [Lq,H,E] fp32.  Query row i sits at
    position ``offset + i`` and sees key j <= its position; with ``window`` > 0 only keys with
    position - j < window or j < keep_first.  ``slopes`` [H]: slope_h * (position - j) is taken
    off the score.  ``sink`` None: an ordinary softmax.  ``temps`` [H]: the score of head h is
    multiplied by temps[h]; ``softcap`` > 0: score <- softcap tanh(score / softcap), after scale
    and temperature.  ``pool`` > 0 (with a window): ``kp`` [Nb,G,D] / ``vp`` [Nb,G,E] hold one key
    and value per block of ``pool`` tokens; block b joins the softmax of a query at position i
    when b pool + pool - 1 <= i - window."""
    Lq, H, _ = q.shape
    Lk, G, _ = k.shape
    r = H // G
    qf = q.float().transpose(0, 1)
    kf = k.float().transpose(0, 1).repeat_interleave(r, 0)
    vf = v.float().transpose(0, 1).repeat_interleave(r, 0)
    s = torch.matmul(qf, kf.transpose(1, 2)) * scale                  # [H, Lq, Lk]
    qi = torch.arange(Lq)[:, None] + offset
    kj = torch.arange(Lk)[None, :]
    dist = (qi - kj).float()
    if slopes is not None:
        s = s - slopes.float()[:, None, None] * dist[None]
    hidden = kj > qi
    if window:
        hidden = hidden | ((qi - kj >= window) & (kj >= keep_first))
    hidden = hidden.expand(Lq, Lk)
    if pool and window and kp is not None and kp.shape[0]:
        Nb = kp.shape[0]
        s = torch.cat([s, torch.matmul(qf, kp.float().transpose(0, 1).repeat_interleave(r, 0)
                                       .transpose(1, 2)) * scale], -1)
        vf = torch.cat([vf, vp.float().transpose(0, 1).repeat_interleave(r, 0)], 1)
        last = torch.arange(Nb)[None, :] * pool + pool - 1
        hidden = torch.cat([hidden, last > qi - window], -1)
    if temps is not None:
        s = s * temps.float()[:, None, None]
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    s = s.masked_fill(hidden[None], float("-inf"))
    n_keys = s.shape[-1]
    if sink is not None:
        s = torch.cat([s, sink.float()[:, None, None].expand(H, Lq, 1)], -1)
    p = torch.softmax(s, -1)[..., :n_keys]
    o = torch.matmul(p, vf).transpose(0, 1)                           # [Lq, H, E]
    if gate is not None:
        o = o * torch.sigmoid(gate.float())[:, :, None]
    return o


def _pooled(k_pool, v_pool, table, ctx, window, pool):
    """The pooled rows a sequence with ``ctx`` keys can see at its last position."""
    if not pool or not window or k_pool is None:
        return None, None
    nb = max(0, (ctx - window) // pool)
    if nb == 0:
        return None, None
    return _gather_paged(k_pool, table, nb), _gather_paged(v_pool, table, nb)


def sink_attention_prefill(q, k_cache, v_cache, cu_q, cu_k, block_tables, scale, sink, gate, out,
                           window=0, keep_first=0, slopes=None, temps=None, softcap=0.0, pool=0,
                           k_pool=None, v_pool=None):
    cq, ck = cu_q.tolist(), cu_k.tolist()
    for b in range(len(cq) - 1):
        s, e = cq[b], cq[b + 1]
        lk = ck[b + 1] - ck[b]
        if e == s:
            continue
        k = _gather_paged(k_cache, block_tables[b], lk)
        v = _gather_paged(v_cache, block_tables[b], lk)
        kp, vp = _pooled(k_pool, v_pool, block_tables[b], lk, window, pool)
        out[s:e] = _sink_attend(q[s:e], k, v, scale, sink, None if gate is None else gate[s:e],
                                lk - (e - s), window, keep_first, slopes, temps, softcap, pool,
                                kp, vp).to(out.dtype)
    return out


def sink_attention_decode(q, k_cache, v_cache, block_tables, context_lens, scale, sink, gate, out,
                          window=0, keep_first=0, slopes=None, temps=None, softcap=0.0, pool=0,
                          k_pool=None, v_pool=None):
    for b, L in enumerate(context_lens.tolist()):
        if L <= 0:
            continue
        k = _gather_paged(k_cache, block_tables[b], L)
        v = _gather_paged(v_cache, block_tables[b], L)
        kp, vp = _pooled(k_pool, v_pool, block_tables[b], L, window, pool)
        out[b:b + 1] = _sink_attend(q[b:b + 1], k, v, scale, sink,
                                    None if gate is None else gate[b:b + 1], L - 1, window,
                                    keep_first, slopes, temps, softcap, pool, kp, vp).to(out.dtype)
    return out


def unit_norm_store(q, k, eps, k_cache, v_cache, slot_mapping):
    """q [T,H,D], k [T,G,D] views of a projection output.  Every q head is divided by its root
    mean square in place; the cache row of a token receives the key before the norm as its VALUE
    and the key divided by its root mean square as its KEY (D = E).  Rows with slot < 0 store
    nothing."""
    qf, kf = q.float(), k.float()
    q.copy_((qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps)).to(q.dtype))
    kn = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps)
    if k_cache is not None and slot_mapping is not None:
        bs = k_cache.shape[1]
        slots = slot_mapping.long()
        keep = slots >= 0
        blk, off = torch.div(slots[keep], bs, rounding_mode="floor"), slots[keep] % bs
        k_cache[blk, off] = kn[keep].to(k_cache.dtype)
        v_cache[blk, off] = kf[keep].to(v_cache.dtype)


# ------------------------------------------------------------------ gated delta rule
def delta_prepare(q, k, v, b, a, conv_w, a_log, dt_bias, conv_state, cu_q, positions, slots,
                  conv_bias=None, ssd=False):
    """(``ssd``: the state-space form - the convolution has a bias ``conv_bias`` [C], q and k stay
    as convolved (no unit vectors, no D^-1/2), beta = softplus(a + dt_bias) is the step size and
    decay = exp(-exp(A_log) beta); ``b`` is not read.)
    Short causal convolution + silu on q / k / v (their last taps-1 inputs per sequence live
    in ``conv_state`` [slots, taps-1, Cq+Ck+Cv] fp32 and are replaced by this step's), unit
    vectors for q (times D^-1/2) and k, beta = sigmoid(b), decay = exp(-exp(A_log) softplus(a +
    dt_bias)).  q, k [T,G,D]; v [T,H,E]; b [T,H]; a and dt_bias [T,H] / [H] (a decay per head) or
    [T,H*D] / [H*D] (one per head and key channel).  Returns fp32 (q, k, v, beta, decay)."""
    T, G, D = q.shape
    H, E = v.shape[1], v.shape[2]
    x = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], -1).float()
    w = conv_w.float()                                                 # [C, taps]: q, k, v rows
    taps = w.shape[1]
    y = torch.empty_like(x)
    B = slots.shape[0]
    rows = _bounds(cu_q, positions, B)
    for i in range(B):
        s, e, slot = rows[i], rows[i + 1], int(slots[i])
        if e == s or slot < 0:
            continue
        if taps > 1:
            tail = conv_state[slot] if int(positions[s]) > 0 else torch.zeros_like(conv_state[slot])
            full = torch.cat([tail, x[s:e]], 0)
            conv_state[slot] = full[full.shape[0] - (taps - 1):]
        else:
            full = x[s:e]
        win = full.unfold(0, taps, 1)                                  # [n, C, taps]
        y[s:e] = (win * w[None]).sum(-1)
    if conv_bias is not None:
        y = y + conv_bias.float()
    y = F.silu(y)
    cq, ckk = G * D, 2 * G * D
    qn, kn, vv = y[:, :cq].view(T, G, D), y[:, cq:ckk].view(T, G, D), y[:, ckk:].view(T, H, E)
    sp = F.softplus(a.float() + dt_bias.float())
    if ssd:
        decay = torch.exp(-torch.exp(a_log.float()) * sp)
        return qn.contiguous(), kn.contiguous(), vv.contiguous(), sp, decay
    qn = qn * torch.rsqrt(qn.pow(2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kn = kn * torch.rsqrt(kn.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(b.float())
    if a.shape[-1] == H:                                                 # one decay per head
        decay = torch.exp(-torch.exp(a_log.float()) * sp)
    else:                                                                # one per head and key channel
        decay = torch.exp(-torch.exp(a_log.float())[None, :, None] * sp.view(T, H, D))
    return qn, kn, vv.contiguous(), beta, decay


def delta_scan(qn, kn, vv, beta, decay, state, cu_q, positions, slots, correct=True):
    """Per sequence and head, token after token: S <- decay S; u = beta (v - S^T k); S <- S + k
    u^T; o = S^T q (``correct`` False: u = beta v, the plain gated outer-product update).  ``state`` [slots, H, D, E] fp32 is read (zeros where the sequence starts at
    position 0) and left holding the state after the step.  ``decay`` [T,H] scales a head's whole
    state, [T,H,D] the rows that belong to key channels.  Returns o [T,H,E] fp32."""
    T, G, D = qn.shape
    H, E = vv.shape[1], vv.shape[2]
    r = H // G
    o = torch.zeros(T, H, E, dtype=torch.float32)
    B = slots.shape[0]
    rows = _bounds(cu_q, positions, B)
    qh, kh = qn.repeat_interleave(r, 1), kn.repeat_interleave(r, 1)
    for i in range(B):
        s, e, slot = rows[i], rows[i + 1], int(slots[i])
        if e == s or slot < 0:
            continue
        S = state[slot].clone() if int(positions[s]) > 0 else torch.zeros(H, D, E)
        for t in range(s, e):
            S = S * (decay[t][:, None, None] if decay.dim() == 2 else decay[t][:, :, None])
            u = beta[t][:, None] * ((vv[t] - torch.einsum("hde,hd->he", S, kh[t])) if correct else vv[t])
            S = S + kh[t][:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hde,hd->he", S, qh[t])
        state[slot] = S
    return o


def gated_head_norm(o, w, gate, eps, out_dtype, act="silu"):
    """o [T,H,E] fp32 / rms over E * w * act(gate [T,H,E]); w [E] (shared by the heads) or [H*E];
    act "silu" or "sigmoid"."""
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w.float().view(-1, o.shape[-1])
    gf = gate.float().reshape(o.shape)
    return (y * (F.silu(gf) if act == "silu" else torch.sigmoid(gf))).to(out_dtype)


# ------------------------------------------------------------------ grouped expert routing
def grouped_route(h, router_w, top, groups, keep, score="softmax", bias=None, gates=0):
    """Scores over all experts in fp32 (``score``: "softmax", or "sigmoid" of each logit); only experts of the ``keep`` groups (of ``groups``
    equal runs of neighbours) whose best score is largest are eligible; the ``top`` largest
    eligible scores, unnormalised, are the weights.  Returns [T, experts] fp32, zero elsewhere.
    ``bias`` [rows]: added to the logits.  ``score`` "chosen": the ``top`` largest LOGITS are
    chosen and their weights are the softmax over those alone (one group).  ``gates``: that many
    trailing rows of ``router_w`` are not experts but per-token gates: the result has as many
    trailing columns holding sigmoid(logit)."""
    z = h.float() @ router_w.float().t()
    if bias is not None:
        z = z + bias.float()
    extra = None
    if gates:
        extra = torch.sigmoid(z[:, z.shape[1] - gates:])
        z = z[:, :z.shape[1] - gates]
    if score == "chosen":
        assert groups == 1 and keep == 1
        ids = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
        dense = torch.zeros_like(z)
        dense.scatter_(1, ids, torch.softmax(z.gather(1, ids), -1))
        return dense if extra is None else torch.cat([dense, extra], 1)
    assert not gates
    s = torch.softmax(z, -1) if score == "softmax" else torch.sigmoid(z)
    T, E = s.shape
    per = E // groups
    best = s.view(T, groups, per).max(-1).values
    # ties go to the lower index, as in the kernel: rank by (score desc, index asc)
    kept = torch.zeros(T, groups, dtype=torch.bool)
    kept.scatter_(1, torch.sort(best, dim=-1, descending=True, stable=True).indices[:, :keep], True)
    masked = torch.where(kept.repeat_interleave(per, 1), s, torch.full_like(s, -1.0))
    ids = torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :top]
    dense = torch.zeros_like(s)
    dense.scatter_(1, ids, s.gather(1, ids))
    return dense


def gelu_route_scale(up, dense, ff, out_dtype):
    """up [T, experts*ff] -> gelu(up) * dense[t, expert] (exact erf gelu, fp32 math)."""
    T = up.shape[0]
    y = F.gelu(up.float()).view(T, -1, ff) * dense[:, :, None]
    return y.view(T, -1).to(out_dtype)


def swiglu_route_scale(gu, dense, ff, shared_ff, out_dtype):
    """gu [T, 2 C], C = experts * ff + shared_ff: the gate projections of all experts (and of a
    shared one behind them), then their up projections.  Column c of expert j gets
    silu(w g_c) * (w u_c) with w = dense[t, j] - the routing weight scales the expert's INPUT, and
    the projections are linear, so it is applied to their outputs; exactly zero where w is.
    Shared columns have w = 1.  ``dense`` None: no routed experts.  Returns [T, C]."""
    T, C = gu.shape[0], gu.shape[1] // 2
    g, u = gu[:, :C].float(), gu[:, C:].float()
    if dense is not None:
        w = torch.cat([dense.float().repeat_interleave(ff, 1),
                       torch.ones(T, shared_ff, dtype=torch.float32)], 1)
        g, u = g * w, u * w
    return (F.silu(g) * u).to(out_dtype)


# ------------------------------------------------------------------ positions, grouped norms
def embed_sinusoid(ids, positions, table, inv_freq):
    """fp32 rows ``table[ids]`` + the position vector whose entry 2i is sin(p f_i) and entry
    2i+1 cos(p f_i); the angle is the fp32 product of the position and ``inv_freq`` [W/2]."""
    x = table[ids.long()].float()
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    x[:, 0::2] += torch.sin(ang.double()).float()
    x[:, 1::2] += torch.cos(ang.double()).float()
    return x


def group_rms_norm(x, w, groups, eps, out_dtype):
    """The row is cut into ``groups`` equal consecutive parts, each divided by its own root mean
    square; the whole times w."""
    xf = x.float()
    parts = xf.view(xf.shape[0], groups, -1)
    y = parts * torch.rsqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
    return (y.view(xf.shape) * w.float()).to(out_dtype)


def residual_group_norm(x, ys, w_next, groups, eps, out_dtype):
    """``x += sum(ys)`` in place on the fp32 stream; with ``w_next`` also returns the grouped norm
    of the new x (the next layer's input)."""
    for y in ys:
        x.add_(y.float())
    if w_next is None:
        return None
    return group_rms_norm(x, w_next, groups, eps, out_dtype)


def add_normed_mean(x, parts, eps):
    """``x += mean_i(y_i / rms(y_i) * w_i)`` in place on the fp32 stream; ``parts`` = [(y, w), ...]."""
    acc = torch.zeros_like(x)
    for y, w in parts:
        yf = y.float()
        acc += yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    x.add_(acc / len(parts))


def tanh_cap_(z, cap):
    """z <- cap tanh(z / cap) in place (fp32 math)."""
    z.copy_((cap * torch.tanh(z.float() / cap)).to(z.dtype))
    return z


# ------------------------------------------------------------------ gated outer-product recurrences
def _seq_rows(cu_q, positions, slots):
    B = slots.shape[0]
    rows = _bounds(cu_q, positions, B)
    for i in range(B):
        s, e, slot = rows[i], rows[i + 1], int(slots[i])
        if e > s and slot >= 0:
            yield s, e, slot, int(positions[s]) > 0


def mlstm_scan(q, k, v, i_raw, f_raw, i_bias, f_bias, cap, state, norm_state, max_state,
               cu_q, positions, slots):
    """Matrix memory with exponential gating and a running maximum m (it starts at 0):
    i = cap tanh((i_raw + b_i) / cap), f = logsigmoid(cap tanh((f_raw + b_f) / cap)),
    m' = max(f + m, i); S <- e^(f+m-m') S + e^(i-m') k v^T; n likewise with k alone;
    o = S^T q / (max(|n . q|, e^(-m')) + 1e-6), q scaled by D^-1/2.  q, k [T,H,D]; v [T,H,E];
    gates [T,H]; ``state`` [slots,H,D,E] fp32; ``norm_state`` [slots,H,Z,D] and ``max_state``
    [slots,H,Z] fp32 hold Z = ceil(E/16) identical copies of n and m (the GPU kernel's workgroups,
    one per block of columns, each read and write their own).  Returns o [T,H,E] fp32."""
    T, H, D = q.shape
    E = v.shape[2]
    qf, kf, vf = q.float() * D ** -0.5, k.float(), v.float()
    ig = cap * torch.tanh((i_raw.float() + i_bias.float()) / cap)
    fg = F.logsigmoid(cap * torch.tanh((f_raw.float() + f_bias.float()) / cap))
    o = torch.zeros(T, H, E, dtype=torch.float32)
    for s, e, slot, past in _seq_rows(cu_q, positions, slots):
        S = state[slot].clone() if past else torch.zeros(H, D, E)
        n = norm_state[slot][:, 0].clone() if past else torch.zeros(H, D)
        m = max_state[slot][:, 0].clone() if past else torch.zeros(H)
        for t in range(s, e):
            m2 = torch.maximum(fg[t] + m, ig[t])
            a, b = torch.exp(fg[t] + m - m2), torch.exp(ig[t] - m2)
            S = a[:, None, None] * S + (b[:, None] * kf[t])[:, :, None] * vf[t][:, None, :]
            n = a[:, None] * n + b[:, None] * kf[t]
            m = m2
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            o[t] = torch.einsum("hde,hd->he", S, qf[t]) / den[:, None]
        state[slot] = S
        norm_state[slot] = n[:, None, :]
        max_state[slot] = m[:, None]
    return o


def gla_scan(q, k, v, a_raw, a_bias, tau, state, cu_q, positions, slots):
    """S <- diag(alpha) S + k v^T; o = S^T q with alpha = sigmoid(a_raw + a_bias)^(1/tau) per key
    channel (rows of S) and q scaled by D^-1/2.  q, k, a_raw [T,H,D]; v [T,H,E]; ``state``
    [slots,H,D,E] fp32.  Returns o [T,H,E] fp32."""
    T, H, D = q.shape
    E = v.shape[2]
    qf, kf, vf = q.float() * D ** -0.5, k.float(), v.float()
    alpha = torch.exp(F.logsigmoid(a_raw.float().reshape(T, H, D) + a_bias.float().view(H, D)) / tau)
    o = torch.zeros(T, H, E, dtype=torch.float32)
    for s, e, slot, past in _seq_rows(cu_q, positions, slots):
        S = state[slot].clone() if past else torch.zeros(H, D, E)
        for t in range(s, e):
            S = alpha[t][:, :, None] * S + kf[t][:, :, None] * vf[t][:, None, :]
            o[t] = torch.einsum("hde,hd->he", S, qf[t])
        state[slot] = S
    return o


# ------------------------------------------------------------------ scaled branches, latent keys
def rms_norm_rows(x, w, eps, out_dtype):
    """x [T, n] (rows may be strided, any activation type) / rms * w [n] (fp32 math)."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def residual_sum_norm(x, ys, scales, gain, eps, out_dtype):
    """``x += sum_i scales[i] * ys[i]`` in place on the fp32 stream; with ``gain`` (one number for
    all coordinates) also returns x / rms(x) * gain, the next layer's input."""
    for y, s in zip(ys, scales):
        x.add_(y.float() * float(s))
    if gain is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * float(gain)).to(out_dtype)


def _scatter_rows(cache, rows, slot_mapping):
    bs = cache.shape[1]
    slots = slot_mapping.long()
    keep = slots >= 0
    blk, off = torch.div(slots[keep], bs, rounding_mode="floor"), slots[keep] % bs
    cache[blk, off] = rows[keep].to(cache.dtype)


def row_norm_store(q, k, v, qw, kw, eps, k_cache, v_cache, slot_mapping):
    """q [T,H,D], k [T,G,D], v [T,G,E] views of a projection output.  With ``qw`` [H*D] / ``kw``
    [G*D]: the whole q row (all heads at once) is divided by its root mean square and multiplied
    by qw, in place; the k row likewise with kw on its way into the cache.  Without: k goes in as
    it is.  v always does.  Rows with slot < 0 store nothing."""
    T = q.shape[0]
    kf = k.float()
    if qw is not None:
        q.copy_(rms_norm_rows(q.reshape(T, -1), qw, eps, q.dtype).view(q.shape))
        kf = rms_norm_rows(k.reshape(T, -1), kw, eps, torch.float32).view(k.shape)
    if k_cache is not None and slot_mapping is not None:
        _scatter_rows(k_cache, kf, slot_mapping)
        _scatter_rows(v_cache, v.float(), slot_mapping)


def _rotate_half(x, positions, inv_freq, dims):
    """x [T, ..., n] fp32: entry i < dims/2 is paired with entry i + dims/2 and the pair turned by
    the fp32 angle position * inv_freq[i]; entries from ``dims`` on pass unchanged."""
    if dims == 0:
        return x
    half = dims // 2
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang.double()).float().view(shape), torch.sin(ang.double()).float().view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def latent_rope_store(q_abs, q, dkv, w, eps, positions, inv_freq, rot_dims, k_cache, v_cache,
                      slot_mapping):
    """Assembles the queries and cache rows of attention over a shared latent.  ``q_abs`` [H,T,R]:
    the heads' unrotated query parts carried into the latent's coordinates; ``q`` [T,H,D+P] whose
    last P entries per head are the part to rotate; ``dkv`` [T,R+P]: the raw latent and one key
    part shared by all heads.  K cache row = [rmsnorm(latent) * w | rotated key part] (one KV
    head of R + P), V cache row = the normed latent (R; ``v_cache`` None: not written, the reader
    takes the leading R entries of the key rows).  Returns the queries [T,H,R+P] =
    [q_abs | rotated part].  The rotation turns the first ``rot_dims`` of the P entries."""
    H, T, R = q_abs.shape
    P = dkv.shape[1] - R
    D = q.shape[2] - P
    c = rms_norm_rows(dkv[:, :R], w, eps, torch.float32)
    kr = _rotate_half(dkv[:, R:].float(), positions, inv_freq, rot_dims)
    qr = _rotate_half(q[:, :, D:].float(), positions, inv_freq, rot_dims)
    out = torch.cat([q_abs.transpose(0, 1).float(), qr], -1).to(q.dtype)
    if k_cache is not None and slot_mapping is not None:
        _scatter_rows(k_cache, torch.cat([c, kr], -1)[:, None, :], slot_mapping)
        if v_cache is not None:          # None: the values are the leading part of the key rows
            _scatter_rows(v_cache, c[:, None, :], slot_mapping)
    return out


def xielu(u, ap, aq, out_dtype):
    """ap z^2 + z/2 for z > 0, aq (e^z - 1 - z) + z/2 otherwise (fp32 math); u may be a strided
    column block.  Returns a contiguous tensor."""
    z = u.float()
    neg = torch.clamp(z, max=0.0)
    return torch.where(z > 0, ap * z * z + 0.5 * z, aq * (torch.expm1(neg) - neg) + 0.5 * z).to(out_dtype)


def gated_group_norm(o, skip_x, skip_w, z, w, groups, eps, out_dtype):
    """y = (o + skip_w[h] * skip_x) * silu(z) over [T, H*E]; then y is cut into ``groups`` equal
    consecutive parts, each divided by its own root mean square, times w [H*E].  o, skip_x
    [T,H,E] fp32; skip_w [H]; z [T, H*E] (strided)."""
    T, H, E = o.shape
    y = (o + skip_w.float()[None, :, None] * skip_x).view(T, H * E) * F.silu(z.float())
    parts = y.view(T, groups, -1)
    y = (parts * torch.rsqrt(parts.pow(2).mean(-1, keepdim=True) + eps)).view(T, H * E)
    return (y * w.float()).to(out_dtype)


def sigmoid_gate(o, gate, out_dtype):
    """o [T,H,E] (any strides) * sigmoid(gate [T, H*E]) element by element -> contiguous [T, H*E]."""
    T = o.shape[0]
    return (o.float().reshape(T, -1) * torch.sigmoid(gate.float())).to(out_dtype)


# ------------------------------------------------------------------ rotated values, pooled blocks
def half_rope_store(q, k, v, positions, inv_freq, rot_dims, v_inv_freq, k_cache, v_cache,
                    slot_mapping):
    """q [T,H,D], k [T,G,D], v [T,G,E] views of a projection output.  The first ``rot_dims``
    entries of every q and k head are turned in half-split pairs (entry i with entry i +
    rot_dims/2) by position * inv_freq[i], q in place and k on its way into the cache.  With
    ``v_inv_freq`` [E/2] the value heads are turned the same way over ALL their entries (entry m
    with entry m + E/2 by position * v_inv_freq[m]) before they are cached; None: cached as they
    are.  Rows with slot < 0 store nothing."""
    q.copy_(_rotate_half(q.float(), positions, inv_freq, rot_dims).to(q.dtype))
    kr = _rotate_half(k.float(), positions, inv_freq, rot_dims)
    vf = v.float()
    if v_inv_freq is not None:
        vf = _rotate_half(vf, positions, v_inv_freq, v.shape[-1])
    if k_cache is not None and slot_mapping is not None:
        _scatter_rows(k_cache, kr, slot_mapping)
        _scatter_rows(v_cache, vf, slot_mapping)


def pool_block_means(k_cache, v_cache, k_pool, v_pool, pool, positions, block_tables, row_seq,
                     slot_mapping):
    """For every row of the step whose position ends a block of ``pool`` tokens (position + 1 a
    multiple of ``pool``): the means of that block's ``pool`` cached key rows and value rows
    (fp32 sums) are written to the pooled caches.  Block b of a sequence lives in row b %
    rows_per_page of page block_table[b // rows_per_page] of ``k_pool`` / ``v_pool``
    [pages, rows_per_page, G, D|E], rows_per_page * pool >= the token page size.  ``row_seq`` [T]:
    the sequence (block table row) of each row, negative for rows of no sequence; None: row t is
    sequence t.  Rows whose ``slot_mapping`` entry is negative (they cache nothing) are passed over."""
    bs, pr = k_cache.shape[1], k_pool.shape[1]
    pos = positions.tolist()
    seq = row_seq.tolist() if row_seq is not None else list(range(len(pos)))
    stored = slot_mapping.tolist()
    for t, p in enumerate(pos[:len(seq)]):
        b = seq[t]
        if b < 0 or stored[t] < 0 or b >= block_tables.shape[0] or (p + 1) % pool:
            continue
        table = block_tables[b]
        blk = p // pool
        js = torch.arange(blk * pool, blk * pool + pool)
        pages, offs = table[(js // bs)].long(), js % bs
        page, row = int(table[blk // pr]), blk % pr
        k_pool[page, row] = k_cache[pages, offs].float().mean(0).to(k_pool.dtype)
        v_pool[page, row] = v_cache[pages, offs].float().mean(0).to(v_pool.dtype)


def unturn_gate(o, positions, v_inv_freq, gate, out_dtype):
    """o [T,H,E]: every head turned back by its row's position (half-split pairs over all E
    entries, angles -position * v_inv_freq[m]; None: no turn), then times sigmoid(gate [T, H*E])
    element by element (None: no gate) -> contiguous [T, H*E]."""
    T = o.shape[0]
    of = o.float()
    if v_inv_freq is not None:
        of = _rotate_half(of, -positions, v_inv_freq, o.shape[-1])
    of = of.reshape(T, -1)
    if gate is not None:
        of = of * torch.sigmoid(gate.float())
    return of.to(out_dtype)


# ------------------------------------------------------------------ gated diagonal recurrence
def short_conv(x, w, bias, conv_state, cu_q, positions, slots):
    """Causal convolution per channel without an activation: x [T, C] (rows may be strided),
    w [C, taps] fp32 whose LAST column meets the current token, bias [C] or None.  A sequence's
    last taps-1 inputs live in ``conv_state`` [slots, taps-1, C] fp32 (zeros where it starts at
    position 0) and are replaced by this step's.  Returns fp32 [T, C]."""
    xf = x.float()
    wf = w.float()
    taps = wf.shape[1]
    y = torch.zeros_like(xf)
    for s, e, slot, past in _seq_rows(cu_q, positions, slots):
        if taps > 1:
            tail = conv_state[slot] if past else torch.zeros_like(conv_state[slot])
            full = torch.cat([tail, xf[s:e]], 0)
            conv_state[slot] = full[full.shape[0] - (taps - 1):]
        else:
            full = xf[s:e]
        y[s:e] = (full.unfold(0, taps, 1) * wf[None]).sum(-1)
    if bias is not None:
        y = y + bias.float()
    return y


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))


def rglru_scan(u, gates, gate_bias, lam, y, state, cu_q, positions, slots, sharp, out_dtype):
    """Real-gated diagonal recurrence.  u [T, C] fp32; ``gates`` [nb, T, 2c] fp32, C = nb c: for
    block k of channels the pre-activations of the recurrence gate (first c) and of the input
    gate (last c), ``gate_bias`` [nb, 2c] still to be added; lam [C];
        r, i = sigmoid(.);  d = exp(-sharp r softplus(lam));  S <- d S + sqrt(1 - d^2) i u
    from S = 0 where a sequence starts (``state`` [slots, C] fp32 otherwise, left holding the state
    after the step).  Returns S * gelu_tanh(y) [T, C] in ``out_dtype`` (y [T, C]: the other
    branch's pre-activation, rows may be strided)."""
    T, C = u.shape
    nb = gates.shape[0]
    c = C // nb
    g = torch.sigmoid(gates.float() + gate_bias.float()[:, None, :])          # [nb, T, 2c]
    r = g[:, :, :c].permute(1, 0, 2).reshape(T, C)
    i = g[:, :, c:].permute(1, 0, 2).reshape(T, C)
    la = -sharp * r * F.softplus(lam.float())                 # log of the decay
    d = torch.exp(la)
    add = torch.sqrt(-torch.expm1(2.0 * la)) * i * u          # sqrt(1 - d^2), exact next to d = 1
    out = torch.zeros(T, C, dtype=torch.float32)
    for s, e, slot, past in _seq_rows(cu_q, positions, slots):
        S = state[slot].clone() if past else torch.zeros(C)
        for t in range(s, e):
            S = d[t] * S + add[t]
            out[t] = S
        state[slot] = S
    return (out * gelu_tanh(y.float())).to(out_dtype)


def capped_glu_route_scale(gu, dense, ff, shared_ff, limit, shared_limit, out_dtype, slope=1.702):
    """gu [T, 2 C], C = experts * ff + shared_ff: the gate projections of all experts (and of a
    shared one behind them), then their up projections.  Column c: g = min(gate, L), u =
    clamp(up, -L, L), act = w g sigmoid(slope g) (u + 1) with L = ``limit`` for routed columns and
    ``shared_limit`` for shared ones, w = dense[t, expert] for routed columns (exactly zero where w
    is) and, for shared columns, dense[t, experts] when ``dense`` has that extra column (a
    per-token gate of the shared expert), else 1.  Returns [T, C]."""
    T, C = gu.shape[0], gu.shape[1] // 2
    ne = (C - shared_ff) // ff if ff else 0
    g, u = gu[:, :C].float(), gu[:, C:2 * C].float()
    lim = torch.cat([torch.full((ne * ff,), float(limit)), torch.full((shared_ff,), float(shared_limit))])
    g = torch.minimum(g, lim)
    u = torch.maximum(torch.minimum(u, lim), -lim)
    act = g * torch.sigmoid(slope * g) * (u + 1.0)
    sg = dense[:, ne:ne + 1].float() if dense.shape[1] > ne else torch.ones(T, 1)
    w = torch.cat([dense[:, :ne].float().repeat_interleave(ff, 1), sg.expand(T, shared_ff)], 1)
    return torch.where(w != 0, act * w, torch.zeros_like(act)).to(out_dtype)
