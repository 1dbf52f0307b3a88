"""The ops that the Kidupel family adds, one mechanism at a time.  On the CPU: the plain PyTorch
forms (``ops.torch_seqmix``, what the engine's CPU mode runs) against the float64 oracle's
function of the same mechanism.  On the GPU (``gpu`` tests): the gfx950 kernels
(``ops.hip_hybrid``) against those PyTorch forms on copies of the same inputs, in bfloat16 and
float32, with sizes that are not powers of two, strided inputs, several sequences per step with
unused rows, and state carried from one call to the next."""
import math

import pytest
import torch

import kidupel_oracle as oracle
from minivllm_amd.ops import torch_seqmix as ref

gpu = torch.cuda.is_available()
if gpu:
    from minivllm_amd.ops import hip_hybrid as hk

DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def tol(dt, f32=2e-5):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=f32, atol=f32)


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


# ------------------------------------------------------------------ CPU forms against the oracle
def test_xielu_both_branches_and_the_joint():
    z = torch.tensor([-30.0, -3.0, -1e-3, 0.0, 1e-3, 0.7, 5.0])
    for p, q in ((0.3, -0.8), (-2.0, 1.5), (0.0, 0.0)):
        sp = torch.nn.functional.softplus(torch.tensor([p, q], dtype=F64))
        got = ref.xielu(z, float(sp[0]), float(0.5 + sp[1]), torch.float32)
        torch.testing.assert_close(got.double(), oracle.xielu(z.double(), p, q), rtol=1e-6, atol=1e-6)
    assert float(ref.xielu(torch.zeros(1), 1.0, 1.0, torch.float32)) == 0.0


def test_single_gain_norm_and_scaled_branches():
    torch.manual_seed(1)
    x = torch.randn(5, 24)
    ys = [torch.randn(5, 24) for _ in range(3)]
    want = x.double() + 1.2 * ys[0].double() + 0.7 * ys[1].double() + ys[2].double()
    x2 = x.clone()
    h = ref.residual_sum_norm(x2, ys, [1.2, 0.7, 1.0], 1.5, 1e-5, torch.float32)
    torch.testing.assert_close(x2.double(), want, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(h.double(), oracle.scalar_norm(want, 1.5, 1e-5), rtol=1e-5, atol=1e-5)
    big = torch.full((1, 8), 1e-4)                      # eps inside the root matters here
    got = ref.residual_sum_norm(big.clone(), [], [], 2.0, 1e-6, torch.float32)
    torch.testing.assert_close(got.double(), oracle.scalar_norm(big.double(), 2.0, 1e-6), rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("dims,P", [(8, 8), (4, 10), (0, 6)])
def test_half_rotation_pairs_and_angles(dims, P):
    torch.manual_seed(2)
    T, H, D, R = 6, 2, 3, 5
    base = 50.0
    pos = torch.tensor([0, 1, 7, 300, 4095, 12], dtype=torch.int32)
    inv = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64).float()
    q = torch.randn(T, H, D + P)
    dkv = torch.randn(T, R + P)
    q_abs = torch.randn(H, T, R)
    w = 1 + 0.1 * torch.randn(R)
    kc, vc = torch.zeros(2, 4, 1, R + P), torch.zeros(2, 4, 1, R)
    slots = torch.tensor([0, 1, 2, 3, -1, 7], dtype=torch.int32)
    out = ref.latent_rope_store(q_abs, q, dkv, w, 1e-5, pos, inv, dims, kc, vc, slots)
    for t in range(T):
        p = int(pos[t])
        if dims:
            for hh in range(H):
                want = oracle.rotate_half(q[t, hh, D:D + dims].double(), p, dims, base)
                torch.testing.assert_close(out[t, hh, R:R + dims].double(), want, rtol=1e-4, atol=2e-4)
        torch.testing.assert_close(out[t, :, R + dims:], q[t, :, D + dims:])
        torch.testing.assert_close(out[t, :, :R], q_abs[:, t])
        s = int(slots[t])
        if s >= 0:
            c = oracle.rms(dkv[t, :R].double(), 1e-5) * w.double()
            torch.testing.assert_close(vc[s // 4, s % 4, 0].double(), c, rtol=1e-5, atol=1e-5)
            torch.testing.assert_close(kc[s // 4, s % 4, 0, :R].double(), c, rtol=1e-5, atol=1e-5)
            if dims:
                want = oracle.rotate_half(dkv[t, R:R + dims].double(), p, dims, base)
                torch.testing.assert_close(kc[s // 4, s % 4, 0, R:R + dims].double(), want, rtol=1e-4, atol=2e-4)
    assert float(kc[1, 0].abs().max()) == 0.0            # the row with slot -1 wrote nothing


def test_state_space_ops_follow_the_recurrence():
    """conv + bias + silu, step size, decay, the update without a correction term, skip, gate
    before the grouped norm: the three ops chained as the layer chains them, against the
    oracle's token-by-token form; then the same tokens in two portions through the slot."""
    torch.manual_seed(3)
    T, H, G, N, E, taps, parts, W = 11, 4, 2, 6, 5, 3, 2, 16
    m = {"heads": H, "vdim": E, "state": N, "groups": G, "conv": taps, "norm_groups": parts}
    inner, gn = H * E, G * N
    p = {"in": torch.randn(2 * inner + 2 * gn + H, W) * W ** -0.5, "conv": 0.5 * torch.randn(inner + 2 * gn, taps),
         "conv.b": 0.3 * torch.randn(inner + 2 * gn), "dt_bias": torch.randn(H), "A_log": -1 + 0.5 * torch.randn(H),
         "D": torch.randn(H), "norm": 1 + 0.1 * torch.randn(inner), "o": torch.eye(inner)}
    h = torch.randn(T, W)
    want = oracle.state_space_duality(h.double(), p, m, 1e-5)
    z, x, B, C, dt = (h @ p["in"].t()).split([inner, inner, gn, gn, H], 1)
    proj = torch.cat([C, B, x, z, dt], 1)
    cw = torch.cat([p["conv"].split([inner, gn, gn], 0)[i] for i in (2, 1, 0)], 0)
    cb = torch.cat([p["conv.b"].split([inner, gn, gn], 0)[i] for i in (2, 1, 0)], 0)

    def run(rows, first, state, tail):
        pr = proj[rows]
        n = pr.shape[0]
        lay = (torch.tensor([0, n], dtype=torch.int32), torch.full((n,), first, dtype=torch.int32),
               torch.tensor([1], dtype=torch.int32))
        qn, kn, vv, step, decay = ref.delta_prepare(
            pr[:, :gn].view(n, G, N), pr[:, gn:2 * gn].view(n, G, N), pr[:, 2 * gn:2 * gn + inner].view(n, H, E),
            None, pr[:, 2 * gn + 2 * inner:], cw, p["A_log"], p["dt_bias"], tail, *lay, conv_bias=cb, ssd=True)
        o = ref.delta_scan(qn, kn, vv, step, decay, state, *lay, correct=False)
        return ref.gated_group_norm(o, vv, p["D"], pr[:, 2 * gn + inner:2 * gn + 2 * inner], p["norm"], parts,
                                    1e-5, torch.float32)
    state, tail = torch.full((2, H, N, E), 9.0), torch.full((2, taps - 1, inner + 2 * gn), 9.0)
    torch.testing.assert_close(run(slice(0, T), 0, state, tail).double(), want, rtol=1e-4, atol=1e-4)
    a = run(slice(0, 4), 0, state, tail)
    b = run(slice(4, 5), 4, state, tail)                  # one token: shorter than the convolution
    c = run(slice(5, T), 5, state, tail)
    torch.testing.assert_close(torch.cat([a, b, c]).double(), want, rtol=1e-4, atol=1e-4)


def test_whole_projection_norm_is_not_a_per_head_norm():
    torch.manual_seed(4)
    T, H, G, D, E = 3, 2, 1, 4, 3
    q, k, v = torch.randn(T, H, D), torch.randn(T, G, D), torch.randn(T, G, E)
    q[:, 0] *= 10                                        # one head dominates the projection's rms
    qw, kw = 1 + 0.1 * torch.randn(H * D), 1 + 0.1 * torch.randn(G * D)
    kc, vc = torch.zeros(1, 4, G, D), torch.zeros(1, 4, G, E)
    want = oracle.rms(q.reshape(T, -1).double(), 1e-6) * qw.double()
    q2 = q.clone()
    ref.row_norm_store(q2, k, v, qw, kw, 1e-6, kc, vc, torch.tensor([2, 0, 1], dtype=torch.int32))
    torch.testing.assert_close(q2.reshape(T, -1).double(), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(kc[0, 2].reshape(-1).double(), oracle.rms(k[0].reshape(-1).double(), 1e-6) * kw.double(),
                               rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(vc[0, 1], v[2])


# ------------------------------------------------------------------ kernels against the CPU forms
@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [24, 200, 2048, 5000])
def test_kernel_residual_sum_norm(dt, W):
    torch.manual_seed(0)
    T = 19
    x = torch.randn(T, W)
    wide = torch.randn(T, 4 * W).to(dt)
    ys = [wide[:, :W], wide[:, 2 * W:3 * W], wide[:, 3 * W:]]
    for n, gain in ((3, 1.3), (2, None), (0, 0.6), (1, 1.0)):
        x2, xg = x.clone(), x.cuda()
        sc = [1.2, 0.7, 1.0][:n]
        h = ref.residual_sum_norm(x2, ys[:n], sc, gain, 1e-5, dt)
        wg = wide.cuda()
        hg = hk.residual_sum_norm(xg, [wg[:, :W], wg[:, 2 * W:3 * W], wg[:, 3 * W:]][:n], sc, gain, 1e-5, dt)
        torch.testing.assert_close(xg.cpu(), x2, rtol=1e-6, atol=1e-6)
        if gain is None:
            assert hg is None
        else:
            torch.testing.assert_close(hg.cpu().float(), h.float(), **tol(dt))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES)
def test_kernel_rows_norm_xielu_gate(dt):
    torch.manual_seed(1)
    T, n = 23, 150
    wide = torch.randn(T, 3 * n).to(dt)
    w = 1 + 0.2 * torch.randn(n)
    torch.testing.assert_close(hk.rms_norm_rows(wide.cuda()[:, n:2 * n], w.cuda(), 1e-5, dt).cpu().float(),
                               ref.rms_norm_rows(wide[:, n:2 * n], w, 1e-5, dt).float(), **tol(dt))
    u = (3 * wide)[:, n:2 * n + 7]
    torch.testing.assert_close(hk.xielu((3 * wide).cuda()[:, n:2 * n + 7], 0.8, 1.1, dt).cpu().float(),
                               ref.xielu(u, 0.8, 1.1, dt).float(), **tol(dt))
    H, E = 5, 30
    o = torch.randn(H, T, E).to(dt)
    og = o.cuda().transpose(0, 1)                       # head-major, as the batched product leaves it
    torch.testing.assert_close(hk.sigmoid_gate(og, wide.cuda()[:, :H * E], dt).cpu().float(),
                               ref.sigmoid_gate(o.transpose(0, 1), wide[:, :H * E], dt).float(), **tol(dt))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("normed", [True, False])
def test_kernel_row_norm_store(dt, normed):
    torch.manual_seed(2)
    T, H, G, D, E, bs = 9, 6, 3, 20, 12, 4
    proj = torch.randn(T, H * D + G * D + G * E + 5).to(dt)
    qw, kw = (1 + 0.2 * torch.randn(H * D), 1 + 0.2 * torch.randn(G * D)) if normed else (None, None)
    slots = torch.tensor([3, 2, -1, 0, 11, 10, 9, 8, 1], dtype=torch.int32)

    def views(p):
        q, k, v = p[:, :H * D + G * D + G * E].split([H * D, G * D, G * E], 1)
        return q.view(T, H, D), k.view(T, G, D), v.view(T, G, E)
    pc, pg = proj.clone(), proj.cuda()
    kc, vc = torch.zeros(3, bs, G, D, dtype=dt), torch.zeros(3, bs, G, E, dtype=dt)
    kg, vg = kc.cuda(), vc.cuda()
    ref.row_norm_store(*views(pc), qw, kw, 1e-5, kc, vc, slots)
    hk.row_norm_store(*views(pg), *dev(qw, kw), 1e-5, kg, vg, slots.cuda())
    torch.testing.assert_close(pg.cpu().float(), pc.float(), **tol(dt))
    torch.testing.assert_close(kg.cpu().float(), kc.float(), **tol(dt))
    torch.testing.assert_close(vg.cpu().float(), vc.float(), **tol(dt))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("dims,P,R", [(8, 8, 20), (6, 10, 64), (64, 64, 128), (0, 4, 6)])
def test_kernel_latent_rope_store(dt, dims, P, R):
    torch.manual_seed(3)
    T, H, D, bs = 13, 3, 10, 4
    pos = torch.randint(0, 100000, (T,), dtype=torch.int32)
    pos[0] = 0
    inv = torch.tensor([1e4 ** (-2.0 * i / max(dims, 1)) for i in range(dims // 2)], dtype=F64).float()
    wide = torch.randn(T, H * (D + P) + R + P + 3).to(dt)
    q_abs = torch.randn(H, T, R).to(dt)
    w = 1 + 0.1 * torch.randn(R)
    slots = torch.randperm(16)[:T].to(torch.int32)
    slots[5] = -1

    def args(t):
        return t[:, :H * (D + P)].view(T, H, D + P), t[:, H * (D + P):H * (D + P) + R + P]
    kc, vc = torch.zeros(4, bs, 1, R + P, dtype=dt), torch.zeros(4, bs, 1, R, dtype=dt)
    kg, vg = kc.cuda(), vc.cuda()
    out = ref.latent_rope_store(q_abs, *args(wide), w, 1e-5, pos, inv, dims, kc, vc, slots)
    outg = hk.latent_rope_store(q_abs.cuda(), *args(wide.cuda()), w.cuda(), 1e-5, pos.cuda(), inv.cuda(),
                                dims, kg, vg, slots.cuda())
    # angles up to 1e5 rad: the fp32 product position * frequency is the same on both sides, the
    # sine / cosine of it may differ in the last bits
    t2 = dict(rtol=2e-2, atol=3e-2) if dt == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(outg.cpu().float(), out.float(), **t2)
    torch.testing.assert_close(kg.cpu().float(), kc.float(), **t2)
    torch.testing.assert_close(vg.cpu().float(), vc.float(), **t2)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,N,E,taps,parts", [(4, 2, 6, 5, 3, 2), (8, 1, 64, 64, 4, 1), (6, 2, 32, 32, 4, 2),
                                                (3, 3, 136, 24, 1, 3), (2, 1, 16, 72, 7, 4)])
def test_kernel_state_space_chain(dt, H, G, N, E, taps, parts):
    """Three sequences in one step (one of them an unused row set), then a second step that
    continues two of them with one token and a short portion: prepare, scan and gated norm on
    both sides, states and tails carried in their slots."""
    torch.manual_seed(4)
    inner, gn = H * E, G * N
    C = inner + 2 * gn
    cw, cb = 0.5 * torch.randn(C, taps), 0.3 * torch.randn(C)
    a_log, dtb, skip = -1 + 0.5 * torch.randn(H), torch.randn(H), torch.randn(H)
    nw = 1 + 0.1 * torch.randn(inner)
    S = 5
    st_c, tl_c = torch.randn(S, H, N, E), torch.randn(S, max(taps - 1, 0), C)
    st_g, tl_g = st_c.cuda(), tl_c.cuda()

    def step(lens, firsts, slots):
        T = sum(lens)
        proj = (0.7 * torch.randn(T, C + inner + H + (0 if H == 8 else 3))).to(dt)   # H == 8: rows of whole 16-byte runs
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
        pos = torch.cat([torch.arange(f, f + n) for f, n in zip(firsts, lens)]).to(torch.int32)
        sl = torch.tensor(slots, dtype=torch.int32)
        row_seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)]).to(torch.int32)
        outs = []
        for mod, p, state, tail, mv in ((ref, proj, st_c, tl_c, lambda t: t), (hk, proj.cuda(), st_g, tl_g, lambda t: t.cuda())):
            q, k, v = p[:, :gn].view(T, G, N), p[:, gn:2 * gn].view(T, G, N), p[:, 2 * gn:C].view(T, H, E)
            z, d = p[:, C:C + inner], p[:, C + inner:C + inner + H]
            lay = (mv(cu), mv(pos), mv(sl))
            kw = dict(conv_bias=mv(cb), ssd=True)
            if mod is hk:
                prep = mod.delta_prepare(q, k, v, None, d, mv(cw), mv(a_log), mv(dtb), tail, *lay, mv(row_seq), **kw)
            else:
                prep = mod.delta_prepare(q, k, v, None, d, cw, a_log, dtb, tail, *lay, **kw)
            o = mod.delta_scan(*prep, state, *lay, correct=False)
            outs.append(mod.gated_group_norm(o, prep[2], mv(skip), z, mv(nw), parts, 1e-5, dt).cpu().float())
        live = torch.cat([torch.full((n,), s >= 0) for n, s in zip(lens, slots)])
        t3 = dict(rtol=3e-2, atol=3e-2) if dt == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(outs[1][live], outs[0][live], **t3)
    step([37, 4, 1], [0, 0, 0], [3, -1, 0])
    step([1, 2], [37, 1], [3, 0])
    torch.testing.assert_close(st_g.cpu()[[0, 3]], st_c[[0, 3]], rtol=1e-4, atol=1e-4)
    if taps > 1:
        torch.testing.assert_close(tl_g.cpu()[[0, 3]], tl_c[[0, 3]], rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,D,E,window", [(16, 256, 128, 40), (3, 40, 24, 0), (2, 320, 200, 25), (4, 128, 64, 7),
                                              (5, 640, 520, 0), (3, 400, 300, 30)])
def test_kernel_attention_with_values_inside_the_key_rows(dt, H, D, E, window):
    """One KV head whose value is the leading E entries of its key row (the V cache is a view of
    the K cache): prompt portions (matrix-core tiles, or rows for sizes without an instance) and
    decode rows (split contexts, or rows) against the CPU form on the same view."""
    torch.manual_seed(5)
    bs, nb = 16, 12
    kc = (0.5 * torch.randn(nb, bs, 1, D)).to(dt)
    vc = kc[..., :E]
    kg = kc.cuda()
    vg = kg[..., :E]
    lens_k, lens_q = [70, 33, 5], [70, 9, 5]                 # whole prompt, a late portion, a short one
    tables = torch.tensor([[3, 1, 7, 9, 11], [0, 2, 4, 0, 0], [5, 0, 0, 0, 0]], dtype=torch.int32)
    T = sum(lens_q)
    q = torch.randn(T, H, D).to(dt)
    cu_q = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
    pos = torch.cat([torch.arange(k - n, k) for k, n in zip(lens_k, lens_q)]).to(torch.int32)
    row_seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens_q)]).to(torch.int32)
    scale = D ** -0.5
    out = torch.zeros(T, H, E, dtype=dt)
    ref.sink_attention_prefill(q, kc, vc, cu_q, cu_k, tables, scale, None, None, out, window)
    outg = torch.zeros(T, H, E, dtype=dt, device="cuda")
    hk.sink_attention_prefill(q.cuda(), kg, vg, cu_q.cuda(), cu_k.cuda(), tables.cuda(), scale, None, None,
                              outg, positions=pos.cuda(), max_q=max(lens_q), row_seq=row_seq.cuda(),
                              window=window)
    torch.testing.assert_close(outg.cpu().float(), out.float(), **tol(dt, 1e-4))
    qd = torch.randn(3, H, D).to(dt)
    ctx = torch.tensor(lens_k, dtype=torch.int32)
    out = torch.zeros(3, H, E, dtype=dt)
    ref.sink_attention_decode(qd, kc, vc, tables, ctx, scale, None, None, out, window)
    outg = torch.zeros(3, H, E, dtype=dt, device="cuda")
    hk.sink_attention_decode(qd.cuda(), kg, vg, tables.cuda(), ctx.cuda(), scale, None, None, outg,
                             max(lens_k), window=window)
    torch.testing.assert_close(outg.cpu().float(), out.float(), **tol(dt, 1e-4))
