"""gfx950 kernels that the Zegelix family adds or extends (``ops.hip_hybrid``) against the plain
PyTorch forms of the same ops (``ops.torch_seqmix``) on CPU copies of the same inputs: bfloat16
and float32, sizes that are not powers of two, several sequences per step with unused rows,
state carried from one call to the next, pooled blocks whose pages differ from the token pages."""
import pytest
import torch

pytestmark = pytest.mark.gpu

gpu = torch.cuda.is_available()
if gpu:
    from minivllm_amd.ops import hip_hybrid as hk
from minivllm_amd.ops import torch_seqmix as ref

DTYPES = [torch.float32, torch.bfloat16]


def tol(dt, f32=2e-5):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=f32, atol=f32)


def dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


def inv_freq(n, base=10000.0):
    i = torch.arange(n // 2, dtype=torch.float64)
    return (base ** (-2.0 * i / max(n, 1))).float()


def paged(n, rows, extra_rows, G, d, dt, device):
    """A token cache and a pooled cache behind it in one allocation, as the engine lays them out."""
    flat = torch.zeros(n * (rows + extra_rows), G, d, dtype=dt, device=device)
    return flat[:n * rows].view(n, rows, G, d), flat[n * rows:].view(n, extra_rows, G, d)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,E,dims", [(6, 3, 24, 20, 16), (4, 1, 64, 64, 64), (2, 2, 16, 8, 0)])
def test_rotation_store_and_turn_back(dt, H, G, D, E, dims):
    torch.manual_seed(0)
    T, bs, nb = 21, 8, 6
    proj = torch.randn(T, H * D + G * D + G * E + H * E + 8).to(dt)
    pos = torch.randint(0, 3000, (T,), dtype=torch.int32)
    pos[0] = 0
    slots = torch.randperm(nb * bs)[:T].to(torch.int32)
    slots[4] = -1
    f, vf = (inv_freq(dims) if dims else None), inv_freq(E, 500.0)
    out = {}
    for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: None if t is None else t.cuda())):
        p = to(proj.clone())
        q, k, v, g, _ = p.split([H * D, G * D, G * E, H * E, 8], -1)
        kc, vc = to(torch.zeros(nb, bs, G, D, dtype=dt)), to(torch.zeros(nb, bs, G, E, dtype=dt))
        mod.half_rope_store(q.view(T, H, D), k.view(T, G, D), v.view(T, G, E), to(pos), to(f), dims,
                            to(vf), kc, vc, to(slots))
        o = to(torch.randn(T, H, E, generator=torch.Generator().manual_seed(1)).to(dt))
        back = mod.unturn_gate(o, to(pos), to(vf), g, dt)
        plain = mod.unturn_gate(o, to(pos), None, None, dt)
        out[name] = [t.cpu().float() for t in (p, kc, vc, back, plain)]
    for a, b in zip(out["gpu"], out["cpu"]):
        torch.testing.assert_close(a, b, **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("bs,pool", [(8, 4), (8, 3), (8, 16), (16, 1)])
def test_pool_block_means(dt, bs, pool):
    torch.manual_seed(2)
    G, D, E, n = 2, 12, 20, 9
    pr = -(-bs // pool)
    tables = torch.tensor([[5, 2, 7, -1], [1, 8, 0, 3]], dtype=torch.int32)
    # sequence 0 holds rows of positions 10 .. 19, sequence 1 one row at position 23; one unused row
    pos = torch.tensor(list(range(10, 20)) + [23, 0], dtype=torch.int32)
    row_seq = torch.tensor([0] * 10 + [1, -1], dtype=torch.int32)
    slot = torch.tensor([1] * 11 + [-1], dtype=torch.int32)
    kc0, vc0 = torch.randn(n, bs, G, D).to(dt), torch.randn(n, bs, G, E).to(dt)
    res = {}
    for name, mod, device in (("cpu", ref, "cpu"), ("gpu", hk, "cuda")):
        kc, kp = paged(n, bs, pr, G, D, dt, device)
        vc, vp = paged(n, bs, pr, G, E, dt, device)
        kc.copy_(kc0)
        vc.copy_(vc0)
        mod.pool_block_means(kc, vc, kp, vp, pool, pos.to(device), tables.to(device), row_seq.to(device),
                             slot.to(device))
        res[name] = (kp.cpu().float(), vp.cpu().float())
    assert res["cpu"][0].abs().sum() > 0
    for a, b in zip(res["gpu"], res["cpu"]):
        torch.testing.assert_close(a, b, **tol(dt, 1e-6))


def _attention_case(dt, H, G, D, E, bs, window, pool, softcap, lens, qlens, seed=3):
    """Sequences with ``lens`` keys of which the last ``qlens`` are this step's queries; caches
    filled with random rows, pooled rows made by the op itself."""
    torch.manual_seed(seed)
    B = len(lens)
    pages = [-(-L // bs) for L in lens]
    n = sum(pages) + 2
    perm = torch.randperm(n).tolist()
    tables = torch.full((B, max(pages)), -1, dtype=torch.int32)
    at = 0
    for b, pg in enumerate(pages):
        tables[b, :pg] = torch.tensor(perm[at:at + pg], dtype=torch.int32)
        at += pg
    pr = -(-bs // pool) if pool else 1
    kc, kp = paged(n, bs, pr, G, D, dt, "cpu")
    vc, vp = paged(n, bs, pr, G, E, dt, "cpu")
    kc.copy_(torch.randn(n, bs, G, D))
    vc.copy_(torch.randn(n, bs, G, E))
    if pool:
        for b, L in enumerate(lens):
            p = torch.arange(L, dtype=torch.int32)
            ref.pool_block_means(kc, vc, kp, vp, pool, p, tables, torch.full((L,), b, dtype=torch.int32),
                                 torch.ones(L, dtype=torch.int32))
    T = sum(qlens)
    q = torch.randn(T, H, D).to(dt)
    cu_q = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    pos = torch.cat([torch.arange(L - n_, L) for L, n_ in zip(lens, qlens)]).to(torch.int32)
    row_seq = torch.cat([torch.full((n_,), b) for b, n_ in enumerate(qlens)]).to(torch.int32)
    sink = torch.randn(H)
    temps = 1.0 + 0.3 * torch.randn(H)
    return dict(q=q, kc=kc, vc=vc, kp=kp if pool else None, vp=vp if pool else None, tables=tables,
                cu_q=cu_q, cu_k=cu_k, pos=pos, row_seq=row_seq, sink=sink, temps=temps, n=n, pr=pr,
                opt=dict(window=window, softcap=softcap, pool=pool))


def _to_gpu(c, dt, G, D, E, bs):
    kc, kp = paged(c["n"], bs, c["pr"], G, D, dt, "cuda")
    vc, vp = paged(c["n"], bs, c["pr"], G, E, dt, "cuda")
    kc.copy_(c["kc"])
    vc.copy_(c["vc"])
    if c["kp"] is not None:
        kp.copy_(c["kp"])
        vp.copy_(c["vp"])
    return kc, vc, (kp if c["kp"] is not None else None), (vp if c["kp"] is not None else None)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,D,E,bs,window,pool,cap", [
    (6, 2, 64, 64, 16, 37, 16, 20.0),      # tile kernel, pages of one pooled row
    (4, 2, 128, 64, 64, 33, 5, 0.0),       # pooled rows that straddle pages, no cap
    (4, 4, 24, 20, 8, 7, 3, 2.0),          # sizes without a tile or split instance: row kernel
    (8, 2, 64, 128, 32, 50, 0, 5.0),       # no pooled blocks: window, cap and temperatures alone
    (12, 2, 64, 64, 16, 21, 4, 0.0),       # six query heads per KV head: two groups of heads per workgroup
    (8, 1, 32, 32, 16, 9, 2, 4.0),         # padded tile instance, row kernel for single tokens
])
def test_attention_with_pooled_blocks(dt, H, G, D, E, bs, window, pool, cap):
    lens, qlens = [300, 97, 41, 130], [300, 30, 2, 129]
    c = _attention_case(dt, H, G, D, E, bs, window, pool, cap, lens, qlens)
    T = c["q"].shape[0]
    want = torch.zeros(T, H, E, dtype=dt)
    ref.sink_attention_prefill(c["q"], c["kc"], c["vc"], c["cu_q"], c["cu_k"], c["tables"], 0.2, c["sink"],
                               None, want, c["opt"]["window"], 0, None, c["temps"], cap, pool, c["kp"], c["vp"])
    kc, vc, kp, vp = _to_gpu(c, dt, G, D, E, bs)
    got = torch.zeros(T, H, E, dtype=dt, device="cuda")
    hk.sink_attention_prefill(c["q"].cuda(), kc, vc, c["cu_q"].cuda(), c["cu_k"].cuda(), c["tables"].cuda(),
                              0.2, c["sink"].cuda(), None, got, positions=c["pos"].cuda(), max_q=max(qlens),
                              row_seq=c["row_seq"].cuda(), window=window, temps=c["temps"].cuda(),
                              softcap=cap, pool=pool, k_pool=kp, v_pool=vp)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dt, 3e-5))
    # the same rows one by one (the row kernel, whatever the sizes)
    got2 = torch.zeros(T, H, E, dtype=dt, device="cuda")
    hk.sink_attention_step(c["q"].cuda(), kc, vc, c["tables"].cuda(), c["row_seq"].cuda(), c["pos"].cuda(),
                           0.2, c["sink"].cuda(), None, got2, window=window, temps=c["temps"].cuda(),
                           softcap=cap, pool=pool, k_pool=kp, v_pool=vp)
    torch.testing.assert_close(got2.cpu().float(), want.float(), **tol(dt, 3e-5))
    # decode: every sequence's last row alone
    last = (c["cu_q"][1:] - 1).long()
    qd = c["q"][last].contiguous()
    ctx_lens = torch.tensor(lens, dtype=torch.int32)
    got3 = torch.zeros(len(lens), H, E, dtype=dt, device="cuda")
    hk.sink_attention_decode(qd.cuda(), kc, vc, c["tables"].cuda(), ctx_lens.cuda(), 0.2, c["sink"].cuda(),
                             None, got3, max(lens), window=window, temps=c["temps"].cuda(), softcap=cap,
                             pool=pool, k_pool=kp, v_pool=vp)
    torch.testing.assert_close(got3.cpu().float(), want[last].float(), **tol(dt, 3e-5))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("C,nb,taps", [(72, 6, 4), (192, 1, 1), (130, 2, 3), (96, 3, 9)])
def test_conv_and_recurrence_over_steps(dt, C, nb, taps):
    torch.manual_seed(4)
    c = C // nb
    slots_n = 5
    w, bias = torch.randn(C, taps) * 0.5, torch.randn(C) * 0.1
    gw, gb = torch.randn(nb, c, 2 * c) * c ** -0.5, torch.randn(nb, 2 * c) * 0.1
    lam = torch.randn(C)
    st = {"cpu": (torch.zeros(slots_n, C), torch.zeros(slots_n, max(taps - 1, 0), C)),
          "gpu": (torch.zeros(slots_n, C).cuda(), torch.zeros(slots_n, max(taps - 1, 0), C).cuda())}
    # step 1: three prompts' portions (one of a single row, one long) and an unused sequence;
    # step 2: the same sequences go on with portions of other lengths; step 3: one row each
    steps = [([2, 1, 150, 0], [0, 0, 0, 0]), ([1, 3, 70, 0], [2, 1, 150, 0]), (None, [3, 4, 220, 0])]
    seq_slots = torch.tensor([3, 0, 4, -1], dtype=torch.int32)
    for qlens, starts in steps:
        if qlens is None:
            T = 4
            cu_q, row_seq = None, None
            pos = torch.tensor(starts, dtype=torch.int32)
        else:
            T = sum(qlens)
            cu_q = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
            pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, qlens)]).to(torch.int32)
            row_seq = torch.cat([torch.full((n,), b) for b, n in enumerate(qlens)]).to(torch.int32)
        proj = torch.randn(T, 2 * C + 8).to(dt)
        res = {}
        for name, mod, to in (("cpu", ref, lambda t: t), ("gpu", hk, lambda t: None if t is None else t.cuda())):
            p = to(proj)
            x, y = p[:, :C], p[:, C + 8:]
            state, tail = st[name]
            if name == "gpu":
                u = mod.short_conv(x, to(w), to(bias), tail, to(cu_q), to(pos), to(seq_slots), to(row_seq))
            else:
                u = mod.short_conv(x, w, bias, tail, cu_q, pos, seq_slots)
            gates = torch.bmm(u.view(T, nb, c).transpose(0, 1), to(gw))
            o = mod.rglru_scan(u, gates, to(gb), to(lam), y, state, to(cu_q), to(pos), to(seq_slots), 8.0, dt)
            res[name] = (u.cpu(), o.cpu().float(), state.cpu().clone(), tail.cpu().clone())
        live = slice(0, T - (1 if qlens is None else 0))
        torch.testing.assert_close(res["gpu"][0][live], res["cpu"][0][live], rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(res["gpu"][1][live], res["cpu"][1][live], **tol(dt, 5e-5))
        torch.testing.assert_close(res["gpu"][2], res["cpu"][2], rtol=5e-5, atol=5e-5)
        torch.testing.assert_close(res["gpu"][3], res["cpu"][3], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("NE,top,ff,sff,gates", [(8, 3, 16, 24, 1), (5, 5, 3, 0, 0), (4, 1, 8, 8, 0), (16, 4, 64, 128, 1)])
def test_chosen_route_and_capped_activation(dt, NE, top, ff, sff, gates):
    torch.manual_seed(5)
    T, W = 33, 72
    h = torch.randn(T, W).to(dt)
    wr, rb = torch.randn(NE + gates, W) * 0.3, torch.randn(NE + gates)
    want = ref.grouped_route(h, wr, top, 1, 1, "chosen", rb, gates)
    got = hk.grouped_route(h.cuda(), wr.cuda(), top, 1, 1, "chosen", rb.cuda(), gates)
    assert ((want[:, :NE] > 0).sum(-1) == top).all()
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-5)
    C = NE * ff + sff
    gu = (3 * torch.randn(T, 2 * C + 8)).to(dt)[:, :2 * C]
    a = ref.capped_glu_route_scale(gu, want, ff, sff, 2.0, 1.0, dt)
    b = hk.capped_glu_route_scale(gu.cuda(), want.cuda(), ff, sff, 2.0, 1.0, dt)
    torch.testing.assert_close(b.cpu().float(), a.float(), **tol(dt))
    assert (a.float().view(T, -1)[:, :NE * ff].view(T, NE, ff).abs().sum(-1) > 0).sum() == T * top


@pytest.mark.parametrize("dt", DTYPES)
def test_scaled_embedding(dt):
    torch.manual_seed(6)
    table = torch.randn(40, 96).to(dt)
    ids = torch.randint(0, 40, (17,), dtype=torch.int32)
    torch.testing.assert_close(hk.embed_sum(ids.cuda(), None, table.cuda(), None, 12.5).cpu(),
                               ref.embed_sum(ids, None, table, None, 12.5), rtol=1e-6, atol=1e-6)
