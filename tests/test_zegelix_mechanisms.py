"""The ops the Zegelix family adds (``ops.torch_seqmix``: the engine's CPU path and the kernels'
counterpart) against the oracle's function for the same mechanism, each alone, on inputs made to
show what random numbers hide: a sink that dominates or vanishes, a cap that bites, a pooled block
that is just complete, clamps on both sides, routers with ties, decays next to one."""
import math

import pytest
import torch

import zegelix_oracle as oracle

from minivllm_amd.layers.attention import SinkAttention
from minivllm_amd.layers.rglru import RealGatedLRU
from minivllm_amd.ops import torch_seqmix as ops
from minivllm_amd.utils.context import set_context

F64 = torch.float64


def inv_freq(n, base):
    i = torch.arange(n // 2, dtype=torch.float64)
    return (base ** (-2.0 * i / max(n, 1))).float()


@pytest.mark.parametrize("dims,n", [(8, 8), (4, 10), (0, 6), (2, 2)])
def test_half_rotation_partial_and_full(dims, n):
    torch.manual_seed(0)
    T = 9
    pos = torch.tensor([0, 1, 2, 7, 100, 1000, 4095, 33, 5], dtype=torch.int32)
    x = torch.randn(T, 3, n)
    got = ops._rotate_half(x, pos, inv_freq(dims, 500.0), dims)
    for t in range(T):
        want = oracle.turn_halves(x[t].double(), int(pos[t]), 500.0, dims)
        torch.testing.assert_close(got[t].double(), want, rtol=1e-4, atol=1e-4)
    back = ops._rotate_half(got, -pos, inv_freq(dims, 500.0), dims)
    torch.testing.assert_close(back, x, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("taps", [1, 2, 4, 6])
def test_convolution_whole_and_in_portions(taps):
    torch.manual_seed(1)
    T, C = 23, 10
    x, w, b = torch.randn(T, C), torch.randn(C, taps), torch.randn(C)
    want = oracle.causal_filter(x.double(), w.double(), b.double())
    slots = torch.tensor([1], dtype=torch.int32)
    state = torch.full((3, max(taps - 1, 0), C), 7.0)                # dirty: a start ignores it
    whole = ops.short_conv(x, w, b, state, torch.tensor([0, T], dtype=torch.int32),
                           torch.arange(T, dtype=torch.int32), slots)
    torch.testing.assert_close(whole.double(), want, rtol=1e-5, atol=1e-5)
    state.fill_(-3.0)
    parts, at = [], 0
    for n in (1, 2, 1, 7, 3, 9):                                     # shorter than the filter too
        pos = torch.arange(at, at + n, dtype=torch.int32)
        parts.append(ops.short_conv(x[at:at + n], w, b, state, torch.tensor([0, n], dtype=torch.int32), pos, slots))
        at += n
    torch.testing.assert_close(torch.cat(parts).double(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("C,nb,taps", [(12, 3, 3), (8, 1, 1), (10, 10, 4)])
def test_recurrent_unit_against_the_oracle(C, nb, taps):
    torch.manual_seed(2)
    T, W = 17, 14
    c = C // nb
    w = {"y": torch.randn(C, W) * 0.4, "y.b": torch.randn(C) * 0.2, "x": torch.randn(C, W) * 0.4,
         "x.b": torch.randn(C) * 0.2, "conv": torch.randn(C, taps) * 0.6, "conv.b": torch.randn(C) * 0.2,
         "ra": torch.randn(nb, c, c), "ra.b": torch.randn(nb, c), "ri": torch.randn(nb, c, c),
         "ri.b": torch.randn(nb, c), "lam": torch.cat([torch.tensor([-12.0, 6.0]), torch.randn(C - 2)]),
         "o": torch.eye(C)}
    h = torch.randn(T, W)
    want = oracle.rglru_mixer(h.double(), {k: v.double() for k, v in w.items()},
                              {"width": C, "blocks": nb, "conv": taps})
    unit = RealGatedLRU(C, nb, taps, 8.0, passes=2)
    unit.conv_weight.copy_(w["conv"])
    unit.conv_bias.copy_(w["conv.b"])
    unit.load_gates(w["ra"], w["ra.b"], w["ri"], w["ri.b"])
    unit.lam.copy_(w["lam"])
    for st in unit.slots:
        st.state = torch.full((2, C), 5.0)
        st.conv_state = torch.full((2, max(taps - 1, 0), C), 5.0)
    x, y = h @ w["x"].T + w["x.b"], h @ w["y"].T + w["y.b"]
    outs, at = [], 0
    for n in (6, 1, 1, 9):                       # a portion, two single tokens, a portion
        single = n == 1 and at > 0
        set_context(is_prefill=not single, cu_seqlens_q=torch.tensor([0, n], dtype=torch.int32),
                    positions=torch.arange(at, at + n, dtype=torch.int32),
                    state_slots=torch.tensor([1], dtype=torch.int32))
        outs.append(unit(x[at:at + n], y[at:at + n], torch.float32, which=1))
        at += n
    torch.testing.assert_close(torch.cat(outs).double(), want, rtol=2e-4, atol=2e-5)
    assert float(unit.slots[0].state.min()) == 5.0          # the other pass' state is untouched


def _attend(q, k, v, H, G, window, pool, cap, temps, sink, scale, bs=4):
    """Through the layer: caches of pages of ``bs`` tokens, pooled rows made by ``update_pools``,
    the prompt as one portion and then its last rows again one by one (decode form)."""
    T, D, E = q.shape[0], q.shape[2], v.shape[2]
    a = SinkAttention(H, G, D, E, scale, sink=True, window=window, head_temps=True, softcap=cap, pool=pool)
    a.temps.copy_(temps)
    a.sink.copy_(sink)
    n = -(-T // bs) + 1
    a.k_cache, a.v_cache = torch.zeros(n, bs, G, D), torch.zeros(n, bs, G, E)
    for attr, _, shape in a.block_cache_spec(bs):
        setattr(a, attr, torch.full((n,) + shape, 9.0))
    table = torch.arange(n - 1, -1, -1, dtype=torch.int32)[None, :]
    slots = torch.tensor([int(table[0, t // bs]) * bs + t % bs for t in range(T)], dtype=torch.int32)
    a.k_cache.view(-1, G, D)[slots.long()] = k
    a.v_cache.view(-1, G, E)[slots.long()] = v
    pos = torch.arange(T, dtype=torch.int32)
    set_context(is_prefill=True, cu_seqlens_q=torch.tensor([0, T], dtype=torch.int32),
                cu_seqlens_k=torch.tensor([0, T], dtype=torch.int32), positions=pos, slot_mapping=slots,
                block_tables=table, row_seq=torch.zeros(T, dtype=torch.int32), num_seqs=1)
    a.update_pools()
    whole = a(q, None).view(T, H, E)
    rows = []
    for t in range(T - 3, T):
        set_context(is_prefill=False, positions=pos[t:t + 1], slot_mapping=slots[t:t + 1], block_tables=table,
                    context_lens=torch.tensor([t + 1], dtype=torch.int32), num_seqs=1)
        rows.append(a(q[t:t + 1], None).view(1, H, E))
    return whole, torch.cat(rows)


def _oracle_attention(q, k, v, H, G, window, pool, cap, temps, sink, scale):
    """The oracle's mixer with identity projections: h carries [q | k | v] ready-made."""
    T, D, E = q.shape[0], q.shape[2], v.shape[2]
    Wd = H * D + G * D + G * E
    h = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], -1).double()
    eye = torch.eye(Wd, dtype=F64)
    w = {"q": eye[:H * D], "k": eye[H * D:H * D + G * D], "v": eye[H * D + G * D:], "q.b": torch.zeros(H * D, dtype=F64),
         "k.b": torch.zeros(G * D, dtype=F64), "v.b": torch.zeros(G * E, dtype=F64), "temp": temps.double(),
         "sink": sink.double(), "g": torch.zeros(H * E, Wd, dtype=F64), "o": torch.eye(H * E, dtype=F64)}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "scale": scale, "softcap": cap,
         "mask": {"size": window, "pool": pool}}                       # no 'rot': nothing turns
    return (oracle.attention_mixer(h, w, m) * 2.0).view(T, H, E)       # sigmoid(0) = 1/2


@pytest.mark.parametrize("window,pool,cap", [(5, 3, 0.0), (4, 4, 2.0), (7, 1, 50.0), (3, 6, 0.0), (40, 2, 1.0)])
@pytest.mark.parametrize("sink_value", [-30.0, 0.0, 6.0])
def test_attention_window_pooled_blocks_cap_and_sink(window, pool, cap, sink_value):
    torch.manual_seed(3)
    T, H, G, D, E = 31, 4, 2, 6, 5
    q, k, v = torch.randn(T, H, D) * 2, torch.randn(T, G, D) * 2, torch.randn(T, G, E)
    temps = torch.tensor([1.0, 0.3, 2.0, 1.5])
    sink = torch.tensor([sink_value, sink_value, 0.5, -0.5])
    whole, last = _attend(q, k, v, H, G, window, pool, cap, temps, sink, 0.6)
    want = _oracle_attention(q, k, v, H, G, window, pool, cap, temps, sink, 0.6)
    torch.testing.assert_close(whole.double(), want, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(last.double(), want[-3:], rtol=1e-4, atol=1e-5)


def test_a_pooled_block_joins_exactly_when_it_is_whole_behind_the_window():
    """One key made huge: in block 2 (tokens 8 .. 11, pool 4, window 5) it is seen directly up to
    query 12, by nobody from query 13 to 15 (the block ends at 11 > i - 5), and through the block's
    mean from query 16 on."""
    torch.manual_seed(4)
    T, H, G, D, E = 24, 1, 1, 4, 3
    q = torch.ones(T, H, D)
    k = torch.zeros(T, G, D)
    k[9] = 8.0
    v = torch.zeros(T, G, E)
    v[9] = 1.0
    whole, _ = _attend(q, k, v, H, G, 5, 4, 0.0, torch.ones(1), torch.zeros(1), 1.0)
    seen = whole[:, 0, 0]
    assert all(float(seen[i]) > 0.9 for i in range(9, 14))            # in the window: 9 .. 13
    assert all(float(seen[i]) == 0.0 for i in range(14, 16))          # left the window, block not whole behind it
    assert all(0.2 < float(seen[i]) <= 0.25 + 1e-6 for i in range(16, T))   # a quarter of the value, from 16 on


@pytest.mark.parametrize("experts,top,gates", [(6, 2, 1), (4, 4, 0), (5, 1, 1), (3, 2, 0)])
def test_router_and_capped_experts_against_the_oracle(experts, top, gates):
    torch.manual_seed(5)
    T, W, ff, sff = 19, 12, 6, (8 if gates else 0)
    h = torch.randn(T, W)
    w = {"router": torch.randn(experts, W), "router.b": torch.randn(experts)}
    w["router"][1] = w["router"][0]                                  # an exact tie: the lower index wins
    w["router.b"][1] = w["router.b"][0]
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = torch.randn(ff, W), torch.randn(ff, W), torch.randn(W, ff)
    f = {"expert": {"ff": ff, "limit": 1.2}, "router": {"experts": experts, "top": top}}
    if gates:
        f["shared"] = {"ff": sff, "limit": 0.7}
        w["shared.gate"], w["shared.up"], w["shared.down"] = torch.randn(sff, W), torch.randn(sff, W), torch.randn(W, sff)
        w["shared.sg"] = torch.randn(1, W)
    want = oracle.routed_ff(h.double(), {k: v.double() for k, v in w.items()}, f)
    rw = torch.cat([w["router"]] + ([w["shared.sg"]] if gates else []), 0)
    rb = torch.cat([w["router.b"]] + ([torch.zeros(1)] if gates else []), 0)
    dense = ops.grouped_route(h, rw, top, 1, 1, "chosen", rb, gates)
    assert ((dense[:, :experts] > 0).sum(-1) == top).all()
    torch.testing.assert_close(dense[:, :experts].sum(-1), torch.ones(T), rtol=1e-5, atol=1e-5)
    if top < experts:
        assert not ((dense[:, 1] > 0) & (dense[:, 0] == 0)).any()
    names = [f"e{e}" for e in range(experts)] + (["shared"] if gates else [])
    gu = h @ torch.cat([w[n + ".gate"] for n in names] + [w[n + ".up"] for n in names], 0).T
    act = ops.capped_glu_route_scale(gu, dense, ff, sff, 1.2, 0.7, torch.float32)
    got = act @ torch.cat([w[n + ".down"] for n in names], 1).T
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-4)


def test_the_clamps_bite_on_both_sides():
    g = torch.tensor([[-9.0, 0.5, 9.0, 9.0]])
    u = torch.tensor([[9.0, -9.0, 0.25, -0.25]])
    act = ops.capped_glu_route_scale(torch.cat([g, u], 1), torch.ones(1, 1), 4, 0, 2.0, 0.0, torch.float32)
    sig = lambda z: 1.0 / (1.0 + math.exp(-1.702 * z))
    want = [-9.0 * sig(-9.0) * 3.0, 0.5 * sig(0.5) * -1.0, 2.0 * sig(2.0) * 1.25, 2.0 * sig(2.0) * 0.75]
    torch.testing.assert_close(act[0], torch.tensor(want), rtol=1e-5, atol=1e-6)
