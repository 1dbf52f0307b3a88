"""The Zegelix family inside the engine (registry, loader, scheduler, paged KV with pooled rows,
state slots, kernels) against the plain oracle of ``zegelix_oracle``: every mechanism alone
(one-layer models), whole prompts and the stream after every layer run (looped layers run several
times, each pass behind the embedding re-mix), token-by-token decoding, portions down to two
tokens, mixed batches against each request alone, blocks, pooled rows and slots that are used
again, a key that stands out at the first token / at block borders / just inside and outside the
window / in the newest pooled block and in the block that is not pooled yet / hundreds of
positions back (in prompts and while decoding), long decoding, sizes that are 1 or equal,
configurations drawn at random, greedy generation through ``LLMEngine.generate``, and the replay
entry point.  Every test runs on the CPU (fp32); the ``gpu`` variants run the HIP kernels in
float32 and bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import zegelix_fixtures as fx
import zegelix_oracle as oracle

from minivllm_amd.engine.llm_engine import LLMEngine
from minivllm_amd.models.registry import config_from_path
from minivllm_amd.sampling_parameters import SamplingParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CASES = [pytest.param("cpu", "float32", id="cpu-fp32"),
         pytest.param("cuda", "float32", id="gpu-fp32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]


def make_engine(tmp_path, c, w, device, dtype, blocks=24, block_size=8, seqs=3, score=True, **kw):
    folder = fx.save_checkpoint(str(tmp_path / "ckpt"), c, w)
    mc = config_from_path(folder)
    assert type(mc).__name__ == "ZegelixConfig"
    cfg = dict(model=mc, checkpoint_path=folder, dtype=dtype, device=device,
               block_size=block_size, max_cached_blocks=blocks, max_num_sequences=seqs,
               max_model_length=blocks * block_size,
               max_num_batched_tokens=blocks * block_size, eos=-1, score_only=score,
               graph_batch_sizes=[1, 2, seqs], tuned_gemms=False)
    cfg.update(kw)
    return LLMEngine(cfg)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


class Expected:
    def __init__(self, c, w, toks):
        self.logits, self.trace = oracle.forward(c, w, toks)


def close(got, want, dtype):
    """Error of a logit row: spread of the difference over the vocabulary relative to the spread
    of the logits themselves.  In bfloat16 a router whose two best logits nearly tie may choose
    the other expert, which moves that row: a twentieth of the rows may lie beyond the limit."""
    d = got.double() - want.logits
    d = d - d.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.logits.std(-1)
    if dtype == "float32":
        assert float(e.max()) < 2e-4, f"logits differ: {float(e.max()):.3g} at {int(e.argmax())}"
    else:
        assert float(e.median()) < 0.06, f"typical row differs: {float(e.median()):.3g}"
        assert float((e > 0.3).float().mean()) <= 0.05, f"{int((e > 0.3).sum())} of {len(e)} rows differ"


def run_schedule(eng, reqs, schedule):
    """``schedule``: list of steps, each a list of (name, count).  Returns name -> [len, V]."""
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    for step in schedule:
        entries, end = [], []
        for name, n in step:
            lo = at[name]
            entries.append({"id": name, "tokens": reqs[name][lo:lo + n], "want": list(range(n))})
            at[name] = lo + n
            if at[name] == len(reqs[name]):
                end.append(name)
        out = eng.score_step(entries, end)
        for name, _ in step:
            got[name].append(out[name])
    return {k: torch.cat(v) for k, v in got.items() if v}


ALONE = {
    "rglru": ([(fx.rglru(), None)], None),
    "rglru-one-block-one-tap": ([(fx.rglru(width=20, blocks=1, conv=1), None)], None),
    "rglru-long-convolution": ([(fx.rglru(width=72, blocks=9, conv=6), None)], None),
    "attention": ([(fx.attention(), None)], None),
    "attention-one-kv-head": ([(fx.attention(heads=4, kv_heads=1, dim=12, vdim=6, size=4, pool=2), None)], None),
    "attention-pool-wider-than-a-page": ([(fx.attention(heads=2, kv_heads=2, dim=8, vdim=8, size=3, pool=11,
                                                        rot_dims=None), None)], None),
    "attention-no-cap-pool-of-one": ([(fx.attention(heads=3, kv_heads=3, dim=16, vdim=4, size=6, pool=1,
                                                    softcap=0.0, rot_dims=2), None)], None),
    "attention-serving-sizes": ([(fx.attention(heads=4, kv_heads=2, dim=64, vdim=64, size=10, pool=3,
                                               rot_dims=32, scale=0.11), None)], None),
    "experts": ([(fx.rglru(width=8, blocks=1, conv=1), fx.moe())], None),
    "experts-no-shared": ([(fx.rglru(width=8, blocks=1, conv=1), fx.moe(experts=6, top=3, ff=8, shared_ff=0))], None),
    "one-layer-three-times": ([(fx.rglru(), fx.moe(ff=8))], (0, 1, 3)),
    "attention-three-times": ([(fx.attention(size=5, pool=2), None)], (0, 1, 3)),
}


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("kind", list(ALONE))
def test_each_mechanism_alone(tmp_path, device, dtype, kind):
    """One-layer models: whole prompt, then the same tokens as a prompt portion + single tokens."""
    layers, loop = ALONE[kind]
    c = fx.config(layers, width=32, vocab=53, loop=loop)
    w = fx.weights(c, 40)
    toks = tokens(33, c["vocab"], 41)
    eng = make_engine(tmp_path, c, w, device, dtype)
    seen = []
    eng.model_runner.model.model.layer_hook = lambda i, x: seen.append(x.detach().float().cpu().clone())
    want = Expected(c, w, toks)
    close(run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"], want, dtype)
    lim = 1e-4 if dtype == "float32" else 0.1
    n = len(toks)
    if dtype == "float32" or "experts" not in kind:
        assert float((seen[0][:n].double() - want.trace[0]).abs().max()) < lim * float(want.trace[0].abs().max())
    eng.model_runner.model.model.layer_hook = None
    close(run_schedule(eng, {"b": toks}, [[("b", 5)], [("b", 17)]] + [[("b", 1)]] * 11)["b"], want, dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_whole_prompt_and_every_layer_run(tmp_path, device, dtype):
    c = fx.default_config()
    w = fx.weights(c, 103)
    toks = tokens(37, c["vocab"], 2)
    eng = make_engine(tmp_path, c, w, device, dtype)
    seen = []
    eng.model_runner.model.model.layer_hook = lambda i, x: seen.append(x.detach().float().cpu().clone())
    got = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    want = Expected(c, w, toks)
    close(got, want, dtype)
    assert len(seen) == len(oracle.run_order(c)[0]) == 6        # 1 + 2 * 2 + 1
    if dtype == "float32":
        for x, ref in zip(seen, want.trace):
            assert float((x[:len(toks)].double() - ref).abs().max()) < 1e-4 * float(ref.abs().max())
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_token_by_token_equals_prefill(tmp_path, device, dtype):
    c = fx.default_config()
    w = fx.weights(c, 3)
    toks = tokens(29, c["vocab"], 4)
    eng = make_engine(tmp_path, c, w, device, dtype)
    want = Expected(c, w, toks)
    close(run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in toks])["a"], want, dtype)   # first tokens, then decode
    close(run_schedule(eng, {"b": toks}, [[("b", 20)]] + [[("b", 1)]] * 9)["b"], want, dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("cuts", [[2, 2, 3, 1, 9, 8, 2, 16, 2, 5], [7, 43], [1, 2, 47], [25, 25]])
def test_portions_cut_anywhere(tmp_path, device, dtype, cuts):
    """Portions that end inside a pooled block, inside a page and inside the convolution's reach."""
    c = fx.default_config()
    w = fx.weights(c, 5)
    toks = tokens(sum(cuts), c["vocab"], 6)
    eng = make_engine(tmp_path, c, w, device, dtype)
    got = run_schedule(eng, {"a": toks}, [[("a", n)] for n in cuts])["a"]
    close(got, Expected(c, w, toks), dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_equal_each_request_alone(tmp_path, device, dtype):
    c = fx.default_config()
    w = fx.weights(c, 7)
    reqs = {"a": tokens(41, c["vocab"], 8), "b": tokens(5, c["vocab"], 9), "c": tokens(23, c["vocab"], 10),
            "d": tokens(1, c["vocab"], 11), "e": tokens(18, c["vocab"], 12)}
    sched = [[("a", 9), ("b", 2)],
             [("a", 1), ("b", 1), ("c", 17)],              # a one-token portion next to a prompt
             [("b", 1), ("c", 1)],                         # decode step of two; a sits out
             [("a", 20), ("b", 1), ("c", 1)],              # b ends: its slot and blocks return
             [("a", 1), ("c", 1), ("d", 1)],               # d takes b's slot, first token alone
             [("e", 3), ("a", 1), ("c", 1)],
             [("e", 15), ("a", 9), ("c", 2)]]
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=14, seqs=3)
    got = run_schedule(eng, reqs, sched)
    for k, toks in reqs.items():
        close(got[k], Expected(c, w, toks), dtype)
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == bm.num_blocks and eng.scheduler.state_pool.num_free == 3
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_pool_and_slots_used_again(tmp_path, device, dtype):
    """Two slots, a KV pool of just over one request: every later request runs on blocks, pooled
    rows and a slot (state and convolution tail of every pass) that an earlier one has left dirty."""
    c = fx.default_config()
    w = fx.weights(c, 13)
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=9, seqs=2)
    for i, n in enumerate([60, 33, 64, 9, 2]):
        toks = tokens(n, c["vocab"], 20 + i)
        cut = max(1, n // 3)
        got = run_schedule(eng, {"r": toks}, [[("r", cut)], [("r", n - cut)]] if n > 1 else [[("r", 1)]])["r"]
        close(got, Expected(c, w, toks), dtype)
    eng.exit()


def _swap(t):
    h = t.shape[-1] // 2
    return torch.cat([t[..., h:], t[..., :h]], -1).contiguous()


def _standout_model(size, pool):
    """One attention layer made so that ONE key stands out for the last query: token 38's
    embedding is token 39's with its halves swapped, and the key path is a query head's with its
    input columns swapped the same way, so the unrotated part of key(token 38) equals that of
    q_1(token 39) - wherever token 38 sits - while its value is unlike every other token's.  Only
    the first two of sixteen entries rotate, no cap, a deep sink, temperature one."""
    W, D = 32, 16
    c = fx.config([(fx.attention(heads=2, kv_heads=1, dim=D, vdim=D, size=size, pool=pool, scale=1.2,
                                 softcap=0.0, rot_dims=2), None)], width=W, vocab=40)
    w = fx.weights(c, 50)
    w["l0.mix.k"] = _swap(w["l0.mix.q"][D:2 * D])
    for b in ("q.b", "k.b"):
        w["l0.mix." + b] = torch.zeros_like(w["l0.mix." + b])
    w["l0.mix.temp"] = torch.ones_like(w["l0.mix.temp"])
    w["l0.mix.sink"] = torch.full_like(w["l0.mix.sink"], -4.0)
    w["l0.norm1"] = torch.ones_like(w["l0.norm1"])
    e = w["embed"].clone()
    e[38] = _swap(e[39])
    w["embed"] = e
    return c, w


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("decoded", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("n,size", [(41, 11), (330, 300)], ids=["short", "far"])
def test_keys_at_every_edge(tmp_path, device, dtype, decoded, n, size):
    """Token 38 sits at key positions, token 39 at the query position q (the last one).  With a
    window of `size` and blocks of 4: q - size + 1 is the oldest token of the window; q - size and
    q - size - 1 have left it and their block is not whole behind the window yet (seen by nobody);
    the four tokens before them are the newest pooled block (all four are token 38, so the block's
    mean key is token 38's); 0 .. 3 is the oldest pooled block.  The oracle's logits on either side
    of both edges differ widely, so a window or a pooled range that is off by one cannot pass."""
    bs, pool = 8, 4
    c, w = _standout_model(size, pool)
    q = n - 1
    edge = q - size                                   # 29 in both sizes: block 7 = 28 .. 31
    assert edge % pool == 1
    newest, hidden = tuple(range(edge - 5, edge - 1)), (edge - 1, edge)
    places = [(0,), (0, 1, 2, 3), (edge + 1,), hidden, newest, (edge,)]
    if n < 100:
        places += [(bs - 1,), (bs,), (q - 1,)]
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=n // bs + 4, block_size=bs, seqs=2)
    seen_logits = {}
    for where in places:
        toks = [1 + (t * 7) % 37 for t in range(n)]            # ids 1 .. 37
        for j in where:
            toks[j] = 38
        toks[q] = 39
        sched = [[("a", n)]] if not decoded else [[("a", n - 6)]] + [[("a", 1)]] * 6
        got = run_schedule(eng, {"a": toks}, sched)["a"]
        want = Expected(c, w, toks)
        close(got, want, dtype)
        seen_logits[where] = want.logits[q]
    spread = float(seen_logits[(0,)].std())
    for inside, outside in (((edge + 1,), (edge,)), (newest, hidden), ((0, 1, 2, 3), hidden)):
        assert float((seen_logits[inside] - seen_logits[outside]).std()) > 0.1 * spread, \
            "the fixture does not tell a visible key from a hidden one"
    eng.exit()


def test_the_sink_and_the_turned_values_show(tmp_path):
    """The oracle with the sink taken out, or with values that are not turned back, gives other
    logits than the engine: neither mechanism hides behind the random weights."""
    c = fx.config([(fx.attention(size=6, pool=2), None)], width=32, vocab=53)
    w = fx.weights(c, 44)
    toks = tokens(25, c["vocab"], 45)
    eng = make_engine(tmp_path, c, w, "cpu", "float32")
    got = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    close(got, Expected(c, w, toks), "float32")
    no_sink = dict(w, **{"l0.mix.sink": torch.full_like(w["l0.mix.sink"], -60.0)})
    far = oracle.forward(c, no_sink, toks)[0]
    assert float((got.double() - far).std()) > 0.02 * float(far.std())
    c2 = json.loads(json.dumps(c))
    c2["layers"][0]["mixer"]["rot"]["base"] = 1.0 + 1e-9         # all frequencies one: another turn
    other = oracle.forward(c2, w, toks)[0]
    assert float((got.double() - other).std()) > 0.02 * float(other.std())
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decoding_over_many_blocks(tmp_path, device, dtype):
    """150 single tokens: the window passes over decoded tokens, pooled blocks are completed by
    decoded tokens, many page borders, the recurrent states of both passes run long."""
    c = fx.config([(fx.rglru(width=16, blocks=2, conv=4), fx.moe(experts=3, top=2, ff=8, shared_ff=8)),
                   (fx.attention(heads=2, kv_heads=1, dim=8, vdim=4, size=13, pool=5), None),
                   (fx.attention(heads=2, kv_heads=2, dim=8, vdim=8, size=30, pool=3, softcap=3.0), None)],
                  width=24, vocab=61, loop=(0, 2, 2))
    w = fx.weights(c, 14)
    toks = tokens(150, c["vocab"], 15)
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=40, block_size=4)
    got = run_schedule(eng, {"a": toks}, [[("a", 3)]] + [[("a", 1)]] * 147)["a"]
    close(got, Expected(c, w, toks), dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_sizes_that_happen_to_be_one_or_equal(tmp_path, device, dtype):
    """One head, one block, one tap, one expert, top = experts, a window of one key, a window
    longer than the text, a pool of one token, pool = window = page, scales of one, heads == kv
    heads, key size == value size, a loop that runs once, a loop over everything, no loop at all,
    a model without recurrent layers, one without attention."""
    one = dict(embed_scale=1.0, logit_scale=1.0)
    for layers, loop, extra in (
            ([(fx.rglru(width=8, blocks=1, conv=1), fx.moe(experts=1, top=1, ff=8, shared_ff=8, limit=1.0,
                                                           shared_limit=1.0))], (0, 1, 1), one),
            ([(fx.attention(heads=1, kv_heads=1, dim=8, vdim=8, size=1, pool=1, scale=1.0, rot_dims=None), None),
              (fx.attention(heads=2, kv_heads=2, dim=2, vdim=2, size=8, pool=8, rot_dims=None), None)], (0, 2, 3), {}),
            ([(fx.attention(heads=5, kv_heads=5, dim=6, vdim=6, size=100, pool=2, rot_dims=4), fx.moe(experts=2, top=2, ff=6, shared_ff=6)),
              (fx.rglru(width=16, blocks=16, conv=5), None)], None, {})):
        c = fx.config(layers, width=16, vocab=50, loop=loop, **extra)
        w = fx.weights(c, 16)
        toks = tokens(21, c["vocab"], 17)
        eng = make_engine(tmp_path, c, w, device, dtype)
        got = run_schedule(eng, {"a": toks}, [[("a", 2)], [("a", 12)]] + [[("a", 1)]] * 7)["a"]
        close(got, Expected(c, w, toks), dtype)
        eng.exit()


def _random_config(seed):
    """A configuration drawn from a seed: widths, head counts and sizes (also odd multiples and
    sizes above 128), layer order, windows, pools, taps, blocks, experts, the loop and constants."""
    g = torch.Generator().manual_seed(seed)

    def pick(*xs):
        return xs[int(torch.randint(0, len(xs), (1,), generator=g))]
    width = pick(24, 48, 96, 160)
    layers = []
    for _ in range(pick(2, 3, 4, 5)):
        if pick("rglru", "attention") == "rglru":
            nb = pick(1, 2, 5)
            m = fx.rglru(width=nb * pick(4, 12, 20, 66), blocks=nb, conv=pick(1, 2, 3, 4, 5))
        else:
            kv = pick(1, 2, 3)
            dim = pick(8, 24, 40, 72, 144)
            m = fx.attention(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=dim, vdim=pick(8, 20, 64, 132),
                             size=pick(1, 5, 16, 33, 500), pool=pick(1, 2, 7, 16), scale=pick(0.1, 0.4),
                             softcap=pick(0.0, 5.0, 50.0), rot_dims=pick(None, 2, dim // 2 // 2 * 2),
                             base=pick(10.0, 10000.0, 1e6))
        ne = pick(2, 4, 7)
        layers.append((m, pick(None, fx.moe(experts=ne, top=pick(1, 2, ne), ff=pick(8, 20, 48),
                                            limit=pick(0.5, 2.0, 7.0), shared_ff=pick(0, 8, 40),
                                            shared_limit=pick(0.5, 3.0)))))
    n = len(layers)
    start = pick(*range(n))
    loop = pick(None, (start, pick(*range(start + 1, n + 1)), pick(1, 2, 3)))
    return fx.config(layers, width=width, vocab=pick(50, 131), eps=pick(1e-6, 1e-5), loop=loop,
                     embed_scale=pick(1.0, 5.0, 12.0), logit_scale=pick(0.25, 1.0, 1.5))


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("seed", list(range(8)))
def test_configurations_drawn_at_random(tmp_path, device, dtype, seed):
    c = _random_config(seed)
    w = fx.weights(c, 70 + seed, qk_gain=1.0)
    toks = tokens(45, c["vocab"], 80 + seed)
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=16, block_size=8)
    want = Expected(c, w, toks)
    close(run_schedule(eng, {"a": toks}, [[("a", 45)]])["a"], want, dtype)
    close(run_schedule(eng, {"b": toks}, [[("b", 7)], [("b", 2)], [("b", 26)]] + [[("b", 1)]] * 10)["b"], want, dtype)
    eng.exit()


def _follow(c, w, prompt, gen, dtype):
    """Greedy tokens against the oracle (recomputed from scratch per token: it keeps no state)."""
    toks = list(prompt)
    for t in gen:
        lg = oracle.forward(c, w, toks)[0][-1]
        top2 = lg.topk(2).values
        if dtype == "bfloat16" and float(top2[0] - top2[1]) < 0.15:
            break                          # a near tie: 16-bit rounding may pick either
        if dtype == "bfloat16" and int(lg.argmax()) != t:
            break                          # (a router's near tie upstream; the fp32 cases are exact)
        assert int(lg.argmax()) == t
        toks.append(t)


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_scheduler(tmp_path, device, dtype):
    c = fx.default_config()
    w = fx.weights(c, 18)
    prompts = [tokens(n, c["vocab"], 30 + n) for n in (11, 3, 26, 1)]
    eng = make_engine(tmp_path, c, w, device, dtype, score=False, seqs=3, blocks=30,
                      max_num_batched_tokens=32)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))
    for p, gen in zip(prompts, out["token_ids"]):
        assert len(gen) == 8
        _follow(c, w, p, gen, dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES[:2])
def test_generation_survives_preemption_and_mixed_steps(tmp_path, device, dtype):
    c = fx.default_config()
    w = fx.weights(c, 19)
    prompts = [tokens(n, c["vocab"], 60 + n) for n in (21, 17, 9, 30)]
    eng = make_engine(tmp_path, c, w, device, dtype, score=False, seqs=3, blocks=11, block_size=8,
                      max_num_batched_tokens=24, enable_mixed_batches=True)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=14, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0 and eng.scheduler.num_mixed_steps > 0
    for p, gen in zip(prompts, out["token_ids"]):
        _follow(c, w, p, gen, dtype)
    assert eng.scheduler.state_pool.num_free == 3
    eng.exit()


def test_replay_entry_point_writes_the_oracles_logits(tmp_path):
    c = fx.default_config()
    w = fx.weights(c, 21)
    folder = fx.save_checkpoint(str(tmp_path / "m"), c, w)
    a, b = tokens(70, c["vocab"], 22), tokens(9, c["vocab"], 23)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[40:69], "want": []},
                                     {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]},
                                     {"id": "a", "tokens": a[69:], "want": [0]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder,
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "192",
                        "--block-size", "16", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = oracle.forward(c, w, a)[0].float().numpy(), oracle.forward(c, w, b)[0].float().numpy()
    V = c["vocab"]
    got = {n: np.fromfile(out / f"{n}.f32", "<f4").reshape(-1, V) for n in range(3)}
    np.testing.assert_allclose(got[0], la[[0, 39]], rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(got[1], lb[[7]], rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(got[2], np.stack([lb[8], la[69]]), rtol=2e-4, atol=2e-4)


def test_checkpoint_errors_name_the_tensor(tmp_path):
    c = fx.config([(fx.rglru(), fx.moe()), (fx.attention(), None)], width=32, vocab=53, loop=(0, 1, 2))
    w = fx.weights(c, 60)
    bad = dict(w)
    del bad["l0.mix.lam"]
    with pytest.raises(KeyError, match="l0.mix.lam"):
        make_engine(tmp_path / "x", c, bad, "cpu", "float32")
    bad = dict(w, **{"l1.mix.extra": torch.zeros(3)})
    with pytest.raises(KeyError, match="l1.mix.extra"):
        make_engine(tmp_path / "y", c, bad, "cpu", "float32")
    bad = dict(w, **{"l1.mix.q": torch.zeros(7, 32)})
    with pytest.raises(ValueError, match="l1.mix.q"):
        make_engine(tmp_path / "z", c, bad, "cpu", "float32")
    bad = dict(w)
    del bad["loop.in"]
    with pytest.raises(KeyError, match="loop.in"):
        make_engine(tmp_path / "v", c, bad, "cpu", "float32")
    bad = dict(w)
    del bad["l0.mlp.shared.sg"]
    with pytest.raises(KeyError, match="l0.mlp.shared.sg"):
        make_engine(tmp_path / "u", c, bad, "cpu", "float32")


def test_benchmark_configuration_parses_and_validates():
    import types
    sys.path.insert(0, ROOT)
    import bench
    for size in ("w1024", "w2048"):
        mc = bench.zegelix_model(size)
        mc.validate_engine(types.SimpleNamespace(tp_degree=1))
        runs = mc.run_order()
        assert len(runs) == 8 and sum(first for _, _, first in runs) == 2
        assert [mc.layers[i].type for i, _, _ in runs].count("attention") == 3
    with pytest.raises(ValueError, match="one rank"):
        mc.validate_engine(types.SimpleNamespace(tp_degree=2))
