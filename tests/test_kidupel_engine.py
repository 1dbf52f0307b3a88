"""The Kidupel family inside the engine (registry, loader, scheduler, paged KV + state slots,
kernels) against the plain oracle of ``kidupel_oracle``: every mixer alone (one-layer models),
whole prompts and the stream after every layer run (looped layers run several times), token-by-
token decoding, portions down to two tokens, mixed batches against each request alone, blocks and
slots that are used again, a key that stands out at the first token / at block borders / just
inside and outside the window / hundreds of positions back (in prompts and while decoding, for
all three kinds of attention), long decoding, sizes that are 1 or equal, configurations drawn at
random, greedy generation through ``LLMEngine.generate``, and the replay entry point.  Every test
runs on the CPU (fp32); the ``gpu`` variants run the HIP kernels in float32 and bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import kidupel_fixtures as fx
import kidupel_oracle as oracle

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
    assert type(mc).__name__ == "KidupelConfig"
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
    of the logits themselves."""
    d = got.double() - want.logits
    d = d - d.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.logits.std(-1)
    lim = 2e-4 if dtype == "float32" else 0.25
    assert float(e.max()) < lim, f"logits differ: {float(e.max()):.3g} at {int(e.argmax())} (limit {lim})"
    if dtype != "float32":
        assert float(e.median()) < 0.05, f"typical row differs: {float(e.median()):.3g}"


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
    "attention": ([(fx.attention(), None)], None),
    "attention-one-kv-head": ([(fx.attention(heads=4, kv_heads=1, dim=12, vdim=6, size=4), None)], None),
    "parallel": ([(fx.parallel(), None)], None),
    "parallel-one-tap-one-group": ([(fx.parallel(heads=3, kv_heads=3, dim=8, vdim=8, sheads=3, groups=1,
                                                 state=20, svdim=12, conv=1, norm_groups=1), None)], None),
    "parallel-long-convolution": ([(fx.parallel(conv=6, state=36, sheads=2, groups=2, svdim=72,
                                                norm_groups=8), None)], None),
    "latent": ([(fx.latent(), None)], None),
    "latent-partly-rotated": ([(fx.latent(rot_dim=12, rot_dims=8, q_rank=7, kv_rank=24), None)], None),
    "latent-wide": ([(fx.latent(heads=5, dim=8, rot_dim=6, vdim=8, kv_rank=300, q_rank=9), None)], None),
    "attention-wide-values": ([(fx.attention(heads=6, kv_heads=2, dim=8, vdim=272, size=5), None)], None),
    "feed-forward": ([(fx.attention(heads=1, kv_heads=1, dim=8, vdim=8), fx.dense())], None),
    "one-layer-three-times": ([(fx.parallel(), fx.dense(16))], (0, 1, 3)),
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
    assert len(seen) == len(oracle.layer_order(c)) == 8        # 1 + 3 * 2 + 1
    for x, ref in zip(seen, want.trace):
        lim = 1e-4 if dtype == "float32" else 0.15
        assert float((x[:len(toks)].double() - ref).abs().max()) < lim * float(ref.abs().max())
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
    """Two slots, a KV pool of just over one request: every later request runs on blocks and a
    slot (matrix state and convolution tail of every pass) that an earlier one has left dirty."""
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


def _standout_model(kind, size):
    """One layer made so that ONE key stands out for the last query: token 38's embedding is
    token 39's with its halves swapped, and the key path is a query head's with its input columns
    swapped the same way, so key(token 38) is parallel to q_1(token 39) - wherever token 38 sits
    - while its value is unlike every other token's."""
    W, D = 32, 16
    one = torch.ones((), dtype=torch.bfloat16)
    if kind == "attention":
        c = fx.config([(fx.attention(heads=2, kv_heads=1, dim=D, vdim=D, size=size, scale=1.2), None)],
                      width=W, vocab=40)
        w = fx.weights(c, 50)
        w["l0.mix.k"] = _swap(w["l0.mix.q"][D:2 * D])
        for b in ("q.b", "k.b"):
            w["l0.mix." + b] = torch.zeros_like(w["l0.mix." + b])
        w["l0.mix.q.norm"] = torch.ones_like(w["l0.mix.q.norm"])
        w["l0.mix.k.norm"] = torch.ones_like(w["l0.mix.k.norm"])
    elif kind == "parallel":
        c = fx.config([(fx.parallel(heads=2, kv_heads=1, dim=D, vdim=D, size=size, scale=0.25,
                                    left_scale=2.0, right_scale=0.5, sheads=2, groups=1, state=4,
                                    svdim=4, conv=2, norm_groups=1), None)], width=W, vocab=40)
        w = fx.weights(c, 51)
        w["l0.mix.left.k"] = _swap(w["l0.mix.left.q"][D:2 * D])
    else:
        # the latent path: c_q(39) = c(38) (same down-projection up to the swap, same norm), and
        # head 1's unrotated query and key are both the latent itself, so the score of token 38
        # is scale * |c|^2, the largest a normed latent can reach (the rotated part adds noise)
        R = 24
        c = fx.config([(fx.latent(heads=2, dim=R, rot_dim=4, vdim=8, kv_rank=R, q_rank=R, size=size,
                                  scale=1.5), None)], width=W, vocab=40)
        w = fx.weights(c, 52)
        w["l0.mix.dq"] = _swap(w["l0.mix.dkv"][:R])
        w["l0.mix.dq.norm"] = torch.ones(R, dtype=torch.bfloat16)
        w["l0.mix.dkv.norm"] = torch.ones(R, dtype=torch.bfloat16)
        eye = torch.eye(R, dtype=torch.bfloat16)
        w["l0.mix.uq"][R + 4:2 * R + 4] = eye
        w["l0.mix.uk"][R:2 * R] = eye
    w["l0.norm1"] = one.clone()
    e = w["embed"].clone()
    e[38] = _swap(e[39])
    w["embed"] = e
    return c, w


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("decoded", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("n,size", [(41, 11), (330, 300)], ids=["short", "far"])
@pytest.mark.parametrize("kind", ["attention", "parallel", "latent_attention"])
def test_keys_at_every_edge(tmp_path, device, dtype, kind, decoded, n, size):
    """Token 38 sits at a key position, token 39 at the query position (the last one); key
    positions: the very first token, both sides of a block border, just inside and just outside
    the window (11 keys, or 300 keys: hundreds of positions back), the neighbour.  The oracle's
    logits for a key on either side of the window's edge differ widely, so a window that is off
    by one cannot pass."""
    bs = 8
    c, w = _standout_model(kind, size)
    q = n - 1
    places = [0, bs - 1, bs, q - size + 1, q - size, q - 1] if n < 100 else [0, q - size + 1, q - size]
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=n // bs + 4, block_size=bs, seqs=2)
    seen_logits = {}
    for j in places:
        toks = [1 + (t * 7) % 37 for t in range(n)]            # ids 1 .. 37
        toks[j], toks[q] = 38, 39
        sched = [[("a", n)]] if not decoded else [[("a", n - 6)]] + [[("a", 1)]] * 6
        got = run_schedule(eng, {"a": toks}, sched)["a"]
        want = Expected(c, w, toks)
        close(got, want, dtype)
        seen_logits[j] = want.logits[q]
    spread = float(seen_logits[0].std())
    inside, outside = q - size + 1, q - size
    assert float((seen_logits[inside] - seen_logits[outside]).std()) > 0.1 * spread, \
        "the fixture does not tell a visible key from a hidden one"
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decoding_over_many_blocks(tmp_path, device, dtype):
    """150 single tokens: the windows pass over decoded tokens and many block borders, the
    recurrent states of both passes run long."""
    c = fx.config([(fx.parallel(heads=2, kv_heads=2, dim=8, vdim=4, size=21, sheads=2, groups=2, state=8,
                                svdim=4, conv=4, norm_groups=2), fx.dense(16)),
                   (fx.latent(heads=2, dim=4, rot_dim=8, vdim=6, kv_rank=8, q_rank=6, size=13), None),
                   (fx.attention(heads=2, kv_heads=1, dim=8, vdim=4, size=30), None)],
                  width=24, vocab=61, loop=(0, 2, 2))
    w = fx.weights(c, 14)
    toks = tokens(150, c["vocab"], 15)
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=40, block_size=4)
    got = run_schedule(eng, {"a": toks}, [[("a", 3)]] + [[("a", 1)]] * 147)["a"]
    close(got, Expected(c, w, toks), dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_sizes_that_happen_to_be_one_or_equal(tmp_path, device, dtype):
    """One head, one group, one tap, a window of one key, a window longer than the text, scales
    of one, heads == kv heads, key size == value size, a loop that runs once, a loop over
    everything, no loop entry at all, a model without recurrent layers."""
    for layers, loop in (([(fx.parallel(heads=1, kv_heads=1, dim=8, vdim=8, size=100, left_scale=1.0,
                                        right_scale=1.0, sheads=1, groups=1, state=8, svdim=8, conv=1,
                                        norm_groups=1), fx.dense(8))], (0, 1, 1)),
                         ([(fx.attention(heads=1, kv_heads=1, dim=8, vdim=8, size=1), None),
                           (fx.latent(heads=1, dim=2, rot_dim=2, vdim=2, kv_rank=2, q_rank=2, size=1), None)],
                          (0, 2, 3)),
                         ([(fx.latent(heads=5, dim=6, rot_dim=6, vdim=6, kv_rank=6, q_rank=6, size=100), fx.dense(6)),
                           (fx.parallel(heads=6, kv_heads=6, dim=4, vdim=36, size=2, sheads=6, groups=3,
                                        state=4, svdim=4, conv=5, norm_groups=4), None)], None)):
        c = fx.config(layers, width=16, vocab=50, loop=loop)
        w = fx.weights(c, 16)
        toks = tokens(21, c["vocab"], 17)
        eng = make_engine(tmp_path, c, w, device, dtype)
        got = run_schedule(eng, {"a": toks}, [[("a", 2)], [("a", 12)]] + [[("a", 1)]] * 7)["a"]
        close(got, Expected(c, w, toks), dtype)
        eng.exit()


def _random_config(seed):
    """A configuration drawn from a seed: widths, head counts and sizes (also odd multiples and
    sizes above 128), layer order, windows, taps, groups, the loop and constants all vary."""
    g = torch.Generator().manual_seed(seed)

    def pick(*xs):
        return xs[int(torch.randint(0, len(xs), (1,), generator=g))]
    width = pick(24, 48, 96, 160)
    layers = []
    for _ in range(pick(2, 3, 4, 5)):
        kind = pick("parallel", "latent", "attention")
        if kind == "parallel":
            kv, gs = pick(1, 2, 3), pick(1, 2)
            sh, sv = gs * pick(1, 3), pick(4, 8, 20)
            m = fx.parallel(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=pick(8, 24, 40, 72, 144),
                            vdim=pick(8, 20, 64, 132), size=pick(1, 5, 16, 33, 500), scale=pick(0.1, 0.4),
                            left_scale=pick(0.5, 1.0, 1.7), right_scale=pick(0.4, 1.0, 2.0), sheads=sh,
                            groups=gs, state=pick(4, 12, 40, 136), svdim=sv, conv=pick(1, 2, 3, 4, 5),
                            norm_groups=pick(1, 2, sh))
        elif kind == "latent":
            rot = pick(2, 8, 20)
            m = fx.latent(heads=pick(1, 2, 5), dim=pick(4, 16, 40), rot_dim=rot, rot_dims=pick(rot, rot, 2),
                          vdim=pick(4, 24, 72), kv_rank=pick(6, 20, 100, 200), q_rank=pick(5, 32),
                          size=pick(1, 6, 33, 500), scale=pick(0.1, 0.4), base=pick(10.0, 10000.0, 1e6))
        else:
            kv = pick(1, 2, 3)
            m = fx.attention(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=pick(8, 24, 72, 144),
                             vdim=pick(8, 20, 64, 132), size=pick(1, 5, 16, 33, 500), scale=pick(0.3, 1.1))
        layers.append((m, pick(None, fx.dense(pick(16, 40, 104)))))
    n = len(layers)
    start = pick(*range(n))
    loop = pick(None, (start, pick(*range(start + 1, n + 1)), pick(1, 2, 3)))
    return fx.config(layers, width=width, vocab=pick(50, 131), eps=pick(1e-6, 1e-5), loop=loop)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("seed", list(range(8)))
def test_configurations_drawn_at_random(tmp_path, device, dtype, seed):
    c = _random_config(seed)
    # softer queries and keys than elsewhere: with the sharper ones, a draw with head size 144 at
    # width 24 holds a softmax so close to a tie that 16-bit rounding alone (the plain PyTorch
    # ops in bfloat16 show the same) moves one row by a quarter of the logits' spread
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
    c = fx.config([(fx.parallel(), fx.dense())], width=32, vocab=53)
    w = fx.weights(c, 60)
    bad = dict(w)
    del bad["l0.mix.right.D"]
    with pytest.raises(KeyError, match="l0.mix.right.D"):
        make_engine(tmp_path / "x", c, bad, "cpu", "float32")
    bad = dict(w, **{"l0.mix.extra": torch.zeros(3)})
    with pytest.raises(KeyError, match="l0.mix.extra"):
        make_engine(tmp_path / "y", c, bad, "cpu", "float32")
    bad = dict(w, **{"l0.mix.left.q": torch.zeros(7, 32)})
    with pytest.raises(ValueError, match="l0.mix.left.q"):
        make_engine(tmp_path / "z", c, bad, "cpu", "float32")
    bad = dict(w, **{"l0.norm1": torch.ones(32)})
    with pytest.raises(ValueError, match="one number"):
        make_engine(tmp_path / "v", c, bad, "cpu", "float32")
