"""Zegelix: a pre-norm decoder around a fp32 residual stream, x <- x + mix(norm1 x), then
x <- x + ff(norm2 x), whose layers - in whatever order the configuration lists - carry one of two
mixers and an optional routed feed-forward, and where a stretch of layers may run several times
in a row with the same weights (every pass with its own caches and state).  Ahead of the first
layer of every pass the stream is re-mixed with the embedding output x0: x <- M [x ; x0].

* ``rglru``      Griffin's recurrent block (``layers.rglru.RealGatedLRU``): a tanh-gelu branch
                 times a real-gated diagonal recurrence behind a short causal convolution;
* ``attention``  biased q / k / v on grouped heads, half-split rotation of the first ``rot.dims``
                 entries of q and k, VALUES rotated over all their entries by their own position
                 before they are cached and every head's weighted sum turned back by the query's
                 position, a learned temperature per head and a tanh soft cap on the scores, a
                 sliding window behind which every whole block of ``mask.pool`` tokens is seen as
                 ONE mean key and mean value, a learned sink in the softmax denominator, and an
                 element-wise sigmoid gate read from the mixer's input
                 (``layers.attention.SinkAttention`` with temperatures, cap and pooled blocks);
* feed-forward   ``layers.moe.CappedRoutedExperts``: the router renormalises over the experts it
                 chose, experts clamp their pre-activations, a shared expert with a per-token gate.

The embedding row is scaled on its way into the stream; the head is tied: final norm, then the
same table (its rows as stored) as the output projection, times ``logit_scale``.

Everything that reads a mixer's normed input is ONE projection (``in_proj`` with one bias
vector); the stream update and the following norm are one op (``ops.residual_group_norm`` with a
single group).  ``ZegelixConfig.from_dict`` reads the family's ``config.json``.  One rank only.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from minivllm_amd import ops
from minivllm_amd.layers.attention import SinkAttention
from minivllm_amd.layers.layernorm import GroupRMSNorm
from minivllm_amd.layers.moe import CappedRoutedExperts
from minivllm_amd.layers.rglru import RealGatedLRU
from minivllm_amd.layers.rotary_embedding import HalfRotation
from minivllm_amd.utils.context import get_context

MIXER_TYPES = ("rglru", "attention")
RGLRU_SHARPNESS = 8.0           # the constant in the decay's exponent
EXPERT_SLOPE = 1.702            # the experts' activation is g sigmoid(1.702 g) (u + 1)


# ------------------------------------------------------------------ configuration
@dataclass
class ZegelixLayerSpec:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@dataclass
class ZegelixConfig:
    vocab_size: int
    hidden_size: int
    layers: List[ZegelixLayerSpec] = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    rms_norm_epsilon: float = 1e-6
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    max_position: int = 1 << 20          # no table depends on it: positions enter as fp32 angles
    name: str = "zegelix"
    architecture: str = "zegelix"
    tie_word_embeddings: bool = True

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    def passes(self, i: int) -> int:
        """How often layer i runs per token."""
        return self.loop_times if self.loop_start <= i < self.loop_stop else 1

    def run_order(self) -> List[Tuple[int, int, bool]]:
        """(layer, pass, first layer of a pass of the looped stretch) in the order they run."""
        a, b = self.loop_start, self.loop_stop
        out = [(i, 0, False) for i in range(a)]
        for p in range(self.loop_times if b > a else 0):
            out += [(i, p, i == a) for i in range(a, b)]
        return out + [(i, 0, False) for i in range(b, len(self.layers))]

    @classmethod
    def from_dict(cls, c: dict, name: str = "zegelix") -> "ZegelixConfig":
        layers = []
        for L in c["layers"]:
            if L["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown layer type {L['type']!r}")
            f = L.get("mlp")
            if f and f.get("kind") != "moe":
                raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
            layers.append(ZegelixLayerSpec(L["type"], L["mixer"], f or None))
        loop = c.get("loop") or {}
        start, stop = int(loop.get("start", 0)), int(loop.get("stop", 0))
        times = int(loop.get("times", 1))
        if not (0 <= start <= stop <= len(layers)) or times < 1:
            raise ValueError("the loop must be a stretch of the layers that runs at least once")
        if start == stop:
            times = 1
        return cls(vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), layers=layers,
                   loop_start=start, loop_stop=stop, loop_times=times,
                   rms_norm_epsilon=float(c["norm"]["eps"]),
                   embedding_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                   logit_scale=float(c.get("logit_scale", 1.0)),
                   max_position=int(c.get("max_position", 1 << 20)), name=name)

    def validate_engine(self, engine_cfg) -> None:
        if engine_cfg.tp_degree != 1:
            raise ValueError("Zegelix runs on one rank (its mixers are not sharded)")
        for L in self.layers:
            m = L.mixer
            if L.type == "attention":
                H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
                D, E = int(m["dim"]), int(m.get("vdim", m["dim"]))
                if H % G:
                    raise ValueError("heads must be a multiple of kv_heads")
                if D > 1024 or E > 1024:
                    raise ValueError("the attention kernels take keys and values of at most 1024 "
                                     "numbers per head")
                rot = m.get("rot") or {}
                if int(rot.get("dims", 0)) > D or int(rot.get("dims", 0)) % 2 or (rot and E % 2):
                    raise ValueError("rot.dims must be even and at most dim, and rotated values "
                                     "need an even vdim")
                mask = m.get("mask") or {}
                if int(mask.get("pool", 0)) < 0 or int(mask.get("size", 0)) < 0:
                    raise ValueError("mask.size and mask.pool must not be negative")
            else:
                if int(m["width"]) % int(m.get("blocks", 1)):
                    raise ValueError("the gate blocks must divide the recurrent width")
            f = L.mlp
            if f and not 0 < int(f["router"]["top"]) <= int(f["router"]["experts"]):
                raise ValueError("router: `top` must lie in 1 .. experts")


def _param(t: torch.Tensor, like: torch.Tensor, dtype=None) -> nn.Parameter:
    return nn.Parameter(t.to(device=like.device, dtype=dtype or like.dtype).contiguous(),
                        requires_grad=False)


def _take(w: dict, key: str, shape, where: str) -> torch.Tensor:
    if key not in w:
        raise KeyError(f"checkpoint lacks {where}{key}")
    t = w.pop(key)
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"shape mismatch for {where}{key}: expected {tuple(shape)}, checkpoint "
                         f"has {tuple(t.shape)}")
    return t


def _pad8(rows: List[torch.Tensor], bias: List[torch.Tensor]) -> None:
    """Zero rows so that the next block of the fused projection starts at a column that is a
    multiple of eight (kernels read blocks in aligned 16-byte runs when they can)."""
    pad = -sum(r.shape[0] for r in rows) % 8
    if pad:
        rows.append(torch.zeros(pad, rows[0].shape[1], dtype=rows[0].dtype))
        bias.append(torch.zeros(pad, dtype=bias[0].dtype))


def _up8(n: int) -> int:
    return n + (-n % 8)


# ------------------------------------------------------------------ mixers
# A mixer's ``load`` returns the rows it contributes to the layer's input projection and their
# biases; ``forward(proj, out_dtype, which)`` returns the mixer's output [T, W]; ``which`` is the
# pass of a looped layer.
class ZegelixRecurrentMixer(nn.Module):
    def __init__(self, W: int, m: dict, passes: int):
        super().__init__()
        self.W, self.C = W, int(m["width"])
        self.unit = RealGatedLRU(self.C, int(m.get("blocks", 1)), int(m.get("conv", 1)),
                                 RGLRU_SHARPNESS, passes)
        self.o_proj = nn.Parameter(torch.zeros(W, self.C), requires_grad=False)

    def state_cores(self):
        return list(self.unit.slots)

    def attention_cores(self):
        return []

    def forward(self, proj, out_dtype, which):
        C, C8 = self.C, _up8(self.C)
        s = self.unit(proj[:, :C], proj[:, C8:C8 + C], out_dtype, which)
        return F.linear(s, self.o_proj)

    def load(self, w: dict, where: str, like):
        W, C, u = self.W, self.C, self.unit
        nb, c = u.blocks, self.C // u.blocks
        rows, bias = [_take(w, "x", (C, W), where)], [_take(w, "x.b", (C,), where)]
        _pad8(rows, bias)
        rows.append(_take(w, "y", (C, W), where))
        bias.append(_take(w, "y.b", (C,), where))
        u.conv_weight.copy_(_take(w, "conv", (C, u.taps), where))
        u.conv_bias.copy_(_take(w, "conv.b", (C,), where))
        u.load_gates(_take(w, "ra", (nb, c, c), where), _take(w, "ra.b", (nb, c), where),
                     _take(w, "ri", (nb, c, c), where), _take(w, "ri.b", (nb, c), where))
        u.lam.copy_(_take(w, "lam", (C,), where))
        self.o_proj = _param(_take(w, "o", (W, C), where), like)
        return rows, bias

    @staticmethod
    def shapes(W, m):
        C, nb, taps = int(m["width"]), int(m.get("blocks", 1)), int(m.get("conv", 1))
        c = C // nb
        return [("y", (C, W)), ("y.b", (C,)), ("x", (C, W)), ("x.b", (C,)), ("conv", (C, taps)),
                ("conv.b", (C,)), ("ra", (nb, c, c)), ("ra.b", (nb, c)), ("ri", (nb, c, c)),
                ("ri.b", (nb, c)), ("lam", (C,)), ("o", (W, C))]


class ZegelixAttentionMixer(nn.Module):
    def __init__(self, W: int, m: dict, passes: int):
        super().__init__()
        self.W = W
        H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
        D, E = int(m["dim"]), int(m.get("vdim", m["dim"]))
        mask = m.get("mask") or {}
        rot = m.get("rot") or None
        self.rotation = HalfRotation(int(rot.get("dims", 0)), float(rot["base"])) if rot else None
        # values turn over all their entries at the keys' base, whatever part of a key turns
        self.value_rotation = HalfRotation(E, float(rot["base"])) if rot else None
        self.cores = nn.ModuleList([
            SinkAttention(H, G, D, E, float(m["scale"]), sink=True, window=int(mask.get("size", 0)),
                          head_temps=True, softcap=float(m.get("softcap", 0.0)),
                          pool=int(mask.get("pool", 0))) for _ in range(passes)])
        self.sizes = [H * D, G * D, G * E, H * E]
        self.o_proj = nn.Parameter(torch.zeros(W, H * E), requires_grad=False)

    def state_cores(self):
        return []

    def attention_cores(self):
        return list(self.cores)

    def forward(self, proj, out_dtype, which):
        a = self.cores[which]
        ctx = get_context()
        T = proj.shape[0]
        H, G, D, E = a.num_heads, a.num_kv_heads, a.head_dim, a.v_head_dim
        q, k, v, g = proj[:, :sum(self.sizes)].split(self.sizes, dim=-1)
        q = q.view(T, H, D)
        rot, vrot = self.rotation, self.value_rotation
        ops.half_rope_store(q, k.view(T, G, D), v.view(T, G, E), ctx.positions,
                            rot.inv_freq if rot else None, rot.rotary_dim if rot else 0,
                            vrot.inv_freq if vrot else None, a.k_cache, a.v_cache, ctx.slot_mapping)
        a.update_pools()
        o = a(q, None).view(T, H, E)
        o = ops.unturn_gate(o, ctx.positions, vrot.inv_freq if vrot else None, g, out_dtype)
        return F.linear(o, self.o_proj)

    def load(self, w: dict, where: str, like):
        W, a = self.W, self.cores[0]
        H, G, D, E = a.num_heads, a.num_kv_heads, a.head_dim, a.v_head_dim
        sizes = (("q", H * D), ("k", G * D), ("v", G * E))
        rows = [_take(w, k, (n, W), where) for k, n in sizes]
        bias = [_take(w, k + ".b", (n,), where) for k, n in sizes]
        rows.append(_take(w, "g", (H * E, W), where))
        bias.append(torch.zeros(H * E, dtype=bias[0].dtype))
        temp, sink = _take(w, "temp", (H,), where), _take(w, "sink", (H,), where)
        for core in self.cores:
            core.temps.copy_(temp)
            core.sink.copy_(sink)
        self.o_proj = _param(_take(w, "o", (W, H * E), where), like)
        return rows, bias

    @staticmethod
    def shapes(W, m):
        H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
        D, E = int(m["dim"]), int(m.get("vdim", m["dim"]))
        return [("q", (H * D, W)), ("q.b", (H * D,)), ("k", (G * D, W)), ("k.b", (G * D,)),
                ("v", (G * E, W)), ("v.b", (G * E,)), ("temp", (H,)), ("sink", (H,)),
                ("g", (H * E, W)), ("o", (W, H * E))]


_MIXERS = {"rglru": ZegelixRecurrentMixer, "attention": ZegelixAttentionMixer}


def _make_ff(W: int, f: dict) -> CappedRoutedExperts:
    sh = f.get("shared") or {}
    return CappedRoutedExperts(W, int(f["expert"]["ff"]), int(f["router"]["experts"]),
                               int(f["router"]["top"]), float(f["expert"]["limit"]),
                               int(sh.get("ff", 0)), float(sh.get("limit", 0.0)), slope=EXPERT_SLOPE)


class ZegelixLayer(nn.Module):
    def __init__(self, cfg: ZegelixConfig, spec: ZegelixLayerSpec, passes: int):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.rms_norm_epsilon
        self.W, self.kind, self.passes = W, spec.type, passes
        self.norm1 = GroupRMSNorm(W, 1, eps)
        self.mix = _MIXERS[spec.type](W, spec.mixer, passes)
        self.norm2 = GroupRMSNorm(W, 1, eps) if spec.mlp else None
        self.ff = _make_ff(W, spec.mlp) if spec.mlp else None
        self.in_proj = nn.Parameter(torch.zeros(1, W), requires_grad=False)
        self.in_bias = nn.Parameter(torch.zeros(1), requires_grad=False)

    def mixer(self, h, out_dtype, which: int):
        """h: norm1 of the stream -> the mixer's output [T, W]."""
        return self.mix(F.linear(h, self.in_proj, self.in_bias), out_dtype, which)

    def load(self, w: dict, where: str, like) -> None:
        W = self.W
        self.norm1.weight.copy_(_take(w, "norm1", (W,), where))
        mw = {k[4:]: w.pop(k) for k in [k for k in w if k.startswith("mix.")]}
        rows, bias = self.mix.load(mw, where + "mix.", like)
        if mw:
            raise KeyError(f"checkpoint tensor {where}mix.{next(iter(mw))} has no parameter")
        _pad8(rows, bias)                               # row stride of the output: whole runs of 8
        self.in_proj = _param(torch.cat(rows, 0), like)
        self.in_bias = _param(torch.cat(bias, 0), like)
        if self.ff is not None:
            f = self.ff
            self.norm2.weight.copy_(_take(w, "norm2", (W,), where))
            ne, n, sff = f.experts, f.ff, f.shared_ff
            gates = [_take(w, f"mlp.e{e}.gate", (n, W), where) for e in range(ne)]
            ups = [_take(w, f"mlp.e{e}.up", (n, W), where) for e in range(ne)]
            downs = [_take(w, f"mlp.e{e}.down", (W, n), where) for e in range(ne)]
            router, rb = [_take(w, "mlp.router", (ne, W), where)], [_take(w, "mlp.router.b", (ne,), where)]
            if sff:
                gates.append(_take(w, "mlp.shared.gate", (sff, W), where))
                ups.append(_take(w, "mlp.shared.up", (sff, W), where))
                downs.append(_take(w, "mlp.shared.down", (W, sff), where))
                router.append(_take(w, "mlp.shared.sg", (1, W), where))
                rb.append(torch.zeros(1, dtype=rb[0].dtype))
            f.gate_up = _param(torch.cat(gates + ups, 0), like)
            f.down = _param(torch.cat(downs, 1), like)
            f.router.copy_(torch.cat(router, 0))
            f.router_bias.copy_(torch.cat(rb, 0))
        if w:
            raise KeyError(f"checkpoint tensor {where}{next(iter(w))} has no parameter")


class ZegelixModel(nn.Module):
    def __init__(self, cfg: ZegelixConfig):
        super().__init__()
        W = cfg.hidden_size
        self.embed = nn.Embedding(cfg.vocab_size, W)
        self.embed.weight.requires_grad_(False)
        self.embed_scale = cfg.embedding_scale
        self.layers = nn.ModuleList([ZegelixLayer(cfg, s, cfg.passes(i)) for i, s in enumerate(cfg.layers)])
        self.order = cfg.run_order()
        self.loop_in = (nn.Parameter(torch.zeros(W, 2 * W), requires_grad=False) if cfg.has_loop else None)
        self.eps = cfg.rms_norm_epsilon
        self.act_dtype = self.embed.weight.dtype
        # observer for tests: called with (index of the layer run, fp32 stream) after every run
        self.layer_hook = None

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the fp32 residual stream [T, W] after the last layer (the final norm belongs
        to the head: only the rows whose logits are wanted go through it)."""
        dt, eps, order = self.act_dtype, self.eps, self.order
        x0 = ops.embed_sum(input_ids, None, self.embed.weight, None, self.embed_scale)
        # the stream is updated in place; the embedding output is read again at every pass
        x = x0.clone() if (self.loop_in is not None and order and not order[0][2]) else x0
        h = None
        for n, (i, p, first) in enumerate(order):
            L = self.layers[i]
            if first:
                x = F.linear(torch.cat([x, x0], -1).to(dt), self.loop_in).float()
                h = None
            if h is None:
                h = L.norm1(x, dt)
            y = L.mixer(h, dt, p)
            if L.ff is not None:
                y = L.ff(ops.residual_group_norm(x, [y], L.norm2.weight, 1, eps, dt))
            fused = n + 1 < len(order) and not order[n + 1][2]
            h = ops.residual_group_norm(x, [y], self.layers[order[n + 1][0]].norm1.weight if fused else None,
                                        1, eps, dt)
            if self.layer_hook is not None:
                self.layer_hook(n, x)
        return x


class ScaledTiedHead(nn.Module):
    """Final RMS norm, then the embedding table itself as the output projection, times a constant.
    The constant is folded into the norm's fp32 gain (``gain`` = weight * logit_scale), so the
    logits are rounded once.  Applied to the rows a step wants (each sequence's last row, or the
    context's ``logit_rows``)."""

    def __init__(self, embedding: nn.Embedding, eps: float, logit_scale: float):
        super().__init__()
        self.table = [embedding]                     # not a submodule: the weight is the model's
        self.eps, self.logit_scale = eps, float(logit_scale)
        W = embedding.weight.shape[1]
        self.weight_norm = nn.Parameter(torch.ones(W, dtype=torch.float32), requires_grad=False)
        self.gain = nn.Parameter(torch.ones(W, dtype=torch.float32), requires_grad=False)
        self.num_embeddings = embedding.weight.shape[0]
        self.vocab_start = 0

    @property
    def weight(self) -> torch.Tensor:
        return self.table[0].weight

    @torch.no_grad()
    def load_norm(self, t: torch.Tensor) -> None:
        self.weight_norm.copy_(t)
        self.gain.copy_(self.weight_norm * self.logit_scale)

    def select_last(self, hidden: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        if ctx.logit_rows is not None:
            return hidden.index_select(0, ctx.logit_rows.long())
        if ctx.is_prefill and ctx.cu_seqlens_q is not None:
            return hidden.index_select(0, (ctx.cu_seqlens_q[1:] - 1).long())
        return hidden

    def local_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        rows = self.select_last(hidden)
        w = self.weight
        return F.linear(ops.group_rms_norm(rows, self.gain, 1, self.eps, w.dtype), w)

    def forward(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.local_logits(hidden)


class ZegelixForCausalLM(nn.Module):
    needs_aux_rows = False
    prefix_cacheable = False        # per-pass caches and pooled rows: every prompt is computed

    def __init__(self, config: ZegelixConfig):
        super().__init__()
        self.config = config
        self.model = ZegelixModel(config)
        self.lm_head = ScaledTiedHead(self.model.embed, config.rms_norm_epsilon, config.logit_scale)
        self.has_recurrent_state = bool(self.state_layers())

    def forward(self, input_ids, positions=None):
        if positions is None:
            positions = get_context().positions
        return self.model(input_ids, positions)

    def compute_logits(self, hidden):
        return self.lm_head(hidden)

    def compute_local_logits(self, hidden):
        return self.lm_head.local_logits(hidden)

    # ---- what the engine needs to know about caches and state ---------------------------
    def attention_layers(self):
        """Every (layer, pass) cache holder: a looped layer owns one K / V cache per pass."""
        return [a for l in self.model.layers for a in l.mix.attention_cores()]

    def state_layers(self):
        return [c for l in self.model.layers for c in l.mix.state_cores()]

    # ---- weights -----------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, items) -> int:
        """``items``: iterable of (checkpoint name, tensor).  The tensors of a layer are collected
        and then stacked into its fused parameters; unknown, missing or mis-shaped tensors raise
        with their name."""
        like = self.model.embed.weight
        W = self.config.hidden_size
        per_layer: List[dict] = [dict() for _ in self.model.layers]
        need = {"embed", "final.norm"} | ({"loop.in"} if self.model.loop_in is not None else set())
        n = 0
        for name, t in items:
            n += 1
            if name in need:
                want = {"embed": (self.config.vocab_size, W), "final.norm": (W,), "loop.in": (W, 2 * W)}[name]
                if tuple(t.shape) != want:
                    raise ValueError(f"shape mismatch for {name}: expected {want}, checkpoint has {tuple(t.shape)}")
                if name == "embed":
                    like.copy_(t.to(like.dtype))
                elif name == "final.norm":
                    self.lm_head.load_norm(t.to(device=like.device, dtype=torch.float32))
                else:
                    self.model.loop_in.copy_(t.to(like.dtype))
                need.discard(name)
                continue
            li, _, rest = name.partition(".")
            if not (li.startswith("l") and li[1:].isdigit()) or int(li[1:]) >= len(per_layer):
                raise KeyError(f"checkpoint tensor {name!r} has no parameter")
            per_layer[int(li[1:])][rest] = t
        if need:
            raise KeyError(f"checkpoint lacks {sorted(need)[0]}")
        for i, (layer, w) in enumerate(zip(self.model.layers, per_layer)):
            layer.load(w, f"l{i}.", like)
        return n

    def checkpoint_shapes(self):
        """(name, shape) of every tensor a checkpoint of this configuration holds."""
        c = self.config
        W = c.hidden_size
        yield "embed", (c.vocab_size, W)
        if c.has_loop:
            yield "loop.in", (W, 2 * W)
        for i, L in enumerate(c.layers):
            p = f"l{i}."
            yield p + "norm1", (W,)
            for nm, shape in _MIXERS[L.type].shapes(W, L.mixer):
                yield p + "mix." + nm, tuple(int(s) for s in shape)
            if L.mlp:
                f = L.mlp
                yield p + "norm2", (W,)
                n = int(f["expert"]["ff"])
                for e in range(int(f["router"]["experts"])):
                    yield p + f"mlp.e{e}.gate", (n, W)
                    yield p + f"mlp.e{e}.up", (n, W)
                    yield p + f"mlp.e{e}.down", (W, n)
                yield p + "mlp.router", (int(f["router"]["experts"]), W)
                yield p + "mlp.router.b", (int(f["router"]["experts"]),)
                if f.get("shared"):
                    s = int(f["shared"]["ff"])
                    yield p + "mlp.shared.gate", (s, W)
                    yield p + "mlp.shared.up", (s, W)
                    yield p + "mlp.shared.down", (W, s)
                    yield p + "mlp.shared.sg", (1, W)
        yield "final.norm", (W,)

    def random_checkpoint(self, seed: int = 0):
        """Seeded random tensors (values exactly representable in bfloat16) of every checkpoint
        name, scaled so that activations stay O(1) through the stack."""
        g = torch.Generator().manual_seed(seed)
        W = self.config.hidden_size
        out = {}
        for name, shape in self.checkpoint_shapes():
            leaf = name.rsplit(".", 1)[-1]
            r = torch.randn(shape, generator=g)
            if leaf in ("norm1", "norm2") or name == "final.norm":
                t = 1.0 + 0.1 * r
            elif leaf == "conv":
                t = 0.5 * r
            elif leaf == "b":
                t = 0.1 * r
            elif leaf == "lam":
                t = -1.0 + 1.5 * r
            elif leaf == "temp":
                t = 1.0 + 0.2 * r
            elif leaf == "sink":
                t = 0.5 * r
            elif name == "embed":
                t = r / max(self.config.embedding_scale, 1e-6)
            elif name == "loop.in":
                t = torch.cat([torch.eye(W), torch.zeros(W, W)], 1) * 0.8 + 0.5 * r * (2 * W) ** -0.5
            elif leaf == "down" or leaf == "o":
                t = 0.5 * r * (shape[-1] ** -0.5)
            else:
                t = r * (shape[-1] ** -0.5)
            out[name] = t.to(torch.bfloat16)
        return out

    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        self.load_weights(self.random_checkpoint(seed).items())
