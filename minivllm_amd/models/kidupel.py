"""Kidupel: a decoder of *parallel* layers - one RMS norm with a single gain feeds a sequence
mixer and a feed-forward side by side, x <- x + mixer(h) + ff(h) - around a fp32 residual
stream, where a stretch of layers may run several times in a row with the same weights (every
pass with its own cache and state).  Three mixers, in whatever order the configuration lists:

* ``parallel``          two mixers on the same input, added with a scale each: softmax attention
                        with grouped heads over a sliding window, no positions in the scores, a
                        sigmoid gate per head (``layers.attention.SinkAttention`` without its
                        sink), next to a state-space mixer in its dual form
                        (``layers.state_space.StateSpaceDuality``);
* ``latent_attention``  queries through a normed low-rank latent, keys and values expanded from
                        one cached latent per token plus a rotated key part shared by the heads
                        (``layers.attention.LatentAttention``), windowed, gated element by element;
* ``attention``         biased projections, q and k RMS-normed over their whole projection,
                        windowed softmax.

Feed-forward: down(xIELU(up h)) or none.  Output: the same kind of norm and an untied head.

Everything that reads a layer's normed input is ONE projection (``in_proj``: the mixer's rows,
then the feed-forward's up rows); the branches' outputs are added to the stream, with their
scales, by one kernel that also forms the next layer's input (``ops.residual_sum_norm``).

``KidupelConfig.from_dict`` reads the family's ``config.json``.  Single rank only.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from minivllm_amd import ops
from minivllm_amd.layers.activation import XIELU
from minivllm_amd.layers.attention import LatentAttention, SinkAttention
from minivllm_amd.layers.layernorm import ScalarRMSNorm
from minivllm_amd.layers.rotary_embedding import HalfRotation
from minivllm_amd.layers.state_space import StateSpaceDuality
from minivllm_amd.utils.context import get_context

MIXER_TYPES = ("parallel", "latent_attention", "attention")


# ------------------------------------------------------------------ configuration
@dataclass
class KidupelLayerSpec:
    type: str
    mixer: Dict[str, Any]
    mlp: Optional[Dict[str, Any]]


@dataclass
class KidupelConfig:
    vocab_size: int
    hidden_size: int
    layers: List[KidupelLayerSpec] = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    rms_norm_epsilon: float = 1e-6
    max_position: int = 1 << 20          # no table depends on it: positions enter as fp32 angles
    name: str = "kidupel"
    architecture: str = "kidupel"
    tie_word_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def passes(self, i: int) -> int:
        """How often layer i runs per token."""
        return self.loop_times if self.loop_start <= i < self.loop_stop else 1

    def run_order(self) -> List[Tuple[int, int]]:
        """(layer, pass) in the order they run: the looped stretch repeats as a whole."""
        a, b = self.loop_start, self.loop_stop
        out = [(i, 0) for i in range(a)]
        for p in range(self.loop_times):
            out += [(i, p) for i in range(a, b)]
        return out + [(i, 0) for i in range(b, len(self.layers))]

    @classmethod
    def from_dict(cls, c: dict, name: str = "kidupel") -> "KidupelConfig":
        layers = []
        for L in c["layers"]:
            if L["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown layer type {L['type']!r}")
            f = L.get("mlp")
            if f and f.get("kind") != "dense":
                raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
            layers.append(KidupelLayerSpec(L["type"], L["mixer"], f or None))
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
                   max_position=int(c.get("max_position", 1 << 20)), name=name)

    def validate_engine(self, engine_cfg) -> None:
        if engine_cfg.tp_degree != 1:
            raise ValueError("Kidupel runs on one rank (its mixers are not sharded)")
        for L in self.layers:
            m = L.mixer
            for a in ([m["left"]] if L.type == "parallel" else [m] if L.type == "attention" else []):
                if a["heads"] % a.get("kv_heads", a["heads"]):
                    raise ValueError("heads must be a multiple of kv_heads")
                if int(a.get("vdim", a["dim"])) > 1024 or int(a["dim"]) > 1024:
                    raise ValueError("the attention kernels take keys and values of at most 1024 "
                                     "numbers per head")
            if L.type == "parallel":
                r = m["right"]
                if r["heads"] % r.get("groups", 1) or (r["heads"] * r["vdim"]) % r.get("norm_groups", 1):
                    raise ValueError("state-space heads must be a multiple of groups, and "
                                     "norm_groups must divide heads * vdim")
                if r["state"] > 256:
                    raise ValueError("the recurrence kernel holds states of at most 256 rows")
            if L.type == "latent_attention":
                if int(m["rot"]["dims"]) > int(m["rot_dim"]) or int(m["rot"]["dims"]) % 2:
                    raise ValueError("rot.dims must be even and at most rot_dim")
                if int(m["kv_rank"]) + int(m["rot_dim"]) > 1024:
                    raise ValueError("attention over the latent runs with key rows of at most "
                                     "1024 numbers (kv_rank + rot_dim)")


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


def _pad8(rows: List[torch.Tensor], bias: Optional[List[torch.Tensor]] = None) -> int:
    """Appends zero rows so that the next block of the fused projection starts at a column that is
    a multiple of eight (kernels read blocks in aligned 16-byte runs when they can).  Returns the
    number of rows now in ``rows``."""
    n = sum(r.shape[0] for r in rows)
    pad = -n % 8
    if pad:
        rows.append(torch.zeros(pad, rows[0].shape[1], dtype=rows[0].dtype))
        if bias is not None:
            bias.append(torch.zeros(pad, dtype=bias[0].dtype))
    return n + pad


def _window(m: dict) -> int:
    return int((m.get("mask") or {}).get("size", 0))


# ------------------------------------------------------------------ mixers
# A mixer's ``load`` returns the rows it contributes to the layer's fused projection and their
# biases (None: none); ``forward(proj, out_dtype, which)`` returns [(tensor [T, W], scale)],
# the branches still to be added to the stream; ``which`` is the pass of a looped layer.
class KidupelParallelMixer(nn.Module):
    def __init__(self, W: int, m: dict, eps: float, passes: int):
        super().__init__()
        self.W = W
        l, r = m["left"], m["right"]
        H, G = int(l["heads"]), int(l.get("kv_heads", l["heads"]))
        D, E = int(l["dim"]), int(l.get("vdim", l["dim"]))
        self.left_scale, self.right_scale = float(m["left_scale"]), float(m["right_scale"])
        self.cores = nn.ModuleList([SinkAttention(H, G, D, E, float(l["scale"]), sink=False,
                                                  window=_window(l)) for _ in range(passes)])
        self.left_sizes = [H * D, G * D, G * E, H]
        self.ssd = StateSpaceDuality(int(r["heads"]), int(r.get("groups", 1)), int(r["state"]),
                                     int(r["vdim"]), int(r.get("conv", 1)),
                                     int(r.get("norm_groups", 1)), eps, passes)
        self.left_o = nn.Parameter(torch.zeros(W, H * E), requires_grad=False)
        self.right_o = nn.Parameter(torch.zeros(W, int(r["heads"]) * int(r["vdim"])), requires_grad=False)

    def state_cores(self):
        return list(self.ssd.slots)

    def attention_cores(self):
        return list(self.cores)

    def forward(self, proj, out_dtype, which):
        a = self.cores[which]
        T = proj.shape[0]
        H, G, D, E = a.num_heads, a.num_kv_heads, a.head_dim, a.v_head_dim
        nl = sum(self.left_sizes)
        q, k, v, g = proj[:, :nl].split(self.left_sizes, dim=-1)
        nl += -nl % 8                                   # the state-space block starts on a run of 8
        q = q.view(T, H, D)
        ops.row_norm_store(q, k.view(T, G, D), v.view(T, G, E), None, None, 0.0, a.k_cache,
                           a.v_cache, get_context().slot_mapping)
        left = F.linear(a(q, g), self.left_o)
        right = F.linear(self.ssd(proj[:, nl:], out_dtype, which), self.right_o)
        return [(left, self.left_scale), (right, self.right_scale)]

    def load(self, w: dict, where: str, like):
        W, a, s = self.W, self.cores[0], self.ssd
        H, G, D, E = a.num_heads, a.num_kv_heads, a.head_dim, a.v_head_dim
        rows = [_take(w, "left." + k, (n, W), where) for k, n in
                (("q", H * D), ("k", G * D), ("v", G * E), ("g", H))]
        self.left_o = _param(_take(w, "left.o", (W, H * E), where), like)
        _pad8(rows)
        Hs, Gs, N, Es = s.num_heads, s.groups, s.state_size, s.v_head_dim
        inner, gn = Hs * Es, Gs * N
        # checkpoint order of the input projection: z, x, B, C, dt; of the convolution: x, B, C.
        # The recurrence reads C, B, x, then z and dt (see StateSpaceDuality.split_sizes).
        win = _take(w, "right.in", (2 * inner + 2 * gn + Hs, W), where)
        z, x, B, C, dt = win.split([inner, inner, gn, gn, Hs], 0)
        rows += [C, B, x, z, dt]
        cw = _take(w, "right.conv", (inner + 2 * gn, s.taps), where)
        cb = _take(w, "right.conv.b", (inner + 2 * gn,), where)
        order = [2, 1, 0]
        s.conv_weight.copy_(torch.cat([cw.split([inner, gn, gn], 0)[i] for i in order], 0))
        s.conv_bias.copy_(torch.cat([cb.split([inner, gn, gn], 0)[i] for i in order], 0))
        s.dt_bias.copy_(_take(w, "right.dt_bias", (Hs,), where))
        s.A_log.copy_(_take(w, "right.A_log", (Hs,), where))
        s.skip.copy_(_take(w, "right.D", (Hs,), where))
        s.norm_weight.copy_(_take(w, "right.norm", (inner,), where))
        self.right_o = _param(_take(w, "right.o", (W, inner), where), like)
        return rows, None

    @staticmethod
    def shapes(W, m):
        l, r = m["left"], m["right"]
        H, G, D, E = l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l.get("vdim", l["dim"])
        Hs, Gs, N, Es, taps = r["heads"], r.get("groups", 1), r["state"], r["vdim"], r.get("conv", 1)
        inner, gn = Hs * Es, Gs * N
        return [("left.q", (H * D, W)), ("left.k", (G * D, W)), ("left.v", (G * E, W)),
                ("left.g", (H, W)), ("left.o", (W, H * E)),
                ("right.in", (2 * inner + 2 * gn + Hs, W)), ("right.conv", (inner + 2 * gn, taps)),
                ("right.conv.b", (inner + 2 * gn,)), ("right.dt_bias", (Hs,)), ("right.A_log", (Hs,)),
                ("right.D", (Hs,)), ("right.norm", (inner,)), ("right.o", (W, inner))]


class KidupelLatentMixer(nn.Module):
    def __init__(self, W: int, m: dict, eps: float, passes: int):
        super().__init__()
        self.W, self.eps = W, eps
        H, D, P, E = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
        R, Q = int(m["kv_rank"]), int(m["q_rank"])
        self.q_rank = Q
        rot = HalfRotation(int(m["rot"]["dims"]), float(m["rot"]["base"]))
        self.attn = LatentAttention(H, D, P, E, R, float(m["scale"]), _window(m), rot, eps)
        self.cores = nn.ModuleList([self.attn.core] + [
            LatentAttention.make_core(H, P, R, float(m["scale"]), _window(m)) for _ in range(passes - 1)])
        self.sizes = [Q, R + P, H * E]
        self.q_norm = nn.Parameter(torch.ones(Q, dtype=torch.float32), requires_grad=False)
        self.up_q = nn.Parameter(torch.zeros(H * (D + P), Q), requires_grad=False)
        self.o_proj = nn.Parameter(torch.zeros(W, H * E), requires_grad=False)

    def state_cores(self):
        return []

    def attention_cores(self):
        return list(self.cores)

    def forward(self, proj, out_dtype, which):
        a = self.attn
        T = proj.shape[0]
        cq, dkv, g = proj[:, :sum(self.sizes)].split(self.sizes, dim=-1)
        q = F.linear(ops.rms_norm_rows(cq, self.q_norm, self.eps, out_dtype), self.up_q)
        o = a(q.view(T, a.num_heads, a.head_dim + a.rot_dim), dkv, self.cores[which])
        return [(F.linear(ops.sigmoid_gate(o, g, out_dtype), self.o_proj), 1.0)]

    def load(self, w: dict, where: str, like):
        W, a = self.W, self.attn
        H, D, P, E, R, Q = a.num_heads, a.head_dim, a.rot_dim, a.v_head_dim, a.kv_rank, self.q_rank
        rows = [_take(w, "dq", (Q, W), where), _take(w, "dkv", (R + P, W), where),
                _take(w, "g", (H * E, W), where)]
        self.q_norm.copy_(_take(w, "dq.norm", (Q,), where))
        self.up_q = _param(_take(w, "uq", (H * (D + P), Q), where), like)
        a.latent_norm.copy_(_take(w, "dkv.norm", (R,), where))
        a.up_k = _param(_take(w, "uk", (H * D, R), where).view(H, D, R), like)
        a.up_v = _param(_take(w, "uv", (H * E, R), where).view(H, E, R), like)
        self.o_proj = _param(_take(w, "o", (W, H * E), where), like)
        return rows, None

    @staticmethod
    def shapes(W, m):
        H, D, P, E, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        return [("dq", (Q, W)), ("dq.norm", (Q,)), ("uq", (H * (D + P), Q)), ("dkv", (R + P, W)),
                ("dkv.norm", (R,)), ("uk", (H * D, R)), ("uv", (H * E, R)), ("g", (H * E, W)),
                ("o", (W, H * E))]


class KidupelAttentionMixer(nn.Module):
    def __init__(self, W: int, m: dict, eps: float, passes: int):
        super().__init__()
        self.W, self.eps = W, eps
        H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
        D, E = int(m["dim"]), int(m.get("vdim", m["dim"]))
        self.cores = nn.ModuleList([SinkAttention(H, G, D, E, float(m["scale"]), sink=False,
                                                  window=_window(m)) for _ in range(passes)])
        self.sizes = [H * D, G * D, G * E]
        f32 = dict(dtype=torch.float32)
        self.q_norm = nn.Parameter(torch.ones(H * D, **f32), requires_grad=False)
        self.k_norm = nn.Parameter(torch.ones(G * D, **f32), requires_grad=False)
        self.o_proj = nn.Parameter(torch.zeros(W, H * E), requires_grad=False)
        self.o_bias = nn.Parameter(torch.zeros(W), requires_grad=False)

    def state_cores(self):
        return []

    def attention_cores(self):
        return list(self.cores)

    def forward(self, proj, out_dtype, which):
        a = self.cores[which]
        T = proj.shape[0]
        H, G, D, E = a.num_heads, a.num_kv_heads, a.head_dim, a.v_head_dim
        q, k, v = proj[:, :sum(self.sizes)].split(self.sizes, dim=-1)
        q = q.view(T, H, D)
        ops.row_norm_store(q, k.view(T, G, D), v.view(T, G, E), self.q_norm, self.k_norm, self.eps,
                           a.k_cache, a.v_cache, get_context().slot_mapping)
        return [(F.linear(a(q, None), self.o_proj, self.o_bias), 1.0)]

    def load(self, w: dict, where: str, like):
        W, a = self.W, self.cores[0]
        H, G, D, E = a.num_heads, a.num_kv_heads, a.head_dim, a.v_head_dim
        sizes = (("q", H * D), ("k", G * D), ("v", G * E))
        rows = [_take(w, k, (n, W), where) for k, n in sizes]
        bias = [_take(w, k + ".b", (n,), where) for k, n in sizes]
        self.q_norm.copy_(_take(w, "q.norm", (H * D,), where))
        self.k_norm.copy_(_take(w, "k.norm", (G * D,), where))
        self.o_proj = _param(_take(w, "o", (W, H * E), where), like)
        self.o_bias = _param(_take(w, "o.b", (W,), where), like)
        return rows, bias

    @staticmethod
    def shapes(W, m):
        H, G, D, E = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
        return [("q", (H * D, W)), ("q.b", (H * D,)), ("k", (G * D, W)), ("k.b", (G * D,)),
                ("v", (G * E, W)), ("v.b", (G * E,)), ("q.norm", (H * D,)), ("k.norm", (G * D,)),
                ("o", (W, H * E)), ("o.b", (W,))]


_MIXERS = {"parallel": KidupelParallelMixer, "latent_attention": KidupelLatentMixer,
           "attention": KidupelAttentionMixer}


class KidupelLayer(nn.Module):
    def __init__(self, cfg: KidupelConfig, spec: KidupelLayerSpec, passes: int):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.rms_norm_epsilon
        self.W, self.kind, self.passes = W, spec.type, passes
        self.norm1 = ScalarRMSNorm(eps)
        self.mix = _MIXERS[spec.type](W, spec.mixer, eps, passes)
        self.ff = int(spec.mlp["ff"]) if spec.mlp else 0
        self.act = XIELU() if self.ff else None
        self.down = nn.Parameter(torch.zeros(W, max(self.ff, 1)), requires_grad=False) if self.ff else None
        self.in_proj = nn.Parameter(torch.zeros(1, W), requires_grad=False)
        self.in_bias = None
        self.mix_rows = 0

    def forward(self, h, out_dtype, which: int):
        """h: the layer's normed input.  Returns [(tensor, scale)] still to be added to the stream."""
        proj = F.linear(h, self.in_proj, self.in_bias)
        ys = self.mix(proj[:, :self.mix_rows], out_dtype, which)
        if self.ff:
            ys.append((F.linear(self.act(proj[:, self.mix_rows:self.mix_rows + self.ff], out_dtype), self.down), 1.0))
        return ys

    def load(self, w: dict, where: str, like) -> None:
        W = self.W
        self.norm1.load(_take(w, "norm1", None, where))
        mw = {k[4:]: w.pop(k) for k in [k for k in w if k.startswith("mix.")]}
        rows, bias = self.mix.load(mw, where + "mix.", like)
        if mw:
            raise KeyError(f"checkpoint tensor {where}mix.{next(iter(mw))} has no parameter")
        self.mix_rows = _pad8(rows, bias) if self.ff else sum(r.shape[0] for r in rows)
        if self.ff:
            rows.append(_take(w, "mlp.up", (self.ff, W), where))
            self.down = _param(_take(w, "mlp.down", (W, self.ff), where), like)
            self.act.load(_take(w, "mlp.act", (2,), where))
            if bias is not None:
                bias.append(torch.zeros(self.ff, dtype=bias[0].dtype))
        if w:
            raise KeyError(f"checkpoint tensor {where}{next(iter(w))} has no parameter")
        _pad8(rows, bias)                               # row stride of the output: whole runs of 8
        self.in_proj = _param(torch.cat(rows, 0), like)
        self.in_bias = _param(torch.cat(bias, 0), like) if bias is not None else None


class KidupelModel(nn.Module):
    def __init__(self, cfg: KidupelConfig):
        super().__init__()
        self.embed = nn.Embedding(cfg.vocab_size, cfg.hidden_size)
        self.embed.weight.requires_grad_(False)
        self.layers = nn.ModuleList([KidupelLayer(cfg, s, cfg.passes(i)) for i, s in enumerate(cfg.layers)])
        self.order = cfg.run_order()
        self.eps = cfg.rms_norm_epsilon
        self.act_dtype = self.embed.weight.dtype
        # observer for tests: called with (index of the layer run, fp32 stream) after every run
        self.layer_hook = None

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the fp32 residual stream [T, W] after the last layer (the final norm belongs
        to the head: only the rows whose logits are wanted go through it)."""
        dt = self.act_dtype
        x = ops.embed_sum(input_ids, None, self.embed.weight, None)
        order = self.order
        h = self.layers[order[0][0]].norm1(x, dt) if order else None
        for n, (i, p) in enumerate(order):
            ys = self.layers[i](h, dt, p)
            nxt = self.layers[order[n + 1][0]].norm1.gain if n + 1 < len(order) else None
            h = ops.residual_sum_norm(x, [y for y, _ in ys], [s for _, s in ys], nxt, self.eps, dt)
            if self.layer_hook is not None:
                self.layer_hook(n, x)
        return x


class ScalarNormedHead(nn.Module):
    """Final single-gain RMS norm + untied output projection, applied to the rows a step wants
    (each sequence's last row, or the context's ``logit_rows``)."""

    def __init__(self, vocab_size: int, hidden_size: int, eps: float):
        super().__init__()
        self.norm = ScalarRMSNorm(eps)
        self.weight = nn.Parameter(torch.zeros(vocab_size, hidden_size), requires_grad=False)
        self.num_embeddings = vocab_size
        self.vocab_start = 0

    def select_last(self, hidden: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        if ctx.logit_rows is not None:
            return hidden.index_select(0, ctx.logit_rows.long())
        if ctx.is_prefill and ctx.cu_seqlens_q is not None:
            return hidden.index_select(0, (ctx.cu_seqlens_q[1:] - 1).long())
        return hidden

    def local_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        rows = self.select_last(hidden)
        return F.linear(self.norm(rows, self.weight.dtype), self.weight)

    def forward(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.local_logits(hidden)


class KidupelForCausalLM(nn.Module):
    needs_aux_rows = False
    prefix_cacheable = False        # untested with per-pass caches: every prompt is computed

    def __init__(self, config: KidupelConfig):
        super().__init__()
        self.config = config
        self.model = KidupelModel(config)
        self.lm_head = ScalarNormedHead(config.vocab_size, config.hidden_size, config.rms_norm_epsilon)
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
        per_layer: List[dict] = [dict() for _ in self.model.layers]
        top = {"embed": self.model.embed.weight, "head": self.lm_head.weight}
        n, seen = 0, set()
        for name, t in items:
            n += 1
            if name == "final.norm":
                self.lm_head.norm.load(t)
                seen.add(name)
                continue
            if name in top:
                if tuple(top[name].shape) != tuple(t.shape):
                    raise ValueError(f"shape mismatch for {name}: expected {tuple(top[name].shape)}, "
                                     f"checkpoint has {tuple(t.shape)}")
                top[name].copy_(t.to(top[name].dtype))
                seen.add(name)
                continue
            li, _, rest = name.partition(".")
            if not (li.startswith("l") and li[1:].isdigit()) or int(li[1:]) >= len(per_layer):
                raise KeyError(f"checkpoint tensor {name!r} has no parameter")
            per_layer[int(li[1:])][rest] = t
        for k in list(top) + ["final.norm"]:
            if k not in seen:
                raise KeyError(f"checkpoint lacks {k}")
        for i, (layer, w) in enumerate(zip(self.model.layers, per_layer)):
            layer.load(w, f"l{i}.", like)
        return n

    def checkpoint_shapes(self):
        """(name, shape) of every tensor a checkpoint of this configuration holds."""
        c = self.config
        W = c.hidden_size
        yield "embed", (c.vocab_size, W)
        for i, L in enumerate(c.layers):
            p = f"l{i}."
            yield p + "norm1", ()
            for nm, shape in _MIXERS[L.type].shapes(W, L.mixer):
                yield p + "mix." + nm, tuple(int(s) for s in shape)
            if L.mlp:
                ff = int(L.mlp["ff"])
                yield p + "mlp.up", (ff, W)
                yield p + "mlp.down", (W, ff)
                yield p + "mlp.act", (2,)
        yield "final.norm", ()
        yield "head", (c.vocab_size, W)

    def random_checkpoint(self, seed: int = 0):
        """Seeded random tensors (values exactly representable in bfloat16) of every checkpoint
        name, scaled so that activations stay O(1) through the stack."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        for name, shape in self.checkpoint_shapes():
            leaf = name.rsplit(".", 1)[-1]
            r = torch.randn(shape, generator=g)
            if leaf in ("norm1", "norm") or name == "final.norm":
                t = 1.0 + 0.1 * r
            elif leaf == "conv":
                t = 0.5 * r
            elif leaf in ("dt_bias", "act", "D"):
                t = 0.5 * r
            elif leaf == "b":
                t = 0.1 * r
            elif leaf == "A_log":
                t = -1.0 + 0.5 * r
            elif name == "embed":
                t = r
            else:
                t = r * (shape[-1] ** -0.5)
            out[name] = t.to(torch.bfloat16)
        return out

    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        self.load_weights(self.random_checkpoint(seed).items())
