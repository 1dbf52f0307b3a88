"""Small Zegelix configurations and random checkpoints for the tests (made here, from the tensor
names and shapes the family's checkpoints use; nothing is read from outside)."""
from __future__ import annotations

import json
import os

import torch


def rglru(width=24, blocks=3, conv=3):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def attention(heads=4, kv_heads=2, dim=12, vdim=10, size=9, pool=4, scale=0.4, softcap=8.0,
              rot_dims=8, base=100.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "softcap": softcap, "mask": {"size": size, "pool": pool},
         "rot": {"base": base, "dims": dim if rot_dims is None else rot_dims}}
    return {"type": "attention", "mixer": m}


def moe(experts=5, top=2, ff=12, limit=1.5, shared_ff=20, shared_limit=0.8):
    f = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return f


def config(layers, width=40, vocab=89, eps=1e-5, loop=None, embed_scale=3.0, logit_scale=0.7):
    """``layers``: list of (mixer dict, mlp dict or None); ``loop``: (start, stop, times) or None."""
    c = {"architecture": "Zegelix", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "embedding": {"scale": embed_scale}, "logit_scale": logit_scale,
         "layers": [dict(m, mlp=f) for m, f in layers]}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def default_config():
    """Both mixers, a layer without feed-forward, and a looped stretch that holds a recurrent
    layer and an attention layer (so every pass needs its own state, caches and pooled rows)."""
    return config([(rglru(), moe()), (attention(), moe(experts=3, top=1, ff=8, shared_ff=0)),
                   (rglru(width=16, blocks=1, conv=2), None),
                   (attention(heads=2, kv_heads=2, dim=16, vdim=8, size=17, pool=3, softcap=0.0,
                              rot_dims=None, scale=0.3), moe(experts=4, top=4, ff=4, shared_ff=8))],
                  loop=(1, 3, 2))


def mixer_shapes(kind, m, W):
    if kind == "rglru":
        C, nb, taps = m["width"], m["blocks"], m["conv"]
        c = C // nb
        return [("y", (C, W)), ("y.b", (C,)), ("x", (C, W)), ("x.b", (C,)), ("conv", (C, taps)),
                ("conv.b", (C,)), ("ra", (nb, c, c)), ("ra.b", (nb, c)), ("ri", (nb, c, c)),
                ("ri.b", (nb, c)), ("lam", (C,)), ("o", (W, C))]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    return [("q", (H * D, W)), ("q.b", (H * D,)), ("k", (G * D, W)), ("k.b", (G * D,)), ("v", (G * E, W)),
            ("v.b", (G * E,)), ("temp", (H,)), ("sink", (H,)), ("g", (H * E, W)), ("o", (W, H * E))]


def shapes(c):
    W, V = c["width"], c["vocab"]
    yield "embed", (V, W)
    loop = c.get("loop")
    if loop and loop["stop"] > loop["start"]:
        yield "loop.in", (W, 2 * W)
    for i, L in enumerate(c["layers"]):
        p = f"l{i}."
        yield p + "norm1", (W,)
        for n, s in mixer_shapes(L["type"], L["mixer"], W):
            yield p + "mix." + n, s
        f = L["mlp"]
        if f:
            yield p + "norm2", (W,)
            ff = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                yield p + f"mlp.e{e}.gate", (ff, W)
                yield p + f"mlp.e{e}.up", (ff, W)
                yield p + f"mlp.e{e}.down", (W, ff)
            yield p + "mlp.router", (f["router"]["experts"], W)
            yield p + "mlp.router.b", (f["router"]["experts"],)
            if f.get("shared"):
                s = f["shared"]["ff"]
                yield p + "mlp.shared.gate", (s, W)
                yield p + "mlp.shared.up", (s, W)
                yield p + "mlp.shared.down", (W, s)
                yield p + "mlp.shared.sg", (1, W)
    yield "final.norm", (W,)


def weights(c, seed=0, qk_gain=2.0):
    """Random tensors, rounded to bfloat16 (what a checkpoint holds); queries and keys are scaled
    up so that softmaxes are peaked, router rows so that the choice is rarely a close call, and
    the experts' inputs so that the clamps bite."""
    g = torch.Generator().manual_seed(seed)
    W = c["width"]
    out = {}
    for name, shape in shapes(c):
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf == "b":
            t = 0.3 * r
        elif leaf == "lam":
            t = -1.5 + 1.5 * r
        elif leaf == "temp":
            t = 1.0 + 0.3 * r
        elif leaf == "sink":
            t = r
        elif name == "embed":
            t = r / c["embedding"]["scale"]
        elif name == "loop.in":
            t = torch.cat([torch.eye(W), torch.zeros(W, W)], 1) * 0.7 + 0.6 * r * (2 * W) ** -0.5
        elif leaf in ("ra", "ri"):
            t = 1.5 * r * shape[-1] ** -0.5
        else:
            gain = qk_gain if leaf in ("q", "k", "router", "gate", "up") else 1.0
            t = r * shape[-1] ** -0.5 * gain
        out[name] = t.to(torch.bfloat16)
    return out


def save_checkpoint(folder, c, w):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(c, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(folder, "model.safetensors"))
    return folder
