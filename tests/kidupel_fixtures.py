"""Small Kidupel configurations and random checkpoints for the tests (made here, from the tensor
names and shapes the family's checkpoints use; nothing is read from outside)."""
from __future__ import annotations

import json
import os

import torch


def parallel(heads=4, kv_heads=2, dim=12, vdim=20, size=9, scale=0.5, left_scale=0.8, right_scale=1.3,
             sheads=4, groups=2, state=8, svdim=6, conv=3, norm_groups=3):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                 "mask": {"size": size}},
        "left_scale": left_scale,
        "right": {"heads": sheads, "groups": groups, "state": state, "vdim": svdim, "conv": conv,
                  "norm_groups": norm_groups},
        "right_scale": right_scale}}


def latent(heads=3, dim=8, rot_dim=12, rot_dims=None, vdim=10, kv_rank=14, q_rank=18, size=11, scale=0.4,
           base=100.0):
    return {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
        "q_rank": q_rank, "scale": scale, "mask": {"size": size},
        "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}}}


def attention(heads=6, kv_heads=3, dim=8, vdim=12, size=7, scale=0.7):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                                           "vdim": vdim, "scale": scale, "mask": {"size": size}}}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def config(layers, width=40, vocab=89, eps=1e-5, loop=None):
    """``layers``: list of (mixer dict, mlp dict or None); ``loop``: (start, stop, times) or None."""
    c = {"architecture": "Kidupel", "vocab": vocab, "width": width, "norm": {"eps": eps},
         "layers": [dict(m, mlp=f) for m, f in layers]}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def default_config():
    """All three mixers, a layer without feed-forward, and a looped stretch that holds a
    recurrent layer and both other kinds (so every pass needs its own state and caches)."""
    return config([(attention(), dense()), (parallel(), dense(24)), (latent(), None),
                   (attention(heads=2, kv_heads=2, dim=16, vdim=8, size=17, scale=0.3), dense(16)),
                   (parallel(heads=2, kv_heads=1, dim=16, vdim=8, size=5, sheads=2, groups=1, state=12,
                             svdim=10, conv=2, norm_groups=1), dense())],
                  loop=(1, 4, 2))


def mixer_shapes(kind, m, W):
    if kind == "parallel":
        l, r = m["left"], m["right"]
        H, G, D, E = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
        Hs, Gs, N, Es, taps = r["heads"], r["groups"], r["state"], r["vdim"], r["conv"]
        inner, gn = Hs * Es, Gs * N
        return [("left.q", (H * D, W)), ("left.k", (G * D, W)), ("left.v", (G * E, W)), ("left.g", (H, W)),
                ("left.o", (W, H * E)), ("right.in", (2 * inner + 2 * gn + Hs, W)),
                ("right.conv", (inner + 2 * gn, taps)), ("right.conv.b", (inner + 2 * gn,)),
                ("right.dt_bias", (Hs,)), ("right.A_log", (Hs,)), ("right.D", (Hs,)),
                ("right.norm", (inner,)), ("right.o", (W, inner))]
    if kind == "latent_attention":
        H, D, P, E, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        return [("dq", (Q, W)), ("dq.norm", (Q,)), ("uq", (H * (D + P), Q)), ("dkv", (R + P, W)),
                ("dkv.norm", (R,)), ("uk", (H * D, R)), ("uv", (H * E, R)), ("g", (H * E, W)),
                ("o", (W, H * E))]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    return [("q", (H * D, W)), ("q.b", (H * D,)), ("k", (G * D, W)), ("k.b", (G * D,)), ("v", (G * E, W)),
            ("v.b", (G * E,)), ("q.norm", (H * D,)), ("k.norm", (G * D,)), ("o", (W, H * E)), ("o.b", (W,))]


def shapes(c):
    W, V = c["width"], c["vocab"]
    yield "embed", (V, W)
    for i, L in enumerate(c["layers"]):
        p = f"l{i}."
        yield p + "norm1", ()
        for n, s in mixer_shapes(L["type"], L["mixer"], W):
            yield p + "mix." + n, s
        f = L["mlp"]
        if f:
            yield p + "mlp.up", (f["ff"], W)
            yield p + "mlp.down", (W, f["ff"])
            yield p + "mlp.act", (2,)
    yield "final.norm", ()
    yield "head", (V, W)


def weights(c, seed=0, qk_gain=2.0):
    """Random tensors, rounded to bfloat16 (what a checkpoint holds); queries and keys are scaled
    up so that softmaxes are peaked."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in shapes(c):
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if leaf in ("norm1", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif leaf == "conv":
            t = 0.6 * r
        elif leaf in ("dt_bias", "D", "act"):
            t = 0.7 * r
        elif leaf == "b":
            t = 0.3 * r
        elif leaf == "A_log":
            t = -1.0 + 0.5 * r
        elif name == "embed":
            t = r
        else:
            gain = qk_gain if leaf in ("q", "k", "uq", "uk", "g") else 1.0
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
