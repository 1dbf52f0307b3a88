"""Plain, slow restatement of the Kidupel design in float64 PyTorch: one function per mechanism,
token by token where the design is a recurrence, no code shared with the package.  ``forward``
runs a whole token list through a checkpoint dictionary (name -> tensor) and a configuration
dictionary (the parsed ``config.json``) and returns the logits of every position and the
residual stream after every layer run (a looped layer counts once per pass).

Notation: W width, H heads, G key/value heads (or groups), D key size, E value size, N state
size, R latent size, t token index.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def lin(w, x, b=None):
    y = x @ w.to(F64).t()
    return y if b is None else y + b.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.nn.functional.softplus(z)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)



def scalar_norm(x, g, eps):
    """RMS norm with a single scalar gain."""
    return rms(x, eps) * float(g)


def xielu(z, p, q):
    """softplus(p) z^2 + z/2 above zero, (1/2 + softplus(q)) (e^z - 1 - z) + z/2 at and below."""
    ap = softplus(torch.tensor(float(p), dtype=F64))
    aq = 0.5 + softplus(torch.tensor(float(q), dtype=F64))
    return torch.where(z > 0, ap * z * z + z / 2, aq * (torch.expm1(torch.clamp(z, max=0.0)) - z) + z / 2)


def windowed_softmax_attention(q, k, v, scale, size):
    """q [T,H,D], k [T,G,D], v [T,G,E]; query i sees key j when 0 <= i - j < size."""
    T, H, _ = q.shape
    G, E = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, E, dtype=F64)
    for i in range(T):
        lo = max(0, i - size + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            w = torch.softmax(s, 0)
            out[i, h] = w @ v[lo:i + 1, g]
    return out


def rotate_half(x, position, dims, base):
    """x [..., dims]: entry i is paired with entry i + dims/2; the pair turns by position * f_i,
    f_i = base^(-2i/dims)."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = position * f
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a)], -1)


# ------------------------------------------------------------------ mixers (h: [T, W])
def gated_window_attention(h, p, m):
    """Grouped-head softmax attention over a sliding window, no positions in the scores, one
    sigmoid gate per head on the output."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = lin(p["q"], h).view(T, H, D)
    k = lin(p["k"], h).view(T, G, D)
    v = lin(p["v"], h).view(T, G, E)
    o = windowed_softmax_attention(q, k, v, float(m["scale"]), int(m["mask"]["size"]))
    o = o * torch.sigmoid(lin(p["g"], h))[:, :, None]
    return lin(p["o"], o.reshape(T, H * E))


def state_space_duality(h, p, m, eps):
    """Mamba-2: per head a state S [N, E] with a scalar decay per token."""
    H, E, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    parts = m["norm_groups"]
    T = h.shape[0]
    inner = H * E
    u = lin(p["in"], h)
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    cw, cb = p["conv"].to(F64), p["conv.b"].to(F64)
    padded = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F64), xbc], 0)
    conv = torch.stack([(padded[t:t + taps].t() * cw).sum(-1) + cb for t in range(T)], 0)
    conv = silu(conv)
    x = conv[:, :inner].view(T, H, E)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    C = conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + p["dt_bias"].to(F64))
    A = torch.exp(p["A_log"].to(F64))
    Dk = p["D"].to(F64)
    S = torch.zeros(H, N, E, dtype=F64)
    y = torch.zeros(T, H, E, dtype=F64)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            S[hh] = torch.exp(-A[hh] * dt[t, hh]) * S[hh] + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S[hh].t() @ C[t, g] + Dk[hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * p["norm"].to(F64)
    return lin(p["o"], y)


def side_by_side(h, p, m, eps):
    left = gated_window_attention(h, {k[5:]: v for k, v in p.items() if k.startswith("left.")}, m["left"])
    right = state_space_duality(h, {k[6:]: v for k, v in p.items() if k.startswith("right.")}, m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def latent_attention(h, p, m, eps):
    """Queries through a normed latent; keys and values expanded from a normed latent c, plus one
    rotated key part shared by all heads; windowed softmax; element-wise sigmoid gate."""
    H, D, Dr, E, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    T = h.shape[0]
    cq = rms(lin(p["dq"], h), eps) * p["dq.norm"].to(F64)
    q = lin(p["uq"], cq).view(T, H, D + Dr)
    kv = lin(p["dkv"], h)
    c = rms(kv[:, :R], eps) * p["dkv.norm"].to(F64)
    kr = kv[:, R:]
    ku = lin(p["uk"], c).view(T, H, D)
    v = lin(p["uv"], c).view(T, H, E)
    qf = torch.zeros(T, H, D + Dr, dtype=F64)
    kf = torch.zeros(T, H, D + Dr, dtype=F64)
    for t in range(T):
        qf[t, :, :D] = q[t, :, :D]
        qf[t, :, D:] = torch.cat([rotate_half(q[t, :, D:D + dims], t, dims, base), q[t, :, D + dims:]], -1)
        kf[t, :, :D] = ku[t]
        kf[t, :, D:] = torch.cat([rotate_half(kr[t, :dims], t, dims, base), kr[t, dims:]], -1)[None, :]
    o = windowed_softmax_attention(qf, kf, v, float(m["scale"]), int(m["mask"]["size"]))
    o = o.reshape(T, H * E) * torch.sigmoid(lin(p["g"], h))
    return lin(p["o"], o)


def normed_projection_attention(h, p, m, eps):
    """Biased projections; q and k RMS-normed over their whole projection (all heads at once);
    windowed softmax; no gate."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms(lin(p["q"], h, p["q.b"]), eps) * p["q.norm"].to(F64)
    k = rms(lin(p["k"], h, p["k.b"]), eps) * p["k.norm"].to(F64)
    v = lin(p["v"], h, p["v.b"])
    o = windowed_softmax_attention(q.view(T, H, D), k.view(T, G, D), v.view(T, G, E),
                                   float(m["scale"]), int(m["mask"]["size"]))
    return lin(p["o"], o.reshape(T, H * E), p["o.b"])


MIXERS = {"parallel": side_by_side, "latent_attention": latent_attention,
          "attention": lambda h, p, m, eps: normed_projection_attention(h, p, m, eps)}


def feed_forward(h, p):
    return lin(p["down"], xielu(lin(p["up"], h), p["act"][0], p["act"][1]))


def layer_order(c):
    """Indices of the layers in the order they run: a looped stretch repeats as a whole."""
    n = len(c["layers"])
    loop = c.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(c, w, tokens):
    """-> (logits [T, V], streams [layer runs, T, W]) in float64.  Every layer run sees the whole
    sequence, so each pass of a loop has its own history."""
    eps = float(c["norm"]["eps"])
    x = w["embed"].to(F64)[torch.tensor(tokens)]
    streams = []
    for i in layer_order(c):
        L = c["layers"][i]
        pre = f"l{i}."
        h = scalar_norm(x, w[pre + "norm1"], eps)
        mp = {k[len(pre) + 4:]: v for k, v in w.items() if k.startswith(pre + "mix.")}
        y = MIXERS[L["type"]](h, mp, L["mixer"], eps)
        if L.get("mlp"):
            y = y + feed_forward(h, {k[len(pre) + 4:]: v for k, v in w.items() if k.startswith(pre + "mlp.")})
        x = x + y
        streams.append(x.clone())
    logits = lin(w["head"], scalar_norm(x, w["final.norm"], eps))
    return logits, torch.stack(streams, 0)
