"""Plain float64 restatement of the Zegelix decoder, one function per mechanism, token loops
written out.  It shares no code with the package: the tests compare the engine with it.

The design in this file's notation (W = width, every norm is x / sqrt(mean(x^2) + eps) * w):

* x = E[token] * s_e; layers run in order, a stretch [a, b) runs n times in a row with the same
  weights, every pass with caches and state of its own; ahead of the first layer of every pass
  (the first too) x <- M [x ; x_0] with x_0 the scaled embedding row;
* a layer: x <- x + mix(norm1 x); x <- x + ff(norm2 x) (ff optional);
* mix "rglru": two branches of c channels, y = gelu_tanh(A h + a) and u = conv(B h + b), conv a
  causal per-channel filter whose LAST tap meets the current token; u is cut into nb equal blocks
  with a square matrix each for the two gates r = sigmoid(R_k u_k + r_k), i = sigmoid(I_k u_k +
  i_k); d = exp(-8 r softplus(lam)); S <- d S + sqrt(1 - d^2) (i u) from S = 0; out = O (S y);
* mix "attention": biased q / k / v, H query heads on G key heads; the first `dims` entries of q
  and k turned in half-split pairs by p f_m, f_m = base^(-2m/dims); values turned over ALL their
  entries by j f'_m, f'_m = base^(-2m/E), before they are cached, each head's weighted sum turned
  back by the query's position; score = cap tanh(scale temp_h (q . k) / cap); query i sees tokens
  j with 0 <= i - j < size and, for every block of P tokens that has passed out of that window as
  a whole (bP + P - 1 <= i - size), ONE key and value, the means of the block's cached keys and
  values;
  one softmax over tokens and blocks whose denominator also holds exp(sink_h); the heads' outputs
  times sigmoid(G_w h) element by element, then the output projection;
* ff: router logits z = R h + r; the `top` largest are chosen, weights = softmax over those;
  expert: g = min(W_g h, L), u = clamp(W_u h, -L, L), W_d (g sigmoid(1.702 g) (u + 1)); a shared
  expert of the same form runs for every token, times sigmoid(w_s . h);
* logits = E norm(x) * s_l (the table as stored, not the scaled rows).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def turn_halves(x, position, base, dims, sign=1.0):
    """x [..., n]: entry m < dims/2 pairs with entry m + dims/2; the pair is turned by
    sign * position * base^(-2m/dims); entries from dims on stay."""
    out = x.clone()
    half = dims // 2
    for m in range(half):
        a = sign * position * base ** (-2.0 * m / dims)
        c, s = math.cos(a), math.sin(a)
        u, v = x[..., m], x[..., m + half]
        out[..., m] = u * c - v * s
        out[..., m + half] = v * c + u * s
    return out


def causal_filter(x, taps_w, bias):
    """x [T, C]; taps_w [C, taps], the last column meets the current token and nothing precedes
    a sequence."""
    T, C = x.shape
    taps = taps_w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = bias.clone()
        for k in range(taps):
            src = t - (taps - 1 - k)
            if src >= 0:
                acc = acc + taps_w[:, k] * x[src]
        out[t] = acc
    return out


def rglru_mixer(h, w, m):
    """h [T, W] -> [T, W].  w: the layer's '.mix.*' tensors without the prefix."""
    T = h.shape[0]
    C, nb = int(m["width"]), int(m["blocks"])
    c = C // nb
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = causal_filter(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    S = torch.zeros(C, dtype=F64)
    out = torch.zeros(T, C, dtype=F64)
    sp = torch.log1p(torch.exp(w["lam"]))
    for t in range(T):
        r = torch.zeros(C, dtype=F64)
        i = torch.zeros(C, dtype=F64)
        for k in range(nb):
            part = u[t, k * c:(k + 1) * c]
            r[k * c:(k + 1) * c] = torch.sigmoid(w["ra"][k] @ part + w["ra.b"][k])
            i[k * c:(k + 1) * c] = torch.sigmoid(w["ri"][k] @ part + w["ri.b"][k])
        d = torch.exp(-8.0 * r * sp)
        S = d * S + torch.sqrt(1.0 - d * d) * (i * u[t])
        out[t] = S * y[t]
    return out @ w["o"].T


def visible(i, size, pool):
    """(tokens, blocks) query position i sees; size 0: every earlier token, no blocks."""
    if not size:
        return list(range(i + 1)), []
    tokens = [j for j in range(i + 1) if i - j < size]
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return tokens, blocks


def attention_mixer(h, w, m):
    T = h.shape[0]
    H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
    D, E = int(m["dim"]), int(m.get("vdim", m["dim"]))
    rot = m.get("rot") or {}
    dims, base = int(rot.get("dims", 0)), float(rot.get("base", 1.0))
    mask = m.get("mask") or {}
    size, pool = int(mask.get("size", 0)), int(mask.get("pool", 0))
    cap = float(m.get("softcap", 0.0))
    scale = float(m["scale"])
    q = (h @ w["q"].T + w["q.b"]).view(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).view(T, G, D)
    v = (h @ w["v"].T + w["v.b"]).view(T, G, E)
    turn_v = bool(rot)
    for t in range(T):
        q[t] = turn_halves(q[t], t, base, dims)
        k[t] = turn_halves(k[t], t, base, dims)
        if turn_v:
            v[t] = turn_halves(v[t], t, base, E)
    out = torch.zeros(T, H, E, dtype=F64)
    for i in range(T):
        tokens, blocks = visible(i, size, pool)
        keys = [k[j] for j in tokens] + [k[b * pool:(b + 1) * pool].mean(0) for b in blocks]
        vals = [v[j] for j in tokens] + [v[b * pool:(b + 1) * pool].mean(0) for b in blocks]
        K, V = torch.stack(keys), torch.stack(vals)                    # [n, G, D], [n, G, E]
        for hd in range(H):
            g = hd // (H // G)
            s = (K[:, g] @ q[i, hd]) * scale * w["temp"][hd]
            if cap:
                s = cap * torch.tanh(s / cap)
            top = torch.maximum(s.max(), w["sink"][hd])
            p = torch.exp(s - top)
            den = p.sum() + torch.exp(w["sink"][hd] - top)
            o = (p[:, None] * V[:, g]).sum(0) / den
            out[i, hd] = turn_halves(o, i, base, E, -1.0) if turn_v else o
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(T, H * E) * gate) @ w["o"].T


def capped_expert(h, gate_w, up_w, down_w, limit):
    g = torch.clamp(h @ gate_w.T, max=limit)
    u = torch.clamp(h @ up_w.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down_w.T


def routed_ff(h, w, f):
    """h [T, W]; w: the layer's '.mlp.*' tensors without the prefix; f: its configuration."""
    T = h.shape[0]
    n, top = int(f["router"]["experts"]), int(f["router"]["top"])
    limit = float(f["expert"]["limit"])
    z = h @ w["router"].T + w["router.b"]
    out = torch.zeros_like(h)
    for t in range(T):
        order = sorted(range(n), key=lambda e: (-float(z[t, e]), e))[:top]
        zs = torch.stack([z[t, e] for e in order])
        p = torch.softmax(zs, 0)
        for e, pe in zip(order, p):
            out[t] += pe * capped_expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)[0]
    if f.get("shared"):
        sh = capped_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], float(f["shared"]["limit"]))
        out = out + sh * torch.sigmoid(h @ w["shared.sg"].T)
    return out


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {}
    a, b, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
    if a == b:
        return [(i, False) for i in range(n)], False
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)], True


def forward(cfg, weights, tokens):
    """tokens: list of ids.  Returns (logits [T, vocab], [stream after every layer run])."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    x = x0.clone()
    seen = []
    order, _ = run_order(cfg)
    for i, first_of_pass in order:
        L = cfg["layers"][i]
        p = f"l{i}."
        if first_of_pass:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T
        mw = {k[len(p) + 4:]: v for k, v in w.items() if k.startswith(p + "mix.")}
        hn = rms_norm(x, w[p + "norm1"], eps)
        x = x + (rglru_mixer(hn, mw, L["mixer"]) if L["type"] == "rglru" else attention_mixer(hn, mw, L["mixer"]))
        if L.get("mlp"):
            fw = {k[len(p) + 4:]: v for k, v in w.items() if k.startswith(p + "mlp.")}
            x = x + routed_ff(rms_norm(x, w[p + "norm2"], eps), fw, L["mlp"])
        seen.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T * float(cfg["logit_scale"])
    return logits, seen


def greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        logits, _ = forward(cfg, weights, toks)
        toks.append(int(torch.argmax(logits[-1])))
    return toks[len(prompt):]
