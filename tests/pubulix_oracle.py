"""A plain float64 implementation of the Pubulix decoder, one function per mechanism, written from the design's
equations with loops over tokens.  Slow on purpose; it shares no code with the engine.

Weights: a dict name -> tensor (any dtype; floats are used as float64).  Config: the config.json dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return rms_unit(x, eps) * float(g)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def input_conv(h, w):
    """h + conv(h): per channel, tap j of w [width, taps] weighs the input taps - 1 - j steps back; nothing before
    the start of the sequence."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate_adjacent(vec, pos, dims, base):
    """Entries 2i and 2i + 1 of the first ``dims`` form pair i, turned by pos * base^(-2i / dims)."""
    out = vec.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        u, v = float(vec[2 * i]), float(vec[2 * i + 1])
        out[2 * i] = u * math.cos(a) - v * math.sin(a)
        out[2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def rotate_halves(vec, pos, dims, base):
    """Entries i and i + dims/2 of the first ``dims`` form pair i, turned by pos * base^(-2i / dims)."""
    out = vec.clone()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = float(vec[i]), float(vec[i + half])
        out[i] = u * math.cos(a) - v * math.sin(a)
        out[i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def window_softmax(scores_of, i, window, sink=None):
    """Weights of the keys j = max(0, i - window + 1) .. i for query i; ``sink``: one more term exp(sink) in the
    denominator that belongs to no key.  -> (first key, weights)."""
    lo = max(0, i - window + 1)
    sc = torch.stack([scores_of(j) for j in range(lo, i + 1)])
    m = sc.max() if sink is None else torch.maximum(sc.max(), torch.as_tensor(float(sink), dtype=F64))
    e = torch.exp(sc - m)
    den = e.sum() + (0.0 if sink is None else math.exp(float(sink) - float(m)))
    return lo, e / den


def attention(h, W, m):
    """Grouped-query sliding-window attention: rotary on halves of the first rot.dims of every q / k head, scores
    capped by softcap * tanh(score / softcap), plain softmax over the window.  h [T, width] -> [T, width]."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    win, scale, cap = m["mask"]["size"], m["scale"], m["softcap"]
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    q = (h @ W("q").T).view(T, H, d)
    k = (h @ W("k").T).view(T, G, d)
    v = (h @ W("v").T).view(T, G, vd)
    kr = [[rotate_halves(k[t, g], t, rd, base) for g in range(G)] for t in range(T)]
    out = torch.zeros(T, H, vd, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            qi = rotate_halves(q[i, hh], i, rd, base)
            lo, p = window_softmax(lambda j: cap * torch.tanh((qi @ kr[j][g]) * scale / cap), i, win)
            for n, j in enumerate(range(lo, i + 1)):
                out[i, hh] += p[n] * v[j, g]
    return out.reshape(T, H * vd) @ W("o").T


def latent_rows(h, W, m, eps):
    """What a latent layer caches per token: (normed latent [T, kv_rank], rotated shared key part [T, rot_dim])."""
    T = h.shape[0]
    R, r = m["kv_rank"], m["rot_dim"]
    ckv = h @ W("dkv").T
    c = rms_unit(ckv[:, :R], eps) * W("dkv.norm")
    kr = torch.stack([rotate_adjacent(ckv[t, R:], t, r, m["rot"]["base"]) for t in range(T)])
    return c, kr


def latent_attention(h, W, m, eps, rows):
    """Sliding-window attention over a latent: per head the key is [W_uk c | shared rotated part], the value W_uv c;
    the softmax's denominator holds a sink per head; the heads are gated by sigmoid(W_g h).  ``rows``: the (latent,
    rotated part) pair to attend to -- this layer's own or another layer's."""
    T = h.shape[0]
    H, d, r, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    win, scale, base = m["mask"]["size"], m["scale"], m["rot"]["base"]
    c, kr = rows
    q = (h @ W("q").T).view(T, H, d + r)
    uk = W("uk").view(H, d, R)
    uv = W("uv").view(H, vd, R)
    sink = W("sink")
    out = torch.zeros(T, H, vd, dtype=F64)
    for hh in range(H):
        kh = c @ uk[hh].T  # [T, d]
        vh = c @ uv[hh].T  # [T, vd]
        for i in range(T):
            qn = q[i, hh, :d]
            qr = rotate_adjacent(q[i, hh, d:], i, r, base)
            lo, p = window_softmax(lambda j: (qn @ kh[j] + qr @ kr[j]) * scale, i, win, sink=sink[hh])
            for n, j in enumerate(range(lo, i + 1)):
                out[i, hh] += p[n] * vh[j]
    gate = torch.sigmoid(h @ W("g").T)
    return (out.reshape(T, H * vd) * gate) @ W("o").T


def expert(x, Wg, Wu, Wd, limit):
    g = torch.clamp(Wg @ x, max=limit)
    u = torch.clamp(Wu @ x, -limit, limit)
    return Wd @ (g * torch.sigmoid(1.702 * g) * (u + 1.0))


def table_experts(h, tokens, W, table, f):
    """Every token's experts come from a table row of its token id; each counts 1 / top."""
    top = f["router"]["top"]
    out = torch.zeros_like(h)
    for t, tok in enumerate(tokens):
        for k in range(top):
            e = int(table[tok, k])
            out[t] += expert(h[t], W(f"e{e}.gate"), W(f"e{e}.up"), W(f"e{e}.down"), f["expert"]["limit"]) / top
    return out


def forward(cfg, sd, tokens, taps=None):
    """Logits [T, vocab] of one sequence (float64).  ``taps``: if a list, the residual after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]

    def P(name):
        return sd[name].to(F64)

    x = P("embed")[torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    cached = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        W = lambda n, p=p: P(p + "mix." + n)
        h = scalar_norm(x, P(p + "norm1"), eps)
        hin = input_conv(h, P(p + "canon1"))
        if L["type"] == "attention":
            y = attention(hin, W, m)
        else:
            if "kv_from" in m and m["kv_from"] is not None:
                rows = cached[int(m["kv_from"])]
            else:
                rows = cached[i] = latent_rows(hin, W, m, eps)
            y = latent_attention(hin, W, m, eps, rows)
        x = x + mult * torch.sigmoid(h @ P(p + "rg1").T + P(p + "rg1.b")) * y
        f = L.get("mlp")
        if f is not None:
            h = scalar_norm(x, P(p + "norm2"), eps)
            y = table_experts(h, tokens, lambda n, p=p: P(p + "mlp." + n), sd[p + "mlp.table"], f)
            x = x + mult * torch.sigmoid(h @ P(p + "rg2").T + P(p + "rg2.b")) * y
        if taps is not None:
            taps.append(x.clone())
    z = scalar_norm(x, P("final.norm"), eps) @ P("head").T
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(z / cap)
