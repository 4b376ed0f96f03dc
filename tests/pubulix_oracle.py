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


def window_softmax(scores, sink=None):
    """Softmax over the scores of a query's visible keys; ``sink``: one more term exp(sink) in the denominator that
    belongs to no key."""
    m = scores.max() if sink is None else torch.maximum(scores.max(), torch.as_tensor(float(sink), dtype=F64))
    e = torch.exp(scores - m)
    return e / (e.sum() + (0.0 if sink is None else math.exp(float(sink) - float(m))))


def capped(z, cap):
    """cap * tanh(z / cap); a cap of 0 (or none) leaves z as it is."""
    return cap * torch.tanh(z / cap) if cap else z


def attention(h, W, m):
    """Grouped-query sliding-window attention: rotary on halves of the first rot.dims of every q / k head, scores
    capped by softcap * tanh(score / softcap), plain softmax over the window.  h [T, width] -> [T, width]."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    win, scale, cap = m["mask"]["size"], m["scale"], m.get("softcap")
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    q = (h @ W("q").T).view(T, H, d)
    k = (h @ W("k").T).view(T, G, d)
    v = (h @ W("v").T).view(T, G, vd)
    kr = torch.stack([torch.stack([rotate_halves(k[t, g], t, rd, base) for g in range(G)]) for t in range(T)])
    out = torch.zeros(T, H, vd, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            qi = rotate_halves(q[i, hh], i, rd, base)
            lo = max(0, i - win + 1) if win else 0  # the query sees itself and the win - 1 positions before it
            p = window_softmax(capped((kr[lo:i + 1, g] @ qi) * scale, cap))
            out[i, hh] = p @ v[lo:i + 1, g]
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
            lo = max(0, i - win + 1) if win else 0
            p = window_softmax((kh[lo:i + 1] @ qn + kr[lo:i + 1] @ qr) * scale, sink=sink[hh])
            out[i, hh] = p @ vh[lo:i + 1]
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
        hin = input_conv(h, P(p + "canon1")) if cfg["canon"]["taps"] else h
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
    return capped(z, cfg.get("logit_softcap"))


# ------------------------------------------------------------------------------------------------ test models
def make_config(width=48, vocab=96, kinds=("attention", "latent", "attention", "shared"), no_mlp=(), heads=4,
                kv_heads=2, dim=12, vdim=12, window=11, softcap=5.0, rot_dims=8, rot_base=100.0, scale=0.35,
                lat_heads=3, lat_dim=8, lat_vdim=10, kv_rank=20, rot_dim=6, lat_window=19, lat_scale=0.3,
                lat_base=50.0, experts=5, top=2, ff=24, limit=1.2, taps=3, eps=1e-5, embed_scale=2.5,
                residual_mult=0.5, logit_softcap=12.0):
    """A small config.json dict.  ``kinds``: "attention", "latent" (a latent layer with its own cache) or "shared" (a
    latent layer that attends to the cache of the nearest "latent" before it)."""
    layers, last = [], None
    for i, kind in enumerate(kinds):
        if kind == "attention":
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
                 "mask": {"size": window}, "rot": {"dims": rot_dims, "base": rot_base}}
        else:
            m = {"heads": lat_heads, "dim": lat_dim, "rot_dim": rot_dim, "vdim": lat_vdim, "kv_rank": kv_rank,
                 "scale": lat_scale, "mask": {"size": lat_window}, "rot": {"dims": rot_dim, "base": lat_base}}
            if kind == "shared":
                m["kv_from"] = last
            else:
                last = i
        mlp = None if i in no_mlp else {"kind": "moe", "expert": {"ff": ff, "limit": limit},
                                        "router": {"experts": experts, "top": top}}
        layers.append({"type": "attention" if kind == "attention" else "latent_attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Pubulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "embedding": {"scale": embed_scale}, "residual_mult": residual_mult, "logit_softcap": logit_softcap,
            "layers": layers}


def make_weights(cfg, seed=0):
    """Random bf16 weights (int32 tables) under the checkpoint's names."""
    g = torch.Generator().manual_seed(4242 + seed)
    W, V = cfg["width"], cfg["vocab"]

    def r(*shape, s=None):
        s = shape[-1] ** -0.5 if s is None else s
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    def num(v=1.0, s=0.15):
        return (v + s * torch.randn((), generator=g)).to(torch.bfloat16)

    sd = {"embed": r(V, W, s=1.0), "head": r(V, W, s=2.0 * W ** -0.5), "final.norm": num()}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        sd[p + "norm1"] = num()
        if cfg["canon"]["taps"]:
            sd[p + "canon1"] = r(W, cfg["canon"]["taps"], s=0.4)
        sd[p + "rg1"], sd[p + "rg1.b"] = r(W, W), r(W, s=0.7)
        if L["type"] == "attention":
            H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd.update({p + "mix.q": r(H * d, W, s=2.0 * W ** -0.5), p + "mix.k": r(G * d, W, s=2.0 * W ** -0.5),
                       p + "mix.v": r(G * vd, W), p + "mix.o": r(W, H * vd)})
        else:
            H, d, rr, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            sd.update({p + "mix.q": r(H * (d + rr), W, s=2.0 * W ** -0.5), p + "mix.uk": r(H * d, R),
                       p + "mix.uv": r(H * vd, R), p + "mix.sink": r(H, s=1.5), p + "mix.g": r(H * vd, W),
                       p + "mix.o": r(W, H * vd)})
            if m.get("kv_from") is None:
                sd[p + "mix.dkv"] = r(R + rr, W, s=2.0 * W ** -0.5)
                sd[p + "mix.dkv.norm"] = (1.0 + 0.2 * torch.randn(R, generator=g)).to(torch.bfloat16)
        f = L["mlp"]
        if f is not None:
            sd[p + "norm2"] = num()
            sd[p + "rg2"], sd[p + "rg2.b"] = r(W, W), r(W, s=0.7)
            E, F = f["router"]["experts"], f["expert"]["ff"]
            for e in range(E):
                sd.update({p + f"mlp.e{e}.gate": r(F, W, s=2.0 * W ** -0.5), p + f"mlp.e{e}.up": r(F, W, s=2.0 * W ** -0.5),
                           p + f"mlp.e{e}.down": r(W, F)})
            rows = [torch.randperm(E, generator=g)[: f["router"]["top"]] for _ in range(V)]
            sd[p + "mlp.table"] = torch.stack(rows).to(torch.int32)
    return sd


def logits_and_taps(cfg, sd, tokens):
    taps = []
    z = forward(cfg, sd, tokens, taps)
    return z, torch.stack(taps)
