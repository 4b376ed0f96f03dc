"""A plain float64 implementation of the Leripel decoder, one function per mechanism, written from the design's
equations with loops over tokens.  Slow on purpose; it shares no code with the engine.

Weights: a dict name -> tensor (any float dtype; used as float64).  Config: the config.json dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def rotate_pairs(vec, pos, dims, base):
    """Rotary position on the first ``dims`` entries of ``vec`` (1-D): entries 2i and 2i + 1 form pair i, turned by
    the angle pos * base^(-2i / dims)."""
    out = vec.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        u, v = float(vec[2 * i]), float(vec[2 * i + 1])
        out[2 * i] = u * math.cos(a) - v * math.sin(a)
        out[2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def retention(h, W, m, eps):
    """Linear attention with one fixed decay per head, no normaliser.  h [T, width] -> [T, width]."""
    T = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    q = (h @ W("q").T).view(T, H, d)
    k = (h @ W("k").T).view(T, H, d) * d ** -0.5
    v = (h @ W("v").T).view(T, H, vd)
    gate = silu(h @ W("g").T)
    out = torch.zeros(T, H * vd, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, vd, dtype=F64)
        lam = float(m["decay"][hh])
        for t in range(T):
            S = lam * S + torch.outer(k[t, hh], v[t, hh])
            out[t, hh * vd:(hh + 1) * vd] = rms_unit(S.T @ q[t, hh], eps)
    return (out * gate) @ W("o").T


def chunk_attention(h, W, m, eps):
    """Softmax attention inside aligned blocks of mask.size positions: query i sees key j when j <= i and both lie in
    the same block.  Partial rotary on adjacent pairs, a temperature per head, a sigmoid gate per head."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    C, scale = m["mask"]["size"], m["scale"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = (h @ W("q").T).view(T, H, d)
    k = (h @ W("k").T).view(T, G, d)
    v = (h @ W("v").T).view(T, G, vd)
    temp = W("temp")
    hg = torch.sigmoid(h @ W("g").T)  # [T, H]
    out = torch.zeros(T, H, vd, dtype=F64)
    kr = [[rotate_pairs(k[t, g], t, rot["dims"], rot["base"]) for g in range(G)] for t in range(T)]
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            qi = rotate_pairs(q[i, hh], i, rot["dims"], rot["base"])
            lo = (i // C) * C
            sc = torch.stack([qi @ kr[j][g] for j in range(lo, i + 1)]) * scale * float(temp[hh])
            p = torch.softmax(sc, 0)
            o = torch.zeros(vd, dtype=F64)
            for n, j in enumerate(range(lo, i + 1)):
                o = o + p[n] * v[j, g]
            out[i, hh] = o * hg[i, hh]
    return out.reshape(T, H * vd) @ W("o").T


def ssm(h, W, m, eps):
    """Selective state-space mixer (scalar decay per head and step), causal depthwise convolution in front, gated
    grouped RMS norm behind."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    taps, ng = m["conv"], m["norm_groups"]
    inner = H * P
    p = h @ W("in").T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    cw, cb = W("conv"), W("conv.b")
    ch = xbc.shape[1]
    conv = torch.zeros(T, ch, dtype=F64)
    for t in range(T):
        acc = cb.clone()
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                acc = acc + cw[:, j] * xbc[s]
        conv[t] = silu(acc)
    x = conv[:, :inner].view(T, H, P)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    Cm = conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W("dt_bias"))
    A = -torch.exp(W("A_log"))
    D = W("D")
    y = torch.zeros(T, H, P, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = torch.exp(A[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ Cm[t, g] + D[hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * W("norm")
    return y @ W("o").T


def expert(h, W, prefix):
    return (silu(h @ W(prefix + "gate").T) * (h @ W(prefix + "up").T)) @ W(prefix + "down").T


def moe(h, W, f):
    """Routed experts (softmax scores, group-limited choice, scores as weights) plus a gated shared expert."""
    T = h.shape[0]
    r = f["router"]
    E, top = r["experts"], r["top"]
    grp = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.softmax(h @ W("router").T, -1)
    out = torch.zeros(T, h.shape[1], dtype=F64)
    per = E // grp["count"]
    for t in range(T):
        best = sorted(range(grp["count"]), key=lambda g: -float(s[t, g * per:(g + 1) * per].max()))[: grp["keep"]]
        allowed = [e for e in range(E) if e // per in best]
        chosen = sorted(allowed, key=lambda e: -float(s[t, e]))[:top]
        for e in chosen:
            out[t] = out[t] + s[t, e] * expert(h[t:t + 1], W, f"e{e}.")[0]
    if f.get("shared") is not None:
        out = out + torch.sigmoid(h @ W("shared.sg").T) * expert(h, W, "shared.")
    return out


MIXERS = {"retention": retention, "attention": chunk_attention, "mamba2": ssm}


def layer_runs(cfg):
    """[(layer, first of its pass)] in execution order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for _ in range(times if b > a else 0):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def logits_and_taps(cfg, sd, toks):
    """-> (logits [T, vocab], residual after every layer run [runs, T, width]), float64."""
    sd = {k: v.to(F64) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x0 = sd["embed"][torch.tensor(toks)]
    x = x0.clone()
    taps = []
    for li, first in layer_runs(cfg):
        L = cfg["layers"][li]
        if first:
            x = torch.cat([x, x0], -1) @ sd["loop.in"].T
        h = rms_unit(x, eps) * sd[f"l{li}.norm1"]
        y = MIXERS[L["type"]](h, lambda n, li=li: sd[f"l{li}.mix.{n}"], L["mixer"], eps)
        if L.get("mlp") is not None:
            y = y + moe(h, lambda n, li=li: sd[f"l{li}.mlp.{n}"], L["mlp"])
        x = x + y
        taps.append(x.clone())
    h = rms_unit(x, eps) * sd["final.norm"]
    return h @ sd["head"].T, torch.stack(taps)


def forward(cfg, sd, toks):
    return logits_and_taps(cfg, sd, toks)[0]


# ------------------------------------------------------------------------------------------------ test models
def make_config(kinds=("retention", "attention", "mamba2", "attention"), loop=(1, 3, 2), no_mlp=(), vocab=96, width=48,
                heads=4, kv_heads=2, dim=16, vdim=8, chunk=7, rot_dims=8, rot_base=100.0, scale=0.3,
                ret_heads=3, ret_dim=8, ret_vdim=12, decay=None,
                ssm_heads=4, ssm_vdim=6, ssm_state=10, ssm_groups=2, ssm_norm_groups=3, taps=4,
                experts=6, top=2, groups=(3, 2), ff=20, shared_ff=28, eps=1e-5):
    decay = list(decay) if decay is not None else [1.0 - 2.0 ** (-2 - 2 * i) for i in range(ret_heads)]
    layers = []
    for i, kind in enumerate(kinds):
        if kind == "retention":
            m = {"heads": ret_heads, "dim": ret_dim, "vdim": ret_vdim, "decay": decay}
        elif kind == "attention":
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                 "mask": {"size": chunk}, "rot": {"dims": rot_dims, "base": rot_base}}
        else:
            m = {"heads": ssm_heads, "vdim": ssm_vdim, "state": ssm_state, "groups": ssm_groups,
                 "norm_groups": ssm_norm_groups, "conv": taps}
        mlp = None if i in no_mlp else {
            "kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": groups[0], "keep": groups[1]}},
            "shared": None if shared_ff is None else {"ff": shared_ff}}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    return {"architecture": "Leripel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
            "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}


def make_weights(cfg, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(1234 + seed)
    W = cfg["width"]

    def r(*shape, s=None):
        s = 1.0 / math.sqrt(shape[-1]) if s is None else s
        return (torch.randn(*shape, generator=g) * s).to(dtype)

    def around(v, n, s=0.1):
        return (v + s * torch.randn(n, generator=g)).to(dtype)

    sd = {"embed": r(cfg["vocab"], W, s=1.0), "head": r(cfg["vocab"], W), "final.norm": around(1.0, W)}
    loop = cfg.get("loop") or {}
    if loop.get("stop", 0) > loop.get("start", 0):
        sd["loop.in"] = (torch.cat([torch.eye(W), 0.3 * torch.eye(W)], 1) + 0.4 * torch.randn(W, 2 * W, generator=g)
                         / math.sqrt(W)).to(dtype)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        sd[p + "norm1"] = around(1.0, W)
        if L["type"] == "retention":
            H, d, vd = m["heads"], m["dim"], m["vdim"]
            sd.update({p + "mix.q": r(H * d, W), p + "mix.k": r(H * d, W), p + "mix.v": r(H * vd, W),
                       p + "mix.g": r(H * vd, W), p + "mix.o": r(W, H * vd)})
        elif L["type"] == "attention":
            H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd.update({p + "mix.q": r(H * d, W), p + "mix.k": r(G * d, W), p + "mix.v": r(G * vd, W),
                       p + "mix.temp": around(1.0, H, 0.3), p + "mix.g": r(H, W), p + "mix.o": r(W, H * vd)})
        else:
            H, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, ch = H * P, H * P + 2 * G * N
            sd.update({p + "mix.in": r(2 * inner + 2 * G * N + H, W), p + "mix.conv": r(ch, K, s=0.5),
                       p + "mix.conv.b": r(ch, s=0.2), p + "mix.dt_bias": r(H, s=1.0),
                       p + "mix.A_log": (torch.rand(H, generator=g) * 2.0 - 1.5).to(dtype), p + "mix.D": around(1.0, H, 0.3),
                       p + "mix.norm": around(1.0, inner), p + "mix.o": r(W, inner)})
        f = L.get("mlp")
        if f is not None:
            F = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                sd.update({p + f"mlp.e{e}.gate": r(F, W), p + f"mlp.e{e}.up": r(F, W), p + f"mlp.e{e}.down": r(W, F)})
            sd[p + "mlp.router"] = r(f["router"]["experts"], W, s=2.0 / math.sqrt(W))
            if f.get("shared") is not None:
                Fs = f["shared"]["ff"]
                sd.update({p + "mlp.shared.gate": r(Fs, W), p + "mlp.shared.up": r(Fs, W),
                           p + "mlp.shared.down": r(W, Fs), p + "mlp.shared.sg": r(1, W)})
    return sd
