"""Leripel: a decoder whose sublayers run side by side, with three sequence mixers and a mixture of experts, on the
paged-KV engine.

The layer list is data (models/configs.py HybridConfig, arch "leripel").  A layer reads ONE RMS norm of the fp32
residual x and adds both sublayers' outputs at once: x <- x + (mixer(h) + ff(h)), h = norm(x).  A span of layers
may run several times with shared weights; every run of a layer has its own K/V cache or recurrent state, and every
pass of the span starts with x <- W_in [x; embedding].

Mixers:
  "retention"  linear attention with a fixed decay per head and an fp32 [dim, vdim] state per head, k scaled by
               dim^-1/2, no softmax and no denominator; every head's output is divided by its RMS and gated by SiLU
               of a projection                                       [grag_decay_attn_scan, grag_gated_rmsnorm]
  "attention"  softmax attention inside aligned blocks of positions, GQA, rotary on adjacent pairs of the first
               rot dims, a temperature per head, one sigmoid output gate per head
                                                                     [grag_rope_vnorm_store, grag_sink_attn_*]
  "mamba2"     state-space mixer: causal convolution + SiLU over x | B | C, a scalar input-dependent decay per head
               and step, an fp32 [state, vdim] state per head, the output gated by SiLU(z) and then RMS-normed in
               parts                                  [grag_causal_conv, grag_ssm_scan, grag_gated_rmsnorm]
Feed-forward: a router (fp32 logits and softmax scores; the best `top` experts of the best `keep` groups, weighted
by their scores as they are) over SiLU-gated experts that run as two grouped GEMMs over the (token, expert) pairs
[grag_moe_route, grag_moe_align, grag_moe_gemm], and a shared expert with a sigmoid gate per token.

Per layer the mixer's input projections are one GEMM, and the layer boundary is one kernel: residual += mixer +
gate * shared + sum of weighted experts, then the next norm [grag_residual_rmsnorm].  Activations are bf16 (or fp32
end to end with dtype=torch.float32: the GEMMs then run in true fp32); the residual, norms, positions, scores,
softmax weights, router, decays, step sizes and states are fp32 in both.
"""
from __future__ import annotations

import math

import torch

from ..ops.attention import AttnMetadata, sink_attention
from ..ops.elementwise import clamped_glu, rope_table, rope_vnorm_store
from ..ops.linear import linear
from ..ops.moe import moe_experts, moe_route
from ..ops.norm import embed_gather_f32, residual_rmsnorm
from ..ops.recurrent import causal_conv, decay_attention, gated_rmsnorm, ssm_scan
from ..parallel.comm import Group
from .configs import HybridConfig


class _Layer:
    __slots__ = ("spec", "kind", "norm", "wp", "off", "wo", "decay", "temp", "rope", "convw", "convb", "dtb", "alog",
                 "skip", "ynorm", "wr", "wgu", "wd", "wsgu", "wsd")


def _pad8(t: torch.Tensor) -> torch.Tensor:
    """Rows padded with zeros to a multiple of 8 (fused projection matrices: 16-byte output rows)."""
    pad = -t.shape[0] % 8
    return t if not pad else torch.cat([t, torch.zeros(pad, *t.shape[1:], dtype=t.dtype)], 0)


def init_state_dict(cfg: HybridConfig, seed: int = 0, std: float | None = None) -> dict:
    """Random weights under the checkpoint's tensor names (bf16; benches and tests -- not a trained model)."""
    g = torch.Generator().manual_seed(seed * 1000003 + 91)
    W = cfg.hidden_size

    def r(*shape, s=None):
        s = (1.0 / math.sqrt(shape[-1])) if s is None else s
        return (torch.randn(*shape, generator=g) * (std or s)).to(torch.bfloat16)

    def around(v, n, s=0.1):
        return (v + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    sd = {"embed": r(cfg.vocab_size, W, s=1.0), "head": r(cfg.vocab_size, W), "final.norm": around(1.0, W)}
    if cfg.loop_stop > cfg.loop_start:
        sd["loop.in"] = (torch.cat([torch.eye(W), 0.3 * torch.eye(W)], 1)
                         + 0.3 * torch.randn(W, 2 * W, generator=g) / math.sqrt(W)).to(torch.bfloat16)
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        a, kind = L.mixer.spec, L.mixer.kind
        sd[p + "norm1"] = around(1.0, W)
        if kind == "retention":
            sd.update({p + "mix.q": r(a.heads * a.dim, W), p + "mix.k": r(a.heads * a.dim, W),
                       p + "mix.v": r(a.heads * a.vdim, W), p + "mix.g": r(a.heads * a.vdim, W),
                       p + "mix.o": r(W, a.heads * a.vdim)})
        elif kind == "attention":
            sd.update({p + "mix.q": r(a.heads * a.dim, W), p + "mix.k": r(a.kv_heads * a.dim, W),
                       p + "mix.v": r(a.kv_heads * a.vdim, W), p + "mix.temp": around(1.0, a.heads, 0.2),
                       p + "mix.g": r(a.heads, W), p + "mix.o": r(W, a.heads * a.vdim)})
        else:
            ch = a.conv_channels
            sd.update({p + "mix.in": r(2 * a.inner + 2 * a.groups * a.state + a.heads, W),
                       p + "mix.conv": r(ch, a.taps, s=0.5), p + "mix.conv.b": r(ch, s=0.2),
                       p + "mix.dt_bias": r(a.heads, s=1.0),
                       p + "mix.A_log": (torch.rand(a.heads, generator=g) * 2.0 - 1.5).to(torch.bfloat16),
                       p + "mix.D": around(1.0, a.heads, 0.3), p + "mix.norm": around(1.0, a.inner),
                       p + "mix.o": r(W, a.inner)})
        f = L.mlp
        if f is not None:
            for e in range(f.experts):
                sd.update({p + f"mlp.e{e}.gate": r(f.ff, W), p + f"mlp.e{e}.up": r(f.ff, W),
                           p + f"mlp.e{e}.down": r(W, f.ff)})
            sd[p + "mlp.router"] = r(f.experts, W, s=2.0 / math.sqrt(W))
            if f.shared_ff:
                sd.update({p + "mlp.shared.gate": r(f.shared_ff, W), p + "mlp.shared.up": r(f.shared_ff, W),
                           p + "mlp.shared.down": r(W, f.shared_ff), p + "mlp.shared.sg": r(1, W)})
    return sd


class LeripelModel:
    has_state = True  # recurrent state per sequence slot: the engine allocates it and never reuses cached prefixes

    def __init__(self, cfg: HybridConfig, device="cuda", dtype=torch.bfloat16, tp: Group | None = None,
                 seed: int = 0, state_dict: dict | None = None, init_std: float | None = None):
        assert cfg.arch == "leripel", cfg.arch
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or Group([0])
        if not self.tp.trivial:
            raise NotImplementedError("the Leripel decoder runs on one GPU per replica (no tensor parallelism)")
        # the engine sizes the decode attention's split-KV scratch (hq * head_dim floats per row and split) and
        # picks its split plan (hkv) from these: the widest attention among the layers
        att = [L.mixer.spec for L in cfg.layers if L.mixer.kind == "attention"]
        self.hq = max([a.heads for a in att], default=1)
        self.hkv = min([a.kv_heads for a in att], default=1)
        self.head_dim = max([a.vdim for a in att], default=1)
        self.runs = cfg.layer_runs()
        self.looped = cfg.loop_stop > cfg.loop_start
        self._tables: dict = {}
        self._max_pos = 0
        self._load(state_dict if state_dict is not None else init_state_dict(cfg, seed, init_std))
        self.prepare(4096)

    # ------------------------------------------------------------------ weights
    def _load(self, sd: dict):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        W = cfg.hidden_size

        def expect(name, *shape):
            if name not in sd:
                raise KeyError(f"the checkpoint has no tensor {name!r}")
            if tuple(sd[name].shape) != shape:
                raise ValueError(f"{name}: expected {list(shape)}, found {list(sd[name].shape)}")
            return sd[name]

        def act(t):  # a GEMM operand: the activation dtype
            return t.to(device=dev, dtype=dt).contiguous()

        def fused(*parts, pad=True):  # (name, rows) ... -> one matrix, rows fused (and padded to a multiple of 8)
            t = torch.cat([expect(n, rows, W) for n, rows in parts], 0)
            return act(_pad8(t) if pad else t)

        def f32(name, *shape):
            return expect(name, *shape).to(device=dev, dtype=torch.float32).contiguous()

        self.embed = act(expect("embed", cfg.vocab_size, W))
        # LM head rows padded to a multiple of 8: the sampler reads logit rows 8 at a time (zero rows, cut off
        # again in compute_logits)
        self.head = act(_pad8(expect("head", cfg.vocab_size, W)))
        self.final_norm = f32("final.norm", W)
        self.w_in = act(expect("loop.in", W, 2 * W)) if self.looped else None
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p, m = f"l{i}.", f"l{i}.mix."
            L = _Layer()
            for n in _Layer.__slots__:
                setattr(L, n, None)
            L.spec, L.kind = spec, spec.mixer.kind
            a = spec.mixer.spec
            L.norm = f32(p + "norm1", W)
            if L.kind == "retention":
                qk, vv = a.heads * a.dim, a.heads * a.vdim
                L.wp = fused((m + "q", qk), (m + "k", qk), (m + "v", vv), (m + "g", vv))
                L.off = (0, qk, 2 * qk, 2 * qk + vv)
                L.wo = act(expect(m + "o", W, vv))
                L.decay = torch.tensor(a.decay, dtype=torch.float32, device=dev)
            elif L.kind == "attention":
                q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
                L.wp = fused((m + "q", q), (m + "k", k), (m + "v", v), (m + "g", a.heads))
                L.off = (0, q, q + k, q + k + v)
                L.wo = act(expect(m + "o", W, a.heads * a.vdim))
                L.temp = f32(m + "temp", a.heads)
                L.rope = (a.rot_dims, a.rot_base) if a.rot_dims else None
            else:
                ch = a.conv_channels
                L.wp = fused((m + "in", 2 * a.inner + 2 * a.groups * a.state + a.heads))
                L.off = (0, a.inner, a.inner + ch)  # z | x B C | dt
                L.wo = act(expect(m + "o", W, a.inner))
                L.convw, L.convb = f32(m + "conv", ch, a.taps), f32(m + "conv.b", ch)
                L.dtb, L.alog, L.skip = f32(m + "dt_bias", a.heads), f32(m + "A_log", a.heads), f32(m + "D", a.heads)
                L.ynorm = f32(m + "norm", a.inner)
            f = spec.mlp
            if f is not None:
                f_ = p + "mlp."
                rows = [expect(f_ + "router", f.experts, W)]
                if f.shared_ff:
                    rows.append(expect(f_ + "shared.sg", 1, W))
                    L.wsgu = fused((f_ + "shared.gate", f.shared_ff), (f_ + "shared.up", f.shared_ff), pad=False)
                    L.wsd = act(expect(f_ + "shared.down", W, f.shared_ff))
                L.wr = torch.cat(rows, 0).to(device=dev, dtype=torch.float32).contiguous()  # fp32 router (+ gate row)
                L.wgu = act(torch.stack([torch.cat([expect(f_ + f"e{e}.gate", f.ff, W), expect(f_ + f"e{e}.up", f.ff, W)], 0)
                                         for e in range(f.experts)], 0))
                L.wd = act(torch.stack([expect(f_ + f"e{e}.down", W, f.ff) for e in range(f.experts)], 0))
            self.layers.append(L)

    def prepare(self, max_len: int) -> None:
        """Rotary tables for positions below ``max_len`` (the engine calls this with its max_model_len before any
        step or graph capture; the design itself has no position limit)."""
        if max_len <= self._max_pos:
            return
        self._max_pos = max_len
        self._tables = {}
        for L in self.layers:
            if L.rope is not None and L.rope not in self._tables:
                self._tables[L.rope] = rope_table(max_len, L.rope[0], L.rope[1], self.device)

    def param_bytes(self) -> int:
        n = 0
        for t in [self.embed, self.head, self.w_in] + [x for L in self.layers
                                                       for x in (L.wp, L.wo, L.wgu, L.wd, L.wsgu, L.wsd, L.wr)]:
            if t is not None:
                n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ cache and state
    def kv_bytes_per_block(self, block_size: int) -> int:
        n = 0
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            if m.kind == "attention":
                n += m.spec.kv_heads * (m.spec.dim + m.spec.vdim)
        return max(1, n * block_size) * torch.finfo(self.dtype).bits // 8

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One (K [blocks, G, BS, dim], V [blocks, G, BS, vdim]) pair per run of an attention layer (None for the
        others); a looped layer has one pair per pass."""
        caches = []
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            a = m.spec
            z = dict(dtype=self.dtype, device=self.device)
            caches.append((torch.zeros(num_blocks, a.kv_heads, block_size, a.dim, **z),
                           torch.zeros(num_blocks, a.kv_heads, block_size, a.vdim, **z))
                          if m.kind == "attention" else None)
        return caches

    def state_bytes_per_slot(self) -> int:
        n = 0
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            a = m.spec
            if m.kind == "retention":
                n += 4 * a.heads * a.dim * a.vdim
            elif m.kind == "mamba2":
                n += 4 * a.heads * a.state * a.vdim + (a.taps - 1) * a.conv_channels * torch.finfo(self.dtype).bits // 8
        return n

    def allocate_state(self, num_slots: int):
        """Per run of a layer: retention -> an fp32 pool [slots, heads, dim, vdim]; the state-space mixer -> (the
        convolution's last taps - 1 inputs [slots, taps - 1, channels] in the activation type, an fp32 pool
        [slots, heads, state, vdim]); attention -> None."""
        pools = []
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            a = m.spec
            if m.kind == "retention":
                pools.append(torch.zeros(num_slots, a.heads, a.dim, a.vdim, dtype=torch.float32, device=self.device))
            elif m.kind == "mamba2":
                pools.append((torch.zeros(num_slots, a.taps - 1, a.conv_channels, dtype=self.dtype, device=self.device),
                              torch.zeros(num_slots, a.heads, a.state, a.vdim, dtype=torch.float32, device=self.device)))
            else:
                pools.append(None)
        return pools

    # ------------------------------------------------------------------ forward
    def _mixer(self, L, h, positions, meta: AttnMetadata, kv, state):
        a, eps = L.spec.mixer.spec, self.cfg.norm_eps
        p = linear(h, L.wp)
        T = h.shape[0]
        if L.kind == "retention":
            qo, ko, vo, go = L.off
            o = decay_attention(p, qo, ko, vo, L.decay, state, meta, a.heads, a.dim, a.vdim, act=False,
                                k_scale=a.dim ** -0.5)
            y = torch.empty(T, a.heads * a.vdim, dtype=h.dtype, device=h.device)
            gated_rmsnorm(o, None, p, go, eps, y, groups=a.heads, gate="silu")
            return linear(y, L.wo)
        if L.kind == "attention":
            qo, ko, vo, go = L.off
            kc, vc = kv
            q = rope_vnorm_store(p, qo, ko, vo, positions, self._tables[L.rope] if L.rope else None, meta.slot_mapping,
                                 kc, vc, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, eps, interleaved=True,
                                 vnorm=False)
            y = sink_attention(q, kc, vc, meta, a.scale, None, head_scale=L.temp, head_gate=p[:, go:go + a.heads],
                               chunk=a.chunk)
            return linear(y, L.wo)
        zo, xo, dto = L.off
        cstate, sstate = state
        xbc = causal_conv(p, xo, L.convw, L.convb, cstate, meta)
        o = ssm_scan(xbc, p, dto, L.dtb, L.alog, L.skip, sstate, meta, a.heads, a.groups, a.state, a.vdim)
        y = torch.empty(T, a.inner, dtype=h.dtype, device=h.device)
        gated_rmsnorm(o, L.ynorm, p, zo, eps, y, groups=a.norm_groups, gate="silu", gate_first=True)
        return linear(y, L.wo)

    def _ff(self, L, h):
        """-> the boundary's feed-forward addends (shared output, its gate [T], experts' outputs [T, top, W], their
        weights [T, top])."""
        f = L.spec.mlp
        ids, wts, sgate = moe_route(h, L.wr, f.experts, f.top, f.groups, f.keep)
        e = moe_experts(h, ids, L.wgu, L.wd)
        b = None
        if L.wsgu is not None:
            b = linear(clamped_glu(linear(h, L.wsgu), None, 1.0, 0.0), L.wsd)
        return b, sgate, e, wts

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta: AttnMetadata, kv_caches,
                state=None, taps: list | None = None) -> torch.Tensor:
        """-> final-normed hidden [T, W].  ``state``: the pools of allocate_state (meta.state_slots names each
        sequence's slot).  ``taps``: if a list, the residual after every layer run is appended."""
        if state is None or meta.state_slots is None:
            raise ValueError("this model carries recurrent state: pass state pools and meta.state_slots")
        dt, eps, W = self.dtype, self.cfg.norm_eps, self.cfg.hidden_size
        x0 = embed_gather_f32(input_ids, self.embed)
        x, cat = x0, None
        if self.looped:  # [x | embedding] in the activation type: the input of every pass's re-entry projection
            x = x0.clone()
            cat = torch.empty(x0.shape[0], 2 * W, dtype=dt, device=x0.device)
            residual_rmsnorm(x0, out_dtype=dt, raw=cat[:, W:])
        pend = {}  # the previous layer's outputs, added at the next boundary
        for ri, (li, _, first) in enumerate(self.runs):
            L = self.layers[li]
            if first:
                residual_rmsnorm(x, **pend, out_dtype=dt, raw=cat[:, :W])
                pend = {"a": linear(cat, self.w_in), "keep": False}
            h = residual_rmsnorm(x, **pend, w=L.norm, eps=eps, out_dtype=dt)
            pend = {"a": self._mixer(L, h, positions, meta, kv_caches[ri], state[ri])}
            if L.wr is not None:
                b, sgate, e, wts = self._ff(L, h)
                pend.update(b=b, bcoef=sgate, e=e, ecoef=wts)
            if taps is not None:
                residual_rmsnorm(x, **pend, out_dtype=dt)
                pend = {}
                taps.append(x.clone())
        return residual_rmsnorm(x, **pend, w=self.final_norm, eps=eps, out_dtype=dt)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [B, W] -> logits [B, vocab] (a view of the padded GEMM output)."""
        return linear(hidden, self.head)[:, : self.cfg.vocab_size]
