"""Pubulix: a pre-norm decoder with two sliding-window attention mixers, an input convolution in front of every mixer,
sigmoid-gated residual branches and table-routed experts, on the paged-KV engine.

The layer list is data (models/configs.py HybridConfig, arch "pubulix").  With the fp32 residual x, the residual
multiplier m and RMS norms whose weight is ONE number,

    h = norm1(x);  x <- x + m * sigmoid(W_rg1 h + b_rg1) * mixer(h + conv(h))
    h = norm2(x);  x <- x + m * sigmoid(W_rg2 h + b_rg2) * experts(h)

conv is a causal per-channel convolution over time of ``conv_taps`` taps, without bias or activation; the last
taps - 1 normed inputs of every layer are the state a sequence carries besides its K/V cache
[grag_causal_conv, identity + residual form].  The embedding rows are multiplied by a constant, the logits go through
cap * tanh(logits / cap).

Mixers:
  "attention"         grouped-query softmax attention over the last ``window`` positions, rotary on halves of the
                      first rot dims, the scaled scores capped by softcap * tanh(score / softcap)
                                                          [grag_rope_vnorm_store, grag_sink_attn_* with window / softcap]
  "latent_attention"  softmax attention with a sink per head over the last ``window`` positions of a cached latent
                      plus one rotated key part shared by the heads (rotary on adjacent pairs).  The key expansion is
                      folded into the query projection when the weights are loaded (per head W_q' = [W_uk^T W_q,nope ;
                      W_q,rot]), so a step attends straight to the cache: one kv head whose key rows are latent |
                      rotated part and whose value rows are the head of the same rows.  The attended latents go through
                      one small value matrix per head, the result is multiplied by sigmoid(W_g input), then W_o.  A layer
                      with ``kv_from`` stores nothing: it attends to an earlier latent layer's cache with its own
                      queries, value matrices, window and sink
                                     [grag_latent_rope_store, grag_sink_attn_*, grag_moe_gemm with the heads as experts]
Feed-forward: the experts of a token are the row of its token id in an integer table, each weighing 1 / top
[grag_moe_table_route]; an expert is g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, +-limit), run
as two grouped GEMMs over the (token, expert) pairs [grag_moe_align, grag_moe_gemm].

Per layer the mixer's input projections are one GEMM (q | k | v, or q' | latent | gate), and every sublayer boundary
is one kernel: residual += m * sigmoid(gate + bias) * (branch output or the experts' weighted sum), then the next norm
[grag_residual_rmsnorm].  Activations are bf16 (or fp32 end to end with dtype=torch.float32: the GEMMs then run in
true fp32); the residual, norms, positions, angles, scores and softmax weights are fp32 in both.
"""
from __future__ import annotations

import math

import torch

from ..ops.attention import AttnMetadata, sink_attention
from ..ops.elementwise import latent_rope_store, rope_table, rope_vnorm_store, tanh_cap_
from ..ops.linear import linear
from ..ops.moe import head_project, moe_experts, moe_table_route
from ..ops.norm import embed_gather_f32, residual_rmsnorm
from ..ops.recurrent import causal_conv
from ..parallel.comm import Group
from .configs import HybridConfig

EXPERT_ALPHA, EXPERT_SHIFT = 1.702, 1.0  # the experts' unit: g sigmoid(1.702 g) (u + 1)


class _Layer:
    __slots__ = ("spec", "kind", "norm1", "norm2", "convw", "rg1", "rg1b", "rg2", "rg2b", "wp", "off", "wo", "wuv",
                 "sink", "ckn", "rope", "src", "table", "wgu", "wd")


def _pad8(t: torch.Tensor) -> torch.Tensor:
    """Rows padded with zeros to a multiple of 8 (fused projection matrices: 16-byte output rows)."""
    pad = -t.shape[0] % 8
    return t if not pad else torch.cat([t, torch.zeros(pad, *t.shape[1:], dtype=t.dtype)], 0)


def init_state_dict(cfg: HybridConfig, seed: int = 0, std: float | None = None) -> dict:
    """Random weights under the checkpoint's tensor names (bf16, the expert tables int32; benches and tests -- not a
    trained model)."""
    g = torch.Generator().manual_seed(seed * 1000003 + 53)
    W = cfg.hidden_size

    def r(*shape, s=None):
        s = (1.0 / math.sqrt(shape[-1])) if s is None else s
        return (torch.randn(*shape, generator=g) * (std or s)).to(torch.bfloat16)

    def one(v=1.0, s=0.1):
        return (v + s * torch.randn((), generator=g)).to(torch.bfloat16)

    sd = {"embed": r(cfg.vocab_size, W, s=1.0), "head": r(cfg.vocab_size, W), "final.norm": one()}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        a, kind = L.mixer.spec, L.mixer.kind
        sd[p + "norm1"] = one()
        if cfg.conv_taps:
            sd[p + "canon1"] = r(W, cfg.conv_taps, s=0.3)
        sd[p + "rg1"], sd[p + "rg1.b"] = r(W, W), r(W, s=0.5)
        if kind == "attention":
            sd.update({p + "mix.q": r(a.heads * a.dim, W), p + "mix.k": r(a.kv_heads * a.dim, W),
                       p + "mix.v": r(a.kv_heads * a.vdim, W), p + "mix.o": r(W, a.heads * a.vdim)})
        else:
            sd.update({p + "mix.q": r(a.heads * (a.dim + a.rot_dim), W), p + "mix.uk": r(a.heads * a.dim, a.kv_rank),
                       p + "mix.uv": r(a.heads * a.vdim, a.kv_rank), p + "mix.sink": r(a.heads, s=1.0),
                       p + "mix.g": r(a.heads * a.vdim, W), p + "mix.o": r(W, a.heads * a.vdim)})
            if a.kv_from is None:
                sd[p + "mix.dkv"] = r(a.kv_rank + a.rot_dim, W)
                sd[p + "mix.dkv.norm"] = (1.0 + 0.1 * torch.randn(a.kv_rank, generator=g)).to(torch.bfloat16)
        f = L.mlp
        if f is not None:
            sd[p + "norm2"] = one()
            sd[p + "rg2"], sd[p + "rg2.b"] = r(W, W), r(W, s=0.5)
            for e in range(f.experts):
                sd.update({p + f"mlp.e{e}.gate": r(f.ff, W), p + f"mlp.e{e}.up": r(f.ff, W),
                           p + f"mlp.e{e}.down": r(W, f.ff)})
            sd[p + "mlp.table"] = torch.rand(cfg.vocab_size, f.experts, generator=g).argsort(1)[:, : f.top].to(torch.int32)
    return sd


class PubulixModel:
    has_state = True  # the input convolutions' last inputs per sequence slot: the engine allocates them and never
    #                   reuses cached prefixes

    def __init__(self, cfg: HybridConfig, device="cuda", dtype=torch.bfloat16, tp: Group | None = None,
                 seed: int = 0, state_dict: dict | None = None, init_std: float | None = None):
        assert cfg.arch == "pubulix", cfg.arch
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or Group([0])
        if not self.tp.trivial:
            raise NotImplementedError("the Pubulix decoder runs on one GPU per replica (no tensor parallelism)")
        if cfg.loop_stop > cfg.loop_start:
            raise ValueError("the Pubulix design has no looped layers")
        # the engine sizes the decode attention's split-KV scratch (hq * head_dim floats per row and split) and picks
        # its split plan (hkv) from these: the widest output rows among the layers (a latent layer's are kv_rank wide)
        rows = [(L.mixer.spec.heads, L.mixer.spec.kv_heads, L.mixer.spec.vdim) if L.mixer.kind == "attention"
                else (L.mixer.spec.heads, 1, L.mixer.spec.kv_rank) for L in cfg.layers]
        self.hq = max([h for h, _, _ in rows], default=1)
        self.hkv = min([g for _, g, _ in rows], default=1)
        self.head_dim = max([v for _, _, v in rows], default=1)
        self.runs = cfg.layer_runs()
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

        def f32(name, *shape):
            return expect(name, *shape).to(device=dev, dtype=torch.float32).contiguous()

        def scalar_norm(name):  # one number for all coordinates: spread to the row the norm kernels multiply by
            if name not in sd or sd[name].numel() != 1:
                raise ValueError(f"{name}: expected one number")
            return torch.full((W,), float(sd[name].float().reshape(())), dtype=torch.float32, device=dev)

        self.embed = act(expect("embed", cfg.vocab_size, W))
        # LM head rows padded to a multiple of 8: the sampler reads logit rows 8 at a time (zero rows, cut off
        # again in compute_logits)
        self.head = act(_pad8(expect("head", cfg.vocab_size, W)))
        self.final_norm = scalar_norm("final.norm")
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p, m = f"l{i}.", f"l{i}.mix."
            L = _Layer()
            for n in _Layer.__slots__:
                setattr(L, n, None)
            L.spec, L.kind = spec, spec.mixer.kind
            a = spec.mixer.spec
            L.norm1 = scalar_norm(p + "norm1")
            if cfg.conv_taps:
                L.convw = f32(p + "canon1", W, cfg.conv_taps)
            L.rg1, L.rg1b = act(expect(p + "rg1", W, W)), f32(p + "rg1.b", W)
            if L.kind == "attention":
                q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
                L.wp = act(_pad8(torch.cat([expect(m + "q", q, W), expect(m + "k", k, W), expect(m + "v", v, W)], 0)))
                L.off = (0, q, q + k)
                L.wo = act(expect(m + "o", W, a.heads * a.vdim))
                L.rope = (a.rot_dims, a.rot_base) if a.rot_dims else None
            else:
                H, d, r, vd, R = a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank
                # the key expansion folded into the queries, once, in float64: per head the unrotated query rows go
                # through W_uk^T (scores against the latent itself), the rotated rows are kept
                wq = expect(m + "q", H * (d + r), W).double().view(H, d + r, W)
                uk = expect(m + "uk", H * d, R).double().view(H, d, R)
                wqf = torch.cat([torch.einsum("hdr,hdw->hrw", uk, wq[:, :d]), wq[:, d:]], 1).reshape(H * (R + r), W)
                parts, L.off = [wqf], [0, None, None]
                if a.kv_from is None:
                    L.off[1] = H * (R + r)
                    parts.append(expect(m + "dkv", R + r, W).double())
                    L.ckn = f32(m + "dkv.norm", R)
                L.off[2] = sum(t.shape[0] for t in parts)
                parts.append(expect(m + "g", H * vd, W).double())
                L.wp = act(_pad8(torch.cat(parts, 0)))
                L.wuv = act(expect(m + "uv", H * vd, R).view(H, vd, R))
                L.wo = act(expect(m + "o", W, H * vd))
                L.sink = f32(m + "sink", H)
                L.rope = (r, a.rot_base)
                L.src = i if a.kv_from is None else a.kv_from
            f = spec.mlp
            if f is not None:
                f_ = p + "mlp."
                L.norm2 = scalar_norm(p + "norm2")
                L.rg2, L.rg2b = act(expect(p + "rg2", W, W)), f32(p + "rg2.b", W)
                t = expect(f_ + "table", cfg.vocab_size, f.top)
                if t.dtype.is_floating_point or int(t.min()) < 0 or int(t.max()) >= f.experts:
                    raise ValueError(f"{f_}table must hold expert numbers below {f.experts}")
                L.table = t.to(device=dev, dtype=torch.int32).contiguous()
                L.wgu = act(torch.stack([torch.cat([expect(f_ + f"e{e}.gate", f.ff, W), expect(f_ + f"e{e}.up", f.ff, W)], 0)
                                         for e in range(f.experts)], 0))
                L.wd = act(torch.stack([expect(f_ + f"e{e}.down", W, f.ff) for e in range(f.experts)], 0))
            self.layers.append(L)
        # the tables of all layers with the same number of choices side by side: one routing launch per step serves
        # them all (a layer's tables entry becomes (stack, row))
        groups: dict = {}
        for L in self.layers:
            if L.table is not None:
                groups.setdefault(L.table.shape[1], []).append(L)
        self.route_tables = {}
        for top, Ls in groups.items():
            self.route_tables[top] = torch.stack([L.table for L in Ls], 0).contiguous()
            for k, L in enumerate(Ls):
                L.table = (top, k)

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
        for t in [self.embed, self.head] + [x for L in self.layers
                                            for x in (L.wp, L.wo, L.wuv, L.rg1, L.rg2, L.wgu, L.wd)] + list(self.route_tables.values()):
            if t is not None:
                n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ cache and state
    def _kv_row(self, li: int) -> int:
        """Numbers cached per token by a layer (0: it reads another layer's cache)."""
        m = self.cfg.layers[li].mixer
        if m.kind == "attention":
            return m.spec.kv_heads * (m.spec.dim + m.spec.vdim)
        return m.spec.kv_rank + m.spec.rot_dim if m.spec.kv_from is None else 0

    def kv_bytes_per_block(self, block_size: int) -> int:
        n = sum(self._kv_row(li) for li, _, _ in self.runs) * block_size
        return max(1, n) * torch.finfo(self.dtype).bits // 8

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One (K, V) pair per layer.  Attention: K [blocks, G, BS, dim], V [blocks, G, BS, vdim].  Latent layers: one
        tensor [blocks, 1, BS, kv_rank + rot_dim] (latent | rotated part); its values are the latents, so V is a view
        of the first kv_rank columns of the same rows.  A layer that attends to another layer's cache gets that
        layer's pair."""
        caches = []
        z = dict(dtype=self.dtype, device=self.device)
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            a = m.spec
            if m.kind == "attention":
                caches.append((torch.zeros(num_blocks, a.kv_heads, block_size, a.dim, **z),
                               torch.zeros(num_blocks, a.kv_heads, block_size, a.vdim, **z)))
            elif a.kv_from is None:
                k = torch.zeros(num_blocks, 1, block_size, a.kv_rank + a.rot_dim, **z)
                caches.append((k, k[..., : a.kv_rank]))
            else:
                caches.append(caches[a.kv_from])
        return caches

    def state_bytes_per_slot(self) -> int:
        taps = self.cfg.conv_taps
        return len(self.runs) * max(0, taps - 1) * self.cfg.hidden_size * torch.finfo(self.dtype).bits // 8

    def allocate_state(self, num_slots: int):
        """Per layer the input convolution's last taps - 1 inputs [slots, taps - 1, width] in the activation type
        (None without a convolution)."""
        taps, W = self.cfg.conv_taps, self.cfg.hidden_size
        return [torch.zeros(num_slots, taps - 1, W, dtype=self.dtype, device=self.device) if taps else None
                for _ in self.runs]

    # ------------------------------------------------------------------ forward
    def _mixer(self, L, h, positions, meta: AttnMetadata, kv):
        a, eps = L.spec.mixer.spec, self.cfg.norm_eps
        p = linear(h, L.wp)
        kc, vc = kv
        if L.kind == "attention":
            qo, ko, vo = L.off
            q = rope_vnorm_store(p, qo, ko, vo, positions, self._tables[L.rope] if L.rope else None, meta.slot_mapping,
                                 kc, vc, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, eps, interleaved=False,
                                 vnorm=False)
            y = sink_attention(q, kc, vc, meta, a.scale, None, window=a.window, softcap=a.softcap)
            return linear(y, L.wo)
        qo, co, go = L.off
        q = latent_rope_store(p, qo, co, L.ckn, positions, self._tables[L.rope], meta.slot_mapping, kc, a.heads, eps,
                              interleaved=a.interleaved)
        o = sink_attention(q, kc, vc, meta, a.scale, L.sink, window=a.window)
        y = head_project(o, L.wuv, gate=p[:, go:go + a.heads * a.vdim])
        return linear(y, L.wo)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta: AttnMetadata, kv_caches,
                state=None, taps: list | None = None) -> torch.Tensor:
        """-> final-normed hidden [T, W].  ``state``: the pools of allocate_state (meta.state_slots names each
        sequence's slot).  ``taps``: if a list, the residual after every layer is appended."""
        cfg = self.cfg
        if cfg.conv_taps and (state is None or meta.state_slots is None):
            raise ValueError("this model carries convolution state: pass state pools and meta.state_slots")
        dt, eps, mult = self.dtype, cfg.norm_eps, cfg.residual_mult
        ids = input_ids.to(torch.int32).contiguous()
        x = embed_gather_f32(ids, self.embed, cfg.embed_scale)
        routes = {top: moe_table_route(ids, t) for top, t in self.route_tables.items()}  # every layer's experts
        pend = {}  # the previous sublayer's output and gate, added at the next boundary
        for ri, (li, _, _) in enumerate(self.runs):
            L = self.layers[li]
            h = residual_rmsnorm(x, **pend, w=L.norm1, eps=eps, out_dtype=dt)
            hin = causal_conv(h, 0, L.convw, None, state[ri], meta, act=False, residual=True) if cfg.conv_taps else h
            y = self._mixer(L, hin, positions, meta, kv_caches[ri])
            pend = {"a": y, "gate": linear(h, L.rg1), "gbias": L.rg1b, "mult": mult}
            f = L.spec.mlp
            if f is not None:
                h = residual_rmsnorm(x, **pend, w=L.norm2, eps=eps, out_dtype=dt)
                eids, wts = routes[L.table[0]][0][L.table[1]], routes[L.table[0]][1]
                e = moe_experts(h, eids, L.wgu, L.wd, f.limit, EXPERT_ALPHA, EXPERT_SHIFT)
                pend = {"e": e, "ecoef": wts, "gate": linear(h, L.rg2), "gbias": L.rg2b, "mult": mult}
            if taps is not None:
                residual_rmsnorm(x, **pend, out_dtype=dt)
                pend = {}
                taps.append(x.clone())
        return residual_rmsnorm(x, **pend, w=self.final_norm, eps=eps, out_dtype=dt)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [B, W] -> capped logits [B, vocab] (a view of the padded GEMM output)."""
        return tanh_cap_(linear(hidden, self.head)[:, : self.cfg.vocab_size], self.cfg.logit_softcap)
