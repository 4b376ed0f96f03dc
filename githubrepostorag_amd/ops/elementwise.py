"""Fused elementwise ops: QKV bias+RoPE+paged-KV store, SiLU*mul, bias+act,
pooling + L2 normalisation."""
from __future__ import annotations

import math

import torch

from ._lib import call, ptr

ACT_NONE, ACT_GELU, ACT_SILU, ACT_GELU_TANH = 0, 1, 2, 3


def rope_cos_sin(max_pos: int, head_dim: int, theta: float, device=None) -> torch.Tensor:
    """NeoX rotary table [max_pos, head_dim] fp32: cos in [:D/2], sin in [D/2:]."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos(), f.sin()], dim=-1).float().to(device)


def qkv_rope_kvstore_ref(qkv, bias, positions, cos_sin, slot_mapping, k_cache, v_cache, Hq, Hkv, D):
    T = qkv.shape[0]
    x = qkv.float()
    if bias is not None:
        x = (x + bias.float()).to(qkv.dtype).float()
    q = x[:, : Hq * D].view(T, Hq, D)
    k = x[:, Hq * D : (Hq + Hkv) * D].view(T, Hkv, D)
    v = x[:, (Hq + Hkv) * D : (Hq + 2 * Hkv) * D].view(T, Hkv, D)
    if cos_sin is not None:  # None: no rotary (GPT-2 absolute positions)
        cs = cos_sin[positions.long()]
        cos, sin = cs[:, : D // 2].unsqueeze(1), cs[:, D // 2 :].unsqueeze(1)

        def rot(t):
            a, b = t[..., : D // 2], t[..., D // 2 :]
            return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)

        q, k = rot(q), rot(k)
    if slot_mapping is not None and k_cache is not None:
        BS = k_cache.shape[2]
        sm = slot_mapping.long()
        ok = sm >= 0
        blk, off = sm[ok] // BS, sm[ok] % BS
        k_cache[blk, :, off] = k[ok].to(k_cache.dtype)
        v_cache[blk, :, off] = v[ok].to(v_cache.dtype)
    return q.to(qkv.dtype).contiguous()


def qkv_rope_kvstore(qkv, bias, positions, cos_sin, slot_mapping, k_cache, v_cache, Hq, Hkv, D):
    """Split packed QKV [T, (Hq+2Hkv)*D], add bias, apply NeoX RoPE to q/k
    (skipped when ``cos_sin`` is None), return q [T, Hq, D] and scatter k/v
    into the paged caches [blocks, Hkv, BS, D].  ``qkv`` may be the deferred fp32 split-K planes of the
    projection (ops/gemm.py SplitKPartial): the kernel then folds the split-K reduce into this pass."""
    from .gemm import SplitKPartial

    if isinstance(qkv, SplitKPartial):
        if not qkv.device.type == "cuda":
            qkv = qkv.materialize()
        else:
            T = qkv.M
            q = torch.empty(T, Hq, D, dtype=qkv.dtype, device=qkv.device)
            call("grag_qkv_rope_kvstore_planes", ptr(qkv.planes), qkv.S, qkv.N, ptr(bias), ptr(positions),
                 ptr(cos_sin), ptr(slot_mapping), ptr(q), ptr(k_cache), ptr(v_cache), T, Hq, Hkv, D,
                 k_cache.shape[2], *_bounds(k_cache, cos_sin, D))
            return q
    if not qkv.is_cuda:
        return qkv_rope_kvstore_ref(qkv, bias, positions, cos_sin, slot_mapping, k_cache, v_cache, Hq, Hkv, D)
    T = qkv.shape[0]
    q = torch.empty(T, Hq, D, dtype=qkv.dtype, device=qkv.device)
    BS = k_cache.shape[2]
    call("grag_qkv_rope_kvstore", ptr(qkv), qkv.stride(0), ptr(bias), ptr(positions), ptr(cos_sin),
         ptr(slot_mapping), ptr(q), ptr(k_cache), ptr(v_cache), T, Hq, Hkv, D, BS, *_bounds(k_cache, cos_sin, D))
    return q


def _bounds(k_cache, cos_sin, D) -> tuple[int, int]:
    """(KV slots, cos/sin rows): the kernel's index-guard limits for slot_mapping / positions."""
    nslots = 0 if k_cache is None else k_cache.shape[0] * k_cache.shape[2]
    npos = 0 if cos_sin is None else cos_sin.numel() // D
    return nslots, npos


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    I = gu.shape[-1] // 2
    if not gu.is_cuda:
        g, u = gu[..., :I].float(), gu[..., I:].float()
        return (torch.nn.functional.silu(g) * u).to(gu.dtype)
    gu = gu.contiguous()
    T = gu.numel() // (2 * I)
    out = torch.empty(*gu.shape[:-1], I, dtype=gu.dtype, device=gu.device)
    call("grag_silu_mul", ptr(gu), ptr(out), T, I)
    return out


def bias_act(x: torch.Tensor, b: torch.Tensor | None, act: int, inplace: bool = False) -> torch.Tensor:
    if not x.is_cuda:
        v = x.float() + (b.float() if b is not None else 0.0)
        if act == ACT_GELU:
            v = torch.nn.functional.gelu(v)
        elif act == ACT_SILU:
            v = torch.nn.functional.silu(v)
        elif act == ACT_GELU_TANH:
            v = torch.nn.functional.gelu(v, approximate="tanh")
        return v.to(x.dtype)
    x = x.contiguous()
    N = x.shape[-1]
    T = x.numel() // N
    y = x if inplace else torch.empty_like(x)
    call("grag_bias_act", ptr(x), ptr(b), ptr(y), T, N, act)
    return y


POOL_MEAN, POOL_CLS = 0, 1


def pool_l2norm_ref(hidden, starts, lengths, mode, normalize=True):
    """hidden [T, H] packed rows; sequence b = rows starts[b] .. +lengths[b]."""
    outs = []
    h = hidden.float()
    for st, ln in zip(starts.tolist(), lengths.tolist()):
        ln = max(1, ln)
        v = h[st] if mode == POOL_CLS else h[st:st + ln].mean(0)
        outs.append(v)
    v = torch.stack(outs) if outs else torch.zeros(0, hidden.shape[-1], device=hidden.device)
    if normalize:
        v = v / v.norm(dim=-1, keepdim=True).clamp_min(1e-12)
    return v


def pool_l2norm(hidden: torch.Tensor, starts: torch.Tensor, lengths: torch.Tensor, mode: int = POOL_MEAN,
                normalize: bool = True, want_bf16: bool = False):
    """Packed hidden rows [T, H] -> fp32 [B, H] (and a bf16 copy) pooled over
    each sequence (mean or CLS) and L2-normalised, in one kernel."""
    if not hidden.is_cuda:
        f = pool_l2norm_ref(hidden, starts, lengths, mode, normalize)
        return (f, f.to(torch.bfloat16)) if want_bf16 else f
    B, H = lengths.numel(), hidden.shape[-1]
    starts = starts.to(torch.int32).contiguous()
    lengths = lengths.to(torch.int32).contiguous()
    outf = torch.empty(B, H, dtype=torch.float32, device=hidden.device)
    outb = torch.empty(B, H, dtype=torch.bfloat16, device=hidden.device) if want_bf16 else None
    call("grag_pool_l2norm", ptr(hidden.contiguous()), ptr(starts), ptr(lengths), ptr(outf), ptr(outb), B, 0,
         H, mode, 1 if normalize else 0)
    return (outf, outb) if want_bf16 else outf


def softmax_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)


# ---------------------------------------------------------------------------------------------- partial rotary + value norm
def rope_table(max_pos: int, rot_dims: int, base: float, device=None) -> torch.Tensor:
    """[max_pos, rot_dims] fp32: cos(p f_i) in [:rot_dims/2], sin in [rot_dims/2:], f_i = base^(-2i/rot_dims);
    angles formed in float64 and rounded once."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    f = torch.outer(torch.arange(max_pos, dtype=torch.float64), torch.as_tensor(base, dtype=torch.float64) ** (-2.0 * i / max(1, rot_dims)))
    return torch.cat([f.cos(), f.sin()], dim=-1).float().to(device)


def rope_vnorm_store(proj: torch.Tensor, qoff: int, koff: int, voff: int, positions: torch.Tensor,
                     table: torch.Tensor, slot_mapping: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     H: int, G: int, d: int, vd: int, rot_dims: int, eps: float, interleaved: bool = False,
                     vnorm: bool = True) -> torch.Tensor:
    """From a fused projection ``proj`` [T, ld] (q heads at column qoff, k at koff, v at voff): rotate the first
    ``rot_dims`` dims of every q / k head (dim i paired with i + rot_dims/2; ``interleaved``: dim 2i with 2i + 1,
    pair i turned by the table's angle i), divide every v head by its root mean square (fp32; ``vnorm`` False: the
    values as they are), store k / v into the paged caches k_cache [blocks, G, BS, d] / v_cache [blocks, G, BS, vd]
    at ``slot_mapping`` (-1: not stored) and return q [T, H, d]."""
    T = proj.shape[0]
    BS = k_cache.shape[2]
    if not proj.is_cuda:
        x = proj.float()
        q = x[:, qoff:qoff + H * d].reshape(T, H, d).clone()
        k = x[:, koff:koff + G * d].reshape(T, G, d).clone()
        v = x[:, voff:voff + G * vd].reshape(T, G, vd)
        if rot_dims:
            h2 = rot_dims // 2
            cs = table[positions.long()]
            c, s = cs[:, None, :h2], cs[:, None, h2:]
            for t in (q, k):
                if interleaved:
                    a, b = t[..., 0:rot_dims:2].clone(), t[..., 1:rot_dims:2].clone()
                    t[..., 0:rot_dims:2] = a * c - b * s
                    t[..., 1:rot_dims:2] = b * c + a * s
                    continue
                a, b = t[..., :h2].clone(), t[..., h2:rot_dims].clone()
                t[..., :h2] = a * c - b * s
                t[..., h2:rot_dims] = b * c + a * s
        if vnorm:
            v = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        ok = slot_mapping >= 0
        sl = slot_mapping[ok].long()
        k_cache[sl // BS, :, sl % BS] = k[ok].to(k_cache.dtype)
        v_cache[sl // BS, :, sl % BS] = v[ok].to(v_cache.dtype)
        return q.to(proj.dtype)
    assert proj.stride(1) == 1 and k_cache.dtype == proj.dtype and v_cache.dtype == proj.dtype
    q = torch.empty(T, H, d, dtype=proj.dtype, device=proj.device)
    call("grag_rope_vnorm_store", ptr(proj), proj.stride(0), qoff, koff, voff, ptr(positions), ptr(table),
         0 if table is None else table.shape[0], ptr(slot_mapping), ptr(q), ptr(k_cache), ptr(v_cache), T, H, G, d, vd, rot_dims, BS,
         k_cache.shape[0] * BS, float(eps), 0 if proj.dtype == torch.bfloat16 else 1,
         (1 if interleaved else 0) | (0 if vnorm else 2))
    return q


def clamped_glu(gu: torch.Tensor, limit: float | None, alpha: float = 1.702, shift: float = 1.0) -> torch.Tensor:
    """gu [T, 2F] (gate | up) -> g sigmoid(alpha g) (u + shift) with g = min(gate, limit), u = clamp(up, +-limit);
    ``limit`` None: no clamp.  (limit None, alpha 1, shift 0 is the plain SiLU-gated unit silu(gate) * up.)"""
    T, F2 = gu.shape
    F = F2 // 2
    limit = math.inf if limit is None else limit
    if not gu.is_cuda:
        g = gu[:, :F].float().clamp(max=limit)
        u = gu[:, F:].float().clamp(-limit, limit)
        return (g * torch.sigmoid(alpha * g) * (u + shift)).to(gu.dtype)
    assert gu.is_contiguous()
    out = torch.empty(T, F, dtype=gu.dtype, device=gu.device)
    call("grag_clamped_glu", ptr(gu), ptr(out), T, F, float(limit), float(alpha),
         0 if gu.dtype == torch.bfloat16 else 1, float(shift))
    return out


# ---------------------------------------------------------------------------------------------- q / k norm + store
def qk_norm_store(proj: torch.Tensor, qoff: int, koff: int, qw: torch.Tensor, kw: torch.Tensor,
                  slot_mapping: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, H: int, G: int, d: int,
                  eps: float) -> torch.Tensor:
    """Attention whose values are its keys.  From a fused projection ``proj`` [T, ld] (q heads at column qoff, k
    heads at koff): returns q / rms(q) * qw [T, H, d]; stores k / rms(k) * kw into k_cache and k as projected into
    v_cache (both [blocks, G, BS, d]) at ``slot_mapping`` (-1: not stored).  The norms are per head, fp32."""
    T = proj.shape[0]
    BS = k_cache.shape[2]
    if not proj.is_cuda:
        x = proj.float()
        q = x[:, qoff:qoff + H * d].reshape(T, H, d)
        k = x[:, koff:koff + G * d].reshape(T, G, d)
        qn = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw.float()
        kn = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw.float()
        ok = slot_mapping >= 0
        sl = slot_mapping[ok].long()
        k_cache[sl // BS, :, sl % BS] = kn[ok].to(k_cache.dtype)
        v_cache[sl // BS, :, sl % BS] = k[ok].to(v_cache.dtype)
        return qn.to(proj.dtype)
    assert proj.stride(1) == 1 and k_cache.dtype == proj.dtype and v_cache.dtype == proj.dtype
    assert k_cache.shape[1:] == (G, BS, d) and v_cache.shape == k_cache.shape and qw.numel() == d and kw.numel() == d
    q = torch.empty(T, H, d, dtype=proj.dtype, device=proj.device)
    call("grag_qk_norm_store", ptr(proj), proj.stride(0), qoff, koff, ptr(qw), ptr(kw), ptr(slot_mapping), ptr(q),
         ptr(k_cache), ptr(v_cache), T, H, G, d, BS, k_cache.shape[0] * BS, float(eps),
         0 if proj.dtype == torch.bfloat16 else 1)
    return q


def latent_store(ckv: torch.Tensor, cw: torch.Tensor, positions: torch.Tensor, table: torch.Tensor,
                 slot_mapping: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, eps: float) -> torch.Tensor:
    """Latent attention's cache row and query rotation.  ``ckv`` [T, R + r]: a latent of R columns and r columns of
    the key part that all heads share (r = the width of ``table``, a rope_table).  Stores latent / rms(latent) * cw |
    rotated part into k_cache [blocks, 1, BS, R + r] at ``slot_mapping`` (the attention reads its values, the normed
    latent, out of the same rows); rotates the last r columns of every head of ``q`` [T, H, R + r] in place."""
    T, H = q.shape[0], q.shape[1]
    BS, r = k_cache.shape[2], table.shape[1]
    R = k_cache.shape[3] - r
    if not ckv.is_cuda:
        x = ckv.float()
        c = x[:, :R]
        c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * cw.float()
        h2 = r // 2
        cs = table[positions.long()]
        co, sn = cs[:, :h2], cs[:, h2:]

        def rot(t, co, sn):
            a, b = t[..., :h2], t[..., h2:]
            return torch.cat([a * co - b * sn, b * co + a * sn], dim=-1)

        kr = rot(x[:, R:], co, sn)
        q[:, :, R:] = rot(q[:, :, R:].float(), co[:, None], sn[:, None]).to(q.dtype)
        ok = slot_mapping >= 0
        sl = slot_mapping[ok].long()
        k_cache[sl // BS, 0, sl % BS] = torch.cat([c, kr], -1)[ok].to(k_cache.dtype)
        return q
    assert ckv.stride(1) == 1 and q.is_contiguous() and q.shape[2] == R + r and ckv.shape[1] == R + r
    assert k_cache.dtype == ckv.dtype and q.dtype == ckv.dtype and k_cache.is_contiguous()
    assert k_cache.shape[1] == 1 and cw.numel() == R and R > 0
    call("grag_latent_store", ptr(ckv), ckv.stride(0), ptr(cw), ptr(positions), ptr(table), table.shape[0],
         ptr(slot_mapping), ptr(q), ptr(k_cache), T, H, R, r, BS, k_cache.shape[0] * BS, float(eps),
         0 if ckv.dtype == torch.bfloat16 else 1)
    return q


def latent_rope_store(proj: torch.Tensor, qoff: int, coff: int | None, cw: torch.Tensor | None,
                      positions: torch.Tensor, table: torch.Tensor, slot_mapping: torch.Tensor,
                      k_cache: torch.Tensor, H: int, eps: float, interleaved: bool = False) -> torch.Tensor:
    """Latent attention's cache row and queries out of one fused projection ``proj`` [T, ld].  Columns qoff ..: H
    query heads of R + r columns each (R against the latent, r = the width of ``table``, a rope_table, to rotate);
    returned as q [T, H, R + r] with the last r columns of every head rotated by ``positions``.  Columns coff ..
    (``coff`` None: this layer reads another layer's cache and stores nothing): a latent of R columns and the r
    columns of the key part all heads share; k_cache [blocks, 1, BS, R + r] <- latent / rms(latent) * cw | rotated
    part at ``slot_mapping`` (-1: not stored).  Rotation pairs dim i with i + r/2, or 2i with 2i + 1 when
    ``interleaved`` (pair i turned by the table's angle i); the statistics and the rotation are fp32."""
    T = proj.shape[0]
    BS, r = k_cache.shape[2], table.shape[1]
    R = k_cache.shape[3] - r
    h2 = r // 2

    if not proj.is_cuda:
        x = proj.float()
        cs = table[positions.long()]
        co, sn = cs[:, :h2], cs[:, h2:]

        def rot(t, co, sn):
            if interleaved:
                a, b = t[..., 0::2], t[..., 1::2]
                return torch.stack([a * co - b * sn, b * co + a * sn], dim=-1).flatten(-2)
            a, b = t[..., :h2], t[..., h2:]
            return torch.cat([a * co - b * sn, b * co + a * sn], dim=-1)

        q = x[:, qoff:qoff + H * (R + r)].reshape(T, H, R + r).clone()
        q[:, :, R:] = rot(q[:, :, R:], co[:, None], sn[:, None])
        if coff is not None:
            c = x[:, coff:coff + R]
            c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * cw.float()
            kr = rot(x[:, coff + R:coff + R + r], co, sn)
            ok = slot_mapping >= 0
            sl = slot_mapping[ok].long()
            k_cache[sl // BS, 0, sl % BS] = torch.cat([c, kr], -1)[ok].to(k_cache.dtype)
        return q.to(proj.dtype)
    assert proj.stride(1) == 1 and k_cache.dtype == proj.dtype and k_cache.is_contiguous() and k_cache.shape[1] == 1
    assert R > 0 and r % 2 == 0 and table.dtype == torch.float32
    assert coff is None or (cw is not None and cw.dtype == torch.float32 and cw.numel() == R)
    assert qoff + H * (R + r) <= proj.shape[1] and (coff is None or coff + R + r <= proj.shape[1])
    q = torch.empty(T, H, R + r, dtype=proj.dtype, device=proj.device)
    call("grag_latent_rope_store", ptr(proj), proj.stride(0), qoff, -1 if coff is None else coff, ptr(cw),
         ptr(positions), ptr(table), table.shape[0], ptr(slot_mapping), ptr(q), ptr(k_cache), T, H, R, r, BS,
         k_cache.shape[0] * BS, float(eps), 0 if proj.dtype == torch.bfloat16 else 1, 1 if interleaved else 0)
    return q


def tanh_cap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """In place: x <- cap * tanh(x / cap), evaluated in fp32 (``cap`` <= 0: x as it is).  x [rows, N], rows may be
    a column slice of a wider tensor."""
    if cap <= 0 or x.numel() == 0:
        return x
    if not x.is_cuda:
        x.copy_((cap * torch.tanh(x.float() / cap)).to(x.dtype))
        return x
    assert x.dim() == 2 and x.stride(1) == 1
    call("grag_tanh_cap", ptr(x), x.stride(0), x.shape[0], x.shape[1], float(cap), 0 if x.dtype == torch.bfloat16 else 1)
    return x
