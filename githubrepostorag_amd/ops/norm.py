"""Normalisation / embedding ops (HIP on device tensors, fp32 reference on CPU)."""
from __future__ import annotations

import os

import torch

from ._lib import call, lib, ptr
from .gemm import SplitKPartial


def _on_gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


def rmsnorm_ref(x, w, eps, residual=None):
    if residual is not None:
        s = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(s)
        xf = s.float()
    else:
        xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(x.dtype)


# the chunked ticket-merge kernel measured slower than one workgroup per row at B = 1 (8.6 vs 5.6 us: the
# agent-scope release / acquire round trips outweigh the parallel plane reads; profiles/decode_step_b1_r5.txt)
SMALL_ROWS = int(os.environ.get("GRAG_NORM_SMALL_ROWS", "0"))


def norm_ws(dev) -> tuple[torch.Tensor, torch.Tensor]:
    """(tickets [64] int32, zeroed; chunk sums [64 * 64] fp32) of the small-batch split-K RMSNorm, owned by
    the caller's workspace owner (ops/gemm.py WS.scratch); allocated before any hipGraph capture (LLMEngine
    does, under its owner) -- every last arriver resets its ticket."""
    from .gemm import WS

    return WS.scratch("norm_tickets", torch.device(dev),
                      lambda d: (torch.zeros(64, dtype=torch.int32, device=d), torch.zeros(64 * 64, device=d)))


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
            out: torch.Tensor | None = None) -> torch.Tensor:
    """y = RMSNorm(x [+ residual]) * w.  With ``residual`` the sum is written
    back into ``residual`` (the decoder's residual stream), fused in one pass."""
    if isinstance(x, SplitKPartial):  # deferred split-K projection: reduce + residual add + norm in one pass
        if residual is None:
            x = x.materialize()
        else:
            out = torch.empty(x.M, x.N, dtype=x.dtype, device=x.device) if out is None else out
            if x.M <= SMALL_ROWS:  # 1-16 rows: the row's planes reduced by ceil(N / 512) workgroups
                ws = norm_ws(x.device)
                call("grag_splitk_add_rmsnorm_small", ptr(x.planes), x.S, ptr(residual), ptr(w), ptr(out), x.M, x.N,
                     float(eps), ptr(ws[1]), ptr(ws[0]))
            else:
                call("grag_splitk_add_rmsnorm", ptr(x.planes), x.S, ptr(residual), ptr(w), ptr(out), x.M, x.N,
                     float(eps))
            return out
    if not _on_gpu(x):
        return rmsnorm_ref(x, w, eps, residual)
    x = x.contiguous()
    T, H = x.shape[0] if x.dim() == 2 else x.numel() // x.shape[-1], x.shape[-1]
    out = torch.empty_like(x) if out is None else out
    call("grag_rmsnorm", ptr(x), ptr(residual), ptr(w), ptr(out), T, H, float(eps))
    return out


def layernorm_ref(x, gamma, beta, eps, bias=None, residual=None):
    v = x.float()
    if bias is not None:
        v = v + bias.float()
    if residual is not None:
        v = v + residual.float()
    return torch.nn.functional.layer_norm(v, (v.shape[-1],), gamma.float(), beta.float(), eps).to(x.dtype)


def layernorm(x, gamma, beta, eps, bias=None, residual=None):
    """y = LN(x [+ bias] [+ residual]) * gamma + beta (BERT post-LN block)."""
    if not _on_gpu(x):
        return layernorm_ref(x, gamma, beta, eps, bias, residual)
    x = x.contiguous()
    H = x.shape[-1]
    T = x.numel() // H
    out = torch.empty_like(x)
    call("grag_layernorm", ptr(x), ptr(bias), ptr(residual), ptr(gamma), ptr(beta), ptr(out), T, H, float(eps))
    return out


def add_layernorm_ref(x, gamma, beta, eps, residual, bias=None):
    v = x.float() + residual.float()
    if bias is not None:
        v = v + bias.float()
    s = v.to(residual.dtype)
    residual.copy_(s)
    return torch.nn.functional.layer_norm(s.float(), (v.shape[-1],), gamma.float(), beta.float(),
                                          eps).to(x.dtype)


def add_layernorm(x, gamma, beta, eps, residual, bias=None):
    """Pre-LN block boundary (GPT-2): ``residual += x [+ bias]`` in place, then
    return LN(residual) * gamma + beta — one pass over the row."""
    if not _on_gpu(x):
        return add_layernorm_ref(x, gamma, beta, eps, residual, bias)
    x = x.contiguous()
    H = x.shape[-1]
    T = x.numel() // H
    out = torch.empty_like(x)
    call("grag_add_layernorm", ptr(x), ptr(bias), ptr(residual), ptr(gamma), ptr(beta), ptr(out), T, H,
         float(eps))
    return out


def bert_embed_ln_ref(ids, pos_ids, type_ids, word, pos, typ, gamma, beta, eps):
    v = word[ids.long()].float() + pos[pos_ids.long()].float()
    v = v + (typ[type_ids.long()].float() if type_ids is not None else typ[0].float())
    return torch.nn.functional.layer_norm(v, (v.shape[-1],), gamma.float(), beta.float(), eps).to(word.dtype)


def bert_embed_ln(ids, pos_ids, type_ids, word, pos, typ, gamma, beta, eps):
    if not _on_gpu(word):
        return bert_embed_ln_ref(ids, pos_ids, type_ids, word, pos, typ, gamma, beta, eps)
    T, H = ids.numel(), word.shape[1]
    out = torch.empty(T, H, dtype=word.dtype, device=word.device)
    ids = ids.to(torch.int32).contiguous()
    pos_ids = pos_ids.to(torch.int32).contiguous()
    type_ids = None if type_ids is None else type_ids.to(torch.int32).contiguous()
    call("grag_bert_embed_ln", ptr(ids), ptr(pos_ids), ptr(type_ids), ptr(word), ptr(pos), ptr(typ),
         ptr(gamma), ptr(beta), ptr(out), T, H, word.shape[0], pos.shape[0], float(eps))
    return out


def embed_gather(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    if not _on_gpu(table):
        return table[ids.long()]
    ids = ids.to(torch.int32).contiguous()
    T, H = ids.numel(), table.shape[1]
    out = torch.empty(T, H, dtype=table.dtype, device=table.device)
    call("grag_embed_gather", ptr(ids), ptr(table), ptr(out), T, H, table.shape[0])
    return out


# ---------------------------------------------------------------------------------------------- Dynamic Tanh
def dyt_ref(x: torch.Tensor, alpha: float, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Dynamic Tanh norm, fp32: tanh(alpha x) w + b (element-wise; no mean, no variance)."""
    return torch.tanh(alpha * x.float()) * w.float() + b.float()


def dyt_residual(resid: torch.Tensor, y: torch.Tensor | None = None, post=None, add_rows: torch.Tensor | None = None,
                 add_vec: torch.Tensor | None = None, pre=None, out_dtype=torch.bfloat16) -> torch.Tensor | None:
    """One pass over the fp32 residual stream ``resid`` [T, H] (updated in place):
    resid += dyt_post(y) (+ add_rows [T, H] fp32) (+ add_vec [H] fp32), then returns dyt_pre(resid) in
    ``out_dtype`` (None without ``pre``).  ``post`` / ``pre`` are (alpha, w fp32 [H], b fp32 [H]) triples:
    the norm that closes one sublayer and the norm that opens the next, fused at the sublayer boundary."""
    assert resid.dtype == torch.float32 and resid.is_contiguous()
    T, H = resid.shape
    if not _on_gpu(resid):
        if y is not None:
            resid += dyt_ref(y, *post)
        if add_rows is not None:
            resid += add_rows
        if add_vec is not None:
            resid += add_vec
        return None if pre is None else dyt_ref(resid, *pre).to(out_dtype)
    out = torch.empty(T, H, dtype=out_dtype, device=resid.device) if pre is not None else None
    if y is not None:
        assert y.dtype == out_dtype and y.is_contiguous() and y.shape == resid.shape
    a1, w1, b1 = post if y is not None else (0.0, None, None)
    a2, w2, b2 = pre if pre is not None else (0.0, None, None)
    call("grag_dyt_residual", ptr(y), float(a1), ptr(w1), ptr(b1), ptr(resid), ptr(add_rows), ptr(add_vec), float(a2),
         ptr(w2), ptr(b2), ptr(out), T, H, 0 if out_dtype == torch.bfloat16 else 1)
    return out


def embed_gather_f32(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Embedding rows as an fp32 [T, H] residual stream (table bf16 or fp32), multiplied by ``scale`` in fp32."""
    if not _on_gpu(table):
        x = table[ids.long()].float()
        return x if scale == 1.0 else x * scale
    ids = ids.to(torch.int32).contiguous()
    T, H = ids.numel(), table.shape[1]
    out = torch.empty(T, H, dtype=torch.float32, device=table.device)
    call("grag_embed_f32", ptr(ids), ptr(table), ptr(out), T, H, table.shape[0],
         0 if table.dtype == torch.bfloat16 else 1, float(scale))
    return out


# ---------------------------------------------------------------------------------------------- hyper-connections
def hyper_mix(streams: torch.Tensor, y: torch.Tensor | None = None, mix: torch.Tensor | None = None,
              outc: torch.Tensor | None = None, inc: torch.Tensor | None = None, w: torch.Tensor | None = None,
              eps: float = 1e-6, out_dtype=torch.bfloat16, want_sum: bool = False):
    """One pass over S fp32 residual streams ``streams`` [S, T, H] (updated in place) at a sublayer boundary:
    with ``y`` [T, H] (the sublayer's output): x_t <- sum_s mix[s, t] x_s + outc[t] y for every stream t at once;
    then, with ``inc`` [S]: u = sum_s inc[s] x_s, returned RMS-normed as u / sqrt(mean(u^2) + eps) * w in
    ``out_dtype`` (``w`` [H] fp32 is the norm's whole multiplier) and / or as it is in fp32 (``want_sum``).
    Returns (normed | None, sum | None).  S = 1 with mix = outc = inc = 1 is the ordinary residual sum."""
    assert streams.dtype == torch.float32 and streams.is_contiguous() and streams.dim() == 3
    S, T, H = streams.shape
    if not _on_gpu(streams):
        if y is not None:
            streams.copy_(torch.einsum("st,snh->tnh", mix.float(), streams) + outc.float()[:, None, None] * y.float())
        if inc is None:
            return None, None
        u = torch.einsum("s,snh->nh", inc.float(), streams)
        h = None if w is None else (u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)
        return h, (u if want_sum else None)
    if S > lib().grag_hyper_max_streams():
        raise ValueError(f"{S} residual streams: the kernel holds at most {lib().grag_hyper_max_streams()}")
    if y is not None:
        assert y.dtype == out_dtype and y.is_contiguous() and y.shape == (T, H)
    out = torch.empty(T, H, dtype=out_dtype, device=streams.device) if (inc is not None and w is not None) else None
    usum = torch.empty(T, H, dtype=torch.float32, device=streams.device) if (inc is not None and want_sum) else None
    call("grag_hyper_mix", ptr(streams), S, ptr(y), ptr(mix), ptr(outc), ptr(inc), ptr(w), float(eps), ptr(out),
         ptr(usum), T, H, 0 if out_dtype == torch.bfloat16 else 1)
    return out, usum


def rmsnorm_rows(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x [T, N] (rows may be a column slice of a wider tensor; bf16 or fp32) -> x / sqrt(mean(x^2) + eps) * w
    (w fp32 [N]), contiguous, in x's dtype; the statistics are fp32."""
    T, N = x.shape
    if not _on_gpu(x):
        xf = x.float()
        return (xf / torch.sqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(x.dtype)
    assert x.stride(1) == 1 and w.dtype == torch.float32 and w.numel() == N
    out = torch.empty(T, N, dtype=x.dtype, device=x.device)
    call("grag_rmsnorm_rows", ptr(x), x.stride(0), ptr(w), ptr(out), T, N, float(eps),
         0 if x.dtype == torch.bfloat16 else 1)
    return out


# ---------------------------------------------------------------------------------------------- parallel-block boundary
def residual_rmsnorm(x: torch.Tensor, a: torch.Tensor | None = None, b: torch.Tensor | None = None,
                     bcoef: torch.Tensor | None = None, e: torch.Tensor | None = None,
                     ecoef: torch.Tensor | None = None, w: torch.Tensor | None = None, eps: float = 1e-6,
                     out_dtype=torch.bfloat16, keep: bool = True, raw: torch.Tensor | None = None,
                     gate: torch.Tensor | None = None, gbias: torch.Tensor | None = None, mult: float = 1.0):
    """One pass over the fp32 residual ``x`` [T, H] (updated in place) at the boundary of a layer whose sublayers
    read the same input: x <- x + (a + bcoef_t b + sum_k ecoef[t, k] e[t, k]) with every addend optional
    (``a``, ``b`` [T, H]; ``bcoef`` [T] fp32, None: 1; ``e`` [T, K, H] with ``ecoef`` [T, K] fp32), all summed in
    fp32; ``keep`` False: x is replaced by the sum instead.  ``raw`` [T, H] (a column slice of a wider buffer is
    fine): receives x in ``out_dtype``.  With ``w`` [H] fp32 returns x / sqrt(mean(x^2) + eps) * w in ``out_dtype``.
    A gated branch: with ``gate`` [T, H] (logits, rows may be a column slice of a wider tensor) and ``gbias`` [H] fp32
    the sum of the addends is multiplied element by element by sigmoid(gate + gbias), and by ``mult``, before it
    joins x."""
    assert x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
    T, H = x.shape
    K = 0 if e is None else e.shape[1]
    if not _on_gpu(x):
        y = torch.zeros_like(x)
        if a is not None:
            y += a.float()
        f = torch.zeros_like(x)
        if b is not None:
            f += b.float() * (1.0 if bcoef is None else bcoef.float()[:, None])
        if e is not None:
            f += (e.float() * ecoef.float()[:, :, None]).sum(1)
        y += f
        if gate is not None:
            y *= torch.sigmoid(gate.float() + (0.0 if gbias is None else gbias.float()))
        if mult != 1.0:
            y *= mult
        x.copy_(x + y if keep else y)
        if raw is not None:
            raw.copy_(x.to(raw.dtype))
        return None if w is None else (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)
    for t in (a, b):
        assert t is None or (t.dtype == out_dtype and t.is_contiguous() and t.shape == (T, H))
    assert e is None or (e.dtype == out_dtype and e.is_contiguous() and e.shape == (T, K, H)
                         and ecoef.dtype == torch.float32 and ecoef.is_contiguous() and ecoef.shape == (T, K))
    assert bcoef is None or (bcoef.dtype == torch.float32 and bcoef.numel() == T)
    assert raw is None or (raw.dtype == out_dtype and raw.stride(1) == 1 and raw.shape == (T, H))
    assert gate is None or (gate.dtype == out_dtype and gate.stride(1) == 1 and gate.shape == (T, H))
    assert gbias is None or (gate is not None and gbias.dtype == torch.float32 and gbias.numel() == H)
    out = torch.empty(T, H, dtype=out_dtype, device=x.device) if w is not None else None
    call("grag_residual_rmsnorm", ptr(x), 1.0 if keep else 0.0, ptr(a), ptr(b), ptr(bcoef), ptr(e), ptr(ecoef), K,
         ptr(w), float(eps), ptr(out), ptr(raw), 0 if raw is None else raw.stride(0), T, H,
         0 if out_dtype == torch.bfloat16 else 1, ptr(gate), 0 if gate is None else gate.stride(0), ptr(gbias),
         float(mult))
    return out
