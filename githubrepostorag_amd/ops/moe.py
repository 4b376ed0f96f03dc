"""Mixture-of-experts feed-forward ops (HIP on device tensors, plain fp32 on CPU): the router with group-limited
top-k choice (or a table that names every token id's experts), and the experts' gated units over the chosen
(token, expert) pairs; the same grouped GEMM also runs one small matrix per attention head.

The router's logits, scores and weights are fp32.  The experts run as two grouped GEMMs over the pairs sorted by
expert; their outputs come back in (token, choice) order and are summed, with the router's weights, in fp32 by the
layer's residual boundary (ops/norm.py residual_rmsnorm)."""
from __future__ import annotations

import torch

from ._lib import call, lib, ptr


def _dt(t: torch.Tensor) -> int:
    return 0 if t.dtype == torch.bfloat16 else 1


def moe_route(h: torch.Tensor, wr: torch.Tensor, E: int, top: int, groups: int = 1, keep: int = 1):
    """h [T, W]; ``wr`` [R, W] fp32 with the experts' router rows first (R = E, or E + 1 when a last row holds the
    shared expert's gate).  Scores s = softmax of the E logits.  The experts form ``groups`` equal groups of
    neighbours; a group's score is its best expert's, and only experts of the ``keep`` best groups can be chosen.
    Returns (ids [T, top] int32: the chosen experts by falling score, wts [T, top] fp32: their scores as they are,
    gate [T] fp32 = sigmoid of the extra row's logit, or None)."""
    T, W = h.shape
    R = wr.shape[0]
    if E % groups or not 1 <= keep <= groups or not 1 <= top <= E or R not in (E, E + 1):
        raise ValueError("bad router sizes")
    if not h.is_cuda:
        z = h.float() @ wr.float().T
        s = torch.softmax(z[:, :E], -1)
        gs = s.view(T, groups, E // groups).amax(-1)
        open_g = torch.zeros(T, groups, dtype=torch.bool)
        open_g.scatter_(1, gs.topk(keep, dim=-1).indices, True)
        masked = s.masked_fill(~open_g.repeat_interleave(E // groups, dim=1), -1.0)
        wts, ids = masked.topk(top, dim=-1)
        wts = wts.clamp_min(0.0)
        return ids.to(torch.int32), wts.contiguous(), (torch.sigmoid(z[:, E]) if R > E else None)
    if R > lib().grag_moe_max_rows() or top > lib().grag_moe_max_top():
        raise ValueError(f"the router kernel holds {lib().grag_moe_max_rows()} logit rows and {lib().grag_moe_max_top()} choices")
    assert h.stride(1) == 1 and wr.dtype == torch.float32 and wr.is_contiguous()
    ids = torch.empty(T, top, dtype=torch.int32, device=h.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=h.device)
    gate = torch.empty(T, dtype=torch.float32, device=h.device) if R > E else None
    call("grag_moe_route", ptr(h), h.stride(0), ptr(wr), W, E, R, top, groups, keep, ptr(ids), ptr(wts), ptr(gate), T,
         _dt(h))
    return ids, wts, gate


def moe_table_route(token_ids: torch.Tensor, table: torch.Tensor):
    """Routing without a router: ``table`` [vocab, top] int32 names the experts of every token id.  Returns
    (ids [T, top] int32 = the rows of the step's token ids, wts [T, top] fp32 = 1 / top each).  ``table``
    [layers, vocab, top]: the tables of several layers in one launch, ids [layers, T, top]."""
    T, top = token_ids.numel(), table.shape[-1]
    if not table.is_cuda:
        ids = table[..., token_ids.long(), :].to(torch.int32).contiguous()
        return ids, torch.full((T, top), 1.0 / top, dtype=torch.float32)
    assert table.dtype == torch.int32 and table.is_contiguous() and token_ids.dtype == torch.int32
    nl = 1 if table.dim() == 2 else table.shape[0]
    ids = torch.empty(*table.shape[:-2], T, top, dtype=torch.int32, device=table.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=table.device)
    call("grag_moe_table_route", ptr(token_ids), ptr(table), nl, table.shape[-2], top, ptr(ids), ptr(wts), T)
    return ids, wts


def moe_experts(h: torch.Tensor, ids: torch.Tensor, wgu: torch.Tensor, wd: torch.Tensor,
                limit: float | None = None, alpha: float = 1.0, shift: float = 0.0) -> torch.Tensor:
    """The chosen experts' outputs, unweighted: h [T, W], ids [T, top] int32, ``wgu`` [E, 2F, W] (every expert's gate
    rows, then its up rows), ``wd`` [E, W, F] -> [T, top, W] with out[t, k] = wd[e] (silu(gate_e h_t) * (up_e h_t)),
    e = ids[t, k].  With ``limit`` / ``alpha`` / ``shift`` the unit is g sigmoid(alpha g) (u + shift) with
    g = min(gate, limit), u = clamp(up, -limit, limit) (``limit`` None: no clamp)."""
    T, W = h.shape
    top = ids.shape[1]
    E, F2, _ = wgu.shape
    F = F2 // 2
    if not h.is_cuda:
        x = h.float()
        out = torch.zeros(T, top, W)
        for t in range(T):
            for k in range(top):
                e = int(ids[t, k])
                gu = wgu[e].float() @ x[t]
                g, u = gu[:F], gu[F:]
                if limit is not None:
                    g, u = g.clamp(max=limit), u.clamp(-limit, limit)
                act = (g * torch.sigmoid(alpha * g) * (u + shift)).to(h.dtype)  # (the kernels store it in h's type)
                out[t, k] = wd[e].float() @ act.float()
        return out.to(h.dtype)
    assert h.stride(1) == 1 and wgu.is_contiguous() and wd.is_contiguous() and ids.is_contiguous()
    assert wgu.dtype == h.dtype and wd.dtype == h.dtype and wd.shape == (E, W, F) and wgu.shape[2] == W
    n = T * top
    offs = torch.empty(E + 1, dtype=torch.int32, device=h.device)
    order = torch.empty(n, dtype=torch.int32, device=h.device)
    call("grag_moe_align", ptr(ids), n, E, ptr(offs), ptr(order))
    act = torch.empty(n, F, dtype=h.dtype, device=h.device)
    lim = float("inf") if limit is None else float(limit)
    call("grag_moe_gemm", ptr(h), h.stride(0), ptr(wgu), ptr(offs), ptr(order), n, E, top, F, W, ptr(act), F, 1, _dt(h),
         lim, float(alpha), float(shift), None, 0)
    out = torch.empty(T, top, W, dtype=h.dtype, device=h.device)
    call("grag_moe_gemm", ptr(act), F, ptr(wd), ptr(offs), ptr(order), n, E, top, W, F, ptr(out), W, 0, _dt(h),
         lim, 1.0, 0.0, None, 0)
    return out


def head_project(x: torch.Tensor, w: torch.Tensor, gate: torch.Tensor | None = None) -> torch.Tensor:
    """One small matrix per head: x [T, H * K] (head h's K columns side by side), ``w`` [H, N, K] -> out [T, H * N] with
    out[t, h] = w[h] x[t, h]; with ``gate`` [T, H * N] (logits; rows may be a column slice of a wider tensor) the
    result is multiplied element by element by sigmoid(gate).  Runs as the experts' grouped GEMM with the heads as
    experts: row (t, h) belongs to "expert" h."""
    T = x.shape[0]
    H, N, K = w.shape
    if not x.is_cuda:
        o = torch.einsum("thk,hnk->thn", x.float().view(T, H, K), w.float()).reshape(T, H * N)
        if gate is not None:
            o = o * torch.sigmoid(gate.float())
        return o.to(x.dtype)
    assert x.is_contiguous() and x.shape[1] == H * K and w.is_contiguous() and w.dtype == x.dtype
    assert gate is None or (gate.dtype == x.dtype and gate.stride(1) == 1 and gate.shape == (T, H * N))
    out = torch.empty(T, H * N, dtype=x.dtype, device=x.device)
    # x viewed [T H, K] and out viewed [T H, N]: row t H + h is head h of token t.  The kernel's row order (sorted by
    # head) follows from H and T alone, so it takes no offset / order arrays: `top` carries T
    call("grag_moe_gemm", ptr(x), K, ptr(w), None, None, T * H, H, T, N, K, ptr(out), N, 2, _dt(x),
         float("inf"), 1.0, 0.0, ptr(gate), 0 if gate is None else gate.stride(0))
    return out
