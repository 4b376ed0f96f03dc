"""Mixture-of-experts feed-forward ops (HIP on device tensors, plain fp32 on CPU): the router with group-limited
top-k choice, and the experts' SiLU-gated units over the chosen (token, expert) pairs.

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


def moe_experts(h: torch.Tensor, ids: torch.Tensor, wgu: torch.Tensor, wd: torch.Tensor) -> torch.Tensor:
    """The chosen experts' outputs, unweighted: h [T, W], ids [T, top] int32, ``wgu`` [E, 2F, W] (every expert's gate
    rows, then its up rows), ``wd`` [E, W, F] -> [T, top, W] with out[t, k] = wd[e] (silu(gate_e h_t) * (up_e h_t)),
    e = ids[t, k]."""
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
                act = (torch.nn.functional.silu(gu[:F]) * gu[F:]).to(h.dtype)  # (the kernels store it in h's type)
                out[t, k] = wd[e].float() @ act.float()
        return out.to(h.dtype)
    assert h.stride(1) == 1 and wgu.is_contiguous() and wd.is_contiguous() and ids.is_contiguous()
    assert wgu.dtype == h.dtype and wd.dtype == h.dtype and wd.shape == (E, W, F) and wgu.shape[2] == W
    n = T * top
    offs = torch.empty(E + 1, dtype=torch.int32, device=h.device)
    order = torch.empty(n, dtype=torch.int32, device=h.device)
    call("grag_moe_align", ptr(ids), n, E, ptr(offs), ptr(order))
    act = torch.empty(n, F, dtype=h.dtype, device=h.device)
    call("grag_moe_gemm", ptr(h), h.stride(0), ptr(wgu), ptr(offs), ptr(order), n, E, top, F, W, ptr(act), F, 1, _dt(h))
    out = torch.empty(T, top, W, dtype=h.dtype, device=h.device)
    call("grag_moe_gemm", ptr(act), F, ptr(wd), ptr(offs), ptr(order), n, E, top, W, F, ptr(out), W, 0, _dt(h))
    return out
