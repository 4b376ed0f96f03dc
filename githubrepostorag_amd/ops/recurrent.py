"""Recurrent sequence mixers with a carried fp32 state per sequence (HIP on device tensors, plain fp32 loops on
CPU): linear attention with a fixed per-head decay, and the minGRU gated recurrence.

State lives in slot-indexed pools ([slots, ...] fp32) owned by the engine; ``meta.state_slots`` [nseq] names each
sequence's slot.  A sequence whose first token of the step is position 0 starts from a zero state (so a freed
slot needs no reset when it is used again); otherwise the step continues from the slot's state and leaves the
state after its last token there.  Tokens are consumed in order, so a prompt may be cut into steps anywhere.
"""
from __future__ import annotations

import torch

from ._lib import call, lib, ptr
from .attention import AttnMetadata


def _chunk_ws(kind: str, m: AttnMetadata, per_chunk: int, device) -> torch.Tensor | None:
    """fp32 scratch for the chunk-parallel passes of a long portion ([sequences * chunks, per_chunk]); None when
    every portion of the step fits one chunk (decode rows, short portions): the one-pass kernels take those."""
    chunk = getattr(lib(), "grag_decay_attn_chunk" if kind == "decay" else "grag_mingru_chunk")()
    if m.max_q_len <= chunk:
        return None
    return torch.empty(m.num_seqs * -(-m.max_q_len // chunk) * per_chunk, dtype=torch.float32, device=device)


def _dt(t: torch.Tensor) -> int:
    return 0 if t.dtype == torch.bfloat16 else 1


def _parts(meta: AttnMetadata):
    """(meta, first row, end row) of a step's parts: prefill chunks, then the decode rows of a mixed step."""
    dec = meta.extra.get("decode_rows")
    if dec is None:
        return [(meta, 0, meta.num_tokens)]
    Tp, dmeta = dec
    return [(meta, 0, Tp), (dmeta, Tp, Tp + dmeta.num_tokens)]


def decay_attention(proj: torch.Tensor, qoff: int, koff: int, voff: int, decay: torch.Tensor, state: torch.Tensor,
                    meta: AttnMetadata, H: int, d: int, vd: int, act: bool = True, positions: torch.Tensor | None = None,
                    rope: torch.Tensor | None = None, k_scale: float = 1.0) -> torch.Tensor:
    """Linear attention with decay.  From the fused projection ``proj`` [T, ld]: q, k = columns qoff / koff (H x d),
    v = columns voff (H x vd), each through SiLU when ``act``.  With ``rope`` (a rope_table [positions, rd]) the
    first rd dims of q and k are rotated by ``positions`` (dim i paired with i + rd/2) in fp32 inside the scan, and
    k is multiplied by ``k_scale`` after the rotation.  Per head S_t = decay_h S_(t-1) + k_t v_t^T (state
    [slots, H, d, vd] fp32), o_t = S_t^T q_t.  Returns o [T, H*vd] fp32."""
    T = proj.shape[0]
    out = torch.empty(T, H * vd, dtype=torch.float32, device=proj.device)
    rd = 0 if rope is None else rope.shape[1]
    if rd and (positions is None or positions.dtype != torch.int32 or rope.dtype != torch.float32 or rd > d or rd % 2):
        raise ValueError("rotary needs int32 positions and an fp32 table of an even width <= the head size")
    for m, r0, r1 in _parts(meta):
        if r1 <= r0:
            continue
        pos = positions[r0:r1] if rd else None
        if not proj.is_cuda:
            _decay_attention_cpu(proj[r0:r1], qoff, koff, voff, decay, state, m, H, d, vd, out[r0:r1], act, pos, rope,
                                 k_scale)
            continue
        assert proj.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous()
        x = proj[r0:r1]
        ws = _chunk_ws("decay", m, H * d * vd, proj.device)
        call("grag_decay_attn_scan", ptr(x), proj.stride(0), qoff, koff, voff, ptr(decay), ptr(state),
             ptr(m.state_slots), ptr(m.q_start), ptr(m.ctx_len), ptr(out[r0:r1]), m.num_seqs, H, d, vd,
             state.shape[0], _dt(proj), ptr(ws), m.max_q_len, 1 if act else 0, ptr(pos), ptr(rope), rd,
             rope.shape[0] if rd else 0, float(k_scale))
    return out


def _decay_attention_cpu(x, qoff, koff, voff, decay, state, m, H, d, vd, out, act=True, pos=None, rope=None,
                         k_scale=1.0):
    F = torch.nn.functional
    qs, cl, sl = m.q_start.tolist(), m.ctx_len.tolist(), m.state_slots.tolist()
    x = x.float()
    f = F.silu if act else (lambda t: t)
    for s in range(m.num_seqs):
        a, b = qs[s], qs[s + 1]
        if b <= a:
            continue
        S = torch.zeros(H, d, vd) if cl[s] - (b - a) == 0 else state[sl[s]].clone()
        q = f(x[a:b, qoff:qoff + H * d]).view(-1, H, d).clone()
        k = f(x[a:b, koff:koff + H * d]).view(-1, H, d).clone()
        v = f(x[a:b, voff:voff + H * vd]).view(-1, H, vd)
        if rope is not None:
            rd = rope.shape[1]
            h2 = rd // 2
            cs = rope[pos[a:b].long()]
            c, sn = cs[:, None, :h2], cs[:, None, h2:]
            for t in (q, k):
                u, w = t[..., :h2].clone(), t[..., h2:rd].clone()
                t[..., :h2] = u * c - w * sn
                t[..., h2:rd] = w * c + u * sn
        k = k * k_scale
        lam = decay.float().view(H, 1, 1)
        for t in range(b - a):
            S = lam * S + k[t, :, :, None] * v[t, :, None, :]
            out[a + t] = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1)
        state[sl[s]] = S


def gated_rmsnorm(x: torch.Tensor, w: torch.Tensor | None, proj: torch.Tensor, goff: int, eps: float,
                  out: torch.Tensor, out_scale: float = 1.0, groups: int = 1, gate: str = "sigmoid",
                  gate_first: bool = False) -> torch.Tensor:
    """out = out_scale * x / rms(x) * w * gate(g): x [T, N] fp32 normalised over each of ``groups`` equal column
    groups (1: the whole row; the head count: per head), ``w`` [N] optional, g read from columns goff.. of the
    fused projection, gate "sigmoid" or "silu"; ``out`` [T, N] may be a column slice of a wider buffer.
    ``gate_first``: the gate comes before the norm, out = out_scale * u / rms(u) * w with u = x * gate(g)."""
    T, N = x.shape
    if gate not in ("sigmoid", "silu") or N % groups:
        raise ValueError("gate is 'sigmoid' or 'silu', and the groups divide the row")
    if not x.is_cuda:
        g = proj[:, goff:goff + N].float()
        g = torch.sigmoid(g) if gate == "sigmoid" else torch.nn.functional.silu(g)
        xg = (x * g if gate_first else x).view(T, groups, N // groups)
        y = (xg / torch.sqrt(xg.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, N)
        out.copy_(y * (1.0 if w is None else w.float()) * (1.0 if gate_first else g) * out_scale)
        return out
    assert x.is_contiguous() and out.stride(1) == 1 and out.dtype == proj.dtype
    call("grag_gated_rmsnorm", ptr(x), ptr(w), ptr(proj), proj.stride(0), goff, ptr(out), out.stride(0), T, N,
         float(eps), float(out_scale), _dt(proj), groups, (1 if gate == "silu" else 0) | (2 if gate_first else 0))
    return out


def mingru_scan(proj: torch.Tensor, zoff: int, xoff: int, goff: int, bz: torch.Tensor, bx: torch.Tensor,
                state: torch.Tensor, meta: AttnMetadata, W: int) -> torch.Tensor:
    """minGRU over a step's tokens.  From the fused projection [T, ld]: z = sigmoid(columns zoff + bz),
    u = columns xoff + bx, candidate = u + 1/2 where u >= 0 else sigmoid(u);
    S_t = (1 - z) S_(t-1) + z candidate (state [slots, W] fp32); returns S_t * silu(columns goff) [T, W]."""
    T = proj.shape[0]
    out = torch.empty(T, W, dtype=proj.dtype, device=proj.device)
    for m, r0, r1 in _parts(meta):
        if r1 <= r0:
            continue
        if not proj.is_cuda:
            _mingru_cpu(proj[r0:r1].float(), zoff, xoff, goff, bz, bx, state, m, W, out[r0:r1])
            continue
        assert proj.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous()
        ws = _chunk_ws("mingru", m, 2 * W, proj.device)
        call("grag_mingru_scan", ptr(proj[r0:r1]), proj.stride(0), zoff, xoff, goff, ptr(bz), ptr(bx), ptr(state),
             ptr(m.state_slots), ptr(m.q_start), ptr(m.ctx_len), ptr(out[r0:r1]), m.num_seqs, W, state.shape[0],
             _dt(proj), ptr(ws), m.max_q_len)
    return out


def _mingru_cpu(x, zoff, xoff, goff, bz, bx, state, m, W, out):
    qs, cl, sl = m.q_start.tolist(), m.ctx_len.tolist(), m.state_slots.tolist()
    z = torch.sigmoid(x[:, zoff:zoff + W] + bz.float())
    u = x[:, xoff:xoff + W] + bx.float()
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = torch.nn.functional.silu(x[:, goff:goff + W])
    for s in range(m.num_seqs):
        a, b = qs[s], qs[s + 1]
        if b <= a:
            continue
        S = torch.zeros(W) if cl[s] - (b - a) == 0 else state[sl[s]].clone()
        for t in range(a, b):
            S = (1.0 - z[t]) * S + z[t] * c[t]
            out[t] = (S * g[t]).to(out.dtype)
        state[sl[s]] = S


# ---------------------------------------------------------------------------------------------- state-space mixer
def causal_conv(proj: torch.Tensor, coff: int, w: torch.Tensor, b: torch.Tensor | None, cstate: torch.Tensor,
                meta: AttnMetadata, act: bool = True, residual: bool = False) -> torch.Tensor:
    """Causal depthwise convolution + SiLU over columns coff .. coff + C of the fused projection ``proj`` [T, ld]:
    out[t, c] = silu(b[c] + sum_j w[c, j] in[t - (taps - 1) + j, c]) with ``w`` [C, taps] fp32 (the last tap is the
    current token's).  Inputs before a portion come from ``cstate`` [slots, taps - 1, C] (the sequence's last
    taps - 1 inputs, oldest first; zeros for a sequence that starts at position 0), which is brought up to date
    after the step.  ``act`` False: no SiLU; ``residual``: the token's own input is added to the result
    (in + conv(in)).  Returns [T, C] in proj's dtype."""
    T = proj.shape[0]
    C, taps = w.shape
    out = torch.empty(T, C, dtype=proj.dtype, device=proj.device)
    for m, r0, r1 in _parts(meta):
        if r1 <= r0:
            continue
        if not proj.is_cuda:
            _causal_conv_cpu(proj[r0:r1], coff, w, b, cstate, m, out[r0:r1], act, residual)
            continue
        assert proj.stride(1) == 1 and cstate.dtype == proj.dtype and cstate.is_contiguous() and w.is_contiguous()
        assert w.dtype == torch.float32 and cstate.shape[1:] == (taps - 1, C) and taps <= lib().grag_conv_max_taps()
        call("grag_causal_conv", ptr(proj[r0:r1]), proj.stride(0), coff, C, taps, ptr(w), ptr(b), ptr(cstate),
             ptr(m.state_slots), ptr(m.q_start), ptr(m.ctx_len), ptr(out[r0:r1]), m.num_seqs, m.max_q_len,
             cstate.shape[0], _dt(proj), (0 if act else 1) | (2 if residual else 0))
    return out


def _causal_conv_cpu(x, coff, w, b, cstate, m, out, act=True, residual=False):
    C, taps = w.shape
    qs, cl, sl = m.q_start.tolist(), m.ctx_len.tolist(), m.state_slots.tolist()
    for s in range(m.num_seqs):
        a, e = qs[s], qs[s + 1]
        if e <= a:
            continue
        past = torch.zeros(taps - 1, C) if cl[s] - (e - a) == 0 else cstate[sl[s]].float()
        full = torch.cat([past, x[a:e, coff:coff + C].float()], 0)
        acc = torch.zeros(e - a, C) if b is None else b.float().expand(e - a, C).clone()
        for j in range(taps):
            acc += w[:, j].float() * full[j:j + (e - a)]
        if act:
            acc = torch.nn.functional.silu(acc)
        if residual:
            acc = acc + full[taps - 1:]
        out[a:e] = acc.to(out.dtype)
        if taps > 1:
            cstate[sl[s]] = full[-(taps - 1):].to(cstate.dtype)


def ssm_scan(xbc: torch.Tensor, proj: torch.Tensor, dtoff: int, dt_bias: torch.Tensor, a_log: torch.Tensor,
             skip: torch.Tensor, state: torch.Tensor, meta: AttnMetadata, H: int, G: int, N: int, P: int) -> torch.Tensor:
    """Selective state-space scan.  ``xbc`` [T, H*P + 2*G*N] (the convolution's output): x heads | B groups | C groups;
    the step sizes' raw values are columns dtoff .. dtoff + H of ``proj``.  Per head h (group h // (H / G)), in fp32:
    dt = softplus(raw + dt_bias[h]), S_t = exp(-exp(a_log[h]) dt) S_(t-1) + dt B_t x_t^T (state [slots, H, N, P]),
    y_t = S_t^T C_t + skip[h] x_t.  Returns y [T, H*P] fp32."""
    T = xbc.shape[0]
    out = torch.empty(T, H * P, dtype=torch.float32, device=xbc.device)
    C = xbc.shape[1]
    assert C == H * P + 2 * G * N
    for m, r0, r1 in _parts(meta):
        if r1 <= r0:
            continue
        if not xbc.is_cuda:
            _ssm_scan_cpu(xbc[r0:r1].float(), proj[r0:r1, dtoff:dtoff + H].float(), dt_bias, a_log, skip, state, m, H, G,
                          N, P, out[r0:r1])
            continue
        assert xbc.is_contiguous() and proj.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous()
        assert xbc.dtype == proj.dtype and state.shape[1:] == (H, N, P)
        chunk = lib().grag_ssm_chunk()
        ws = wa = None
        if m.max_q_len > chunk:
            nch = m.num_seqs * -(-m.max_q_len // chunk)
            ws = torch.empty(nch * H * N * P, dtype=torch.float32, device=xbc.device)
            wa = torch.empty(nch * H, dtype=torch.float32, device=xbc.device)
        call("grag_ssm_scan", ptr(xbc[r0:r1]), C, H * P, H * P + G * N, ptr(proj[r0:r1]), proj.stride(0), dtoff,
             ptr(dt_bias), ptr(a_log), ptr(skip), ptr(state), ptr(m.state_slots), ptr(m.q_start), ptr(m.ctx_len),
             ptr(out[r0:r1]), m.num_seqs, H, G, N, P, state.shape[0], _dt(xbc), ptr(ws), ptr(wa), m.max_q_len)
    return out


def _ssm_scan_cpu(xbc, dtraw, dt_bias, a_log, skip, state, m, H, G, N, P, out):
    qs, cl, sl = m.q_start.tolist(), m.ctx_len.tolist(), m.state_slots.tolist()
    dt = torch.nn.functional.softplus(dtraw + dt_bias.float(), threshold=20.0)
    decay = torch.exp(-torch.exp(a_log.float()) * dt)
    R = H // G
    for s in range(m.num_seqs):
        a, e = qs[s], qs[s + 1]
        if e <= a:
            continue
        S = torch.zeros(H, N, P) if cl[s] - (e - a) == 0 else state[sl[s]].clone()
        x = xbc[a:e, :H * P].view(-1, H, P)
        B = xbc[a:e, H * P:H * P + G * N].view(-1, G, N).repeat_interleave(R, dim=1)
        Cm = xbc[a:e, H * P + G * N:].view(-1, G, N).repeat_interleave(R, dim=1)
        for t in range(e - a):
            S = decay[a + t, :, None, None] * S + (dt[a + t, :, None] * B[t])[:, :, None] * x[t][:, None, :]
            out[a + t] = (torch.einsum("hnp,hn->hp", S, Cm[t]) + skip.float()[:, None] * x[t]).reshape(-1)
        state[sl[s]] = S
