"""``bench.py --hybrid [zofesun|namudra|leripel|pubulix]``: prefill and decode throughput of a hybrid decoder beside the decoders of
equal size that the engine already serves (same width, heads, head size, FFN width, layer count, vocabulary; random
weights, synthetic token ids), all through LLMEngine.generate, and a per-kernel table: each new kernel and the
like kernel of the closest model as a fraction of the roofline of what bounds it (HBM bytes or matrix / vector
flops).  Zofesun stands beside Qwen2; Namudra beside Zofesun (the closest: fp32 residual, decay scan, sink
attention kernels) and Qwen2; Leripel beside Namudra (the closest: fp32 residual, retention scan, the same attention
kernel family, a layer list that is data) and Qwen2; Pubulix beside Leripel (the closest: the same attention kernels
with a window instead of blocks, experts on the same grouped GEMM, the same convolution and boundary kernels) and
Qwen2, with Namudra's latent attention as the like kernel of its latent layers."""
from __future__ import annotations

import json
import time

import torch

HBM_BPS = 8.0e12        # HBM3E
MFMA_BF16 = 2.5e15      # dense bf16 matrix flop/s
VALU_F32 = 1.57e14      # fp32 vector flop/s (fma = 2)

SIZES = {
    # name: (width, heads, kv_heads, head size, ffn, layers, mingru every)
    "1b-like": (1536, 12, 2, 128, 8960, 8, 4),
    "7b-like": (3584, 28, 4, 128, 18944, 4, 4),
}
VOCAB = 32768


def _timed(fn, iters=10, warm=2):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / iters


def _models(name, dev):
    from ..models.configs import DecoderConfig, zofesun_config
    from ..models.qwen2 import Qwen2Model
    from ..models.zofesun import ZofesunModel

    W, H, G, D, ff, nl, every = SIZES[name]
    zc = zofesun_config(f"zofesun-{name}", VOCAB, W, nl, heads=H, kv_heads=G, dim=D, vdim=D, lin_heads=H, lin_dim=D,
                        lin_vdim=D, ff=ff, mingru_every=every)
    qc = DecoderConfig(f"qwen2-{name}", VOCAB, W, ff, nl, H, G, D, max_position=32768)
    return (lambda: ZofesunModel(zc, device=dev, seed=1)), (lambda: Qwen2Model(qc, device=dev, seed=1))


def _namudra_models(name, dev):
    """Namudra at a bench size: per four layers retention, windowed sigmoid attention, latent attention, windowed
    attention (every layer with a feed-forward, two residual streams), beside the Zofesun and Qwen2 stacks."""
    from ..models.configs import namudra_config
    from ..models.namudra import NamudraModel

    W, H, G, D, ff, nl, _ = SIZES[name]
    nc = namudra_config(f"namudra-{name}", VOCAB, W, ("rala" * nl)[:nl], heads=H, kv_heads=G, dim=D, ff=ff,
                        window=1024, kv_rank=192, q_rank=W // 4, rot_dim=64, streams=2, ret_ff=True)
    mk_z, mk_q = _models(name, dev)
    return (lambda: NamudraModel(nc, device=dev, seed=1)), mk_z, mk_q


def _engine_numbers(make, dev, batch, prompt_len, gen_len, graphs=True):
    from .llm_engine import EngineConfig, LLMEngine
    from .sequence import SamplingParams

    model = make()
    need = batch * (prompt_len + gen_len + 16)
    eng = LLMEngine(model, None, EngineConfig(max_num_seqs=batch, max_model_len=prompt_len + gen_len + 16,
                                              max_num_batched_tokens=max(8192, prompt_len), num_blocks=need // 16 + 2,
                                              use_cuda_graph=graphs, enable_prefix_caching=False))
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, VOCAB, (prompt_len,), generator=g).tolist() for _ in range(batch)]

    def run(n):
        t0 = time.perf_counter()
        eng.generate(prompts, SamplingParams(max_tokens=n, temperature=0.0, ignore_eos=True))
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    run(2)  # compile / capture
    run(gen_len + 1)
    t_pre = min(run(1) for _ in range(2))
    t_all = min(run(gen_len + 1) for _ in range(2))
    out = {"prefill_tok_s": round(batch * prompt_len / t_pre), "decode_tok_s": round(batch * gen_len / max(t_all - t_pre, 1e-9)),
           "prefill_ms": round(t_pre * 1e3, 2), "decode_ms_per_step": round((t_all - t_pre) / gen_len * 1e3, 3)}
    del eng, model
    torch.cuda.empty_cache()
    return out


def _kernel_table(dev, H=28, G=4, D=128, W=3584, ff=18944, T=2048, B=64, ctx=2048, bs=16):
    """[(kernel, seconds, bound, fraction of roofline)] for the new kernels and the like kernels of Qwen2."""
    from ..ops.attention import AttnMetadata, paged_attention, sink_attention
    from ..ops.elementwise import (clamped_glu, qkv_rope_kvstore, rope_cos_sin, rope_table, rope_vnorm_store, silu_mul)
    from ..ops.norm import dyt_residual, rmsnorm
    from ..ops.recurrent import decay_attention, gated_rmsnorm, mingru_scan

    bf = torch.bfloat16
    i32 = dict(dtype=torch.int32, device=dev)
    rows = []

    def add(name, sec, flops=0.0, bytes_=0.0, peak=MFMA_BF16):
        t_c, t_m = flops / peak, bytes_ / HBM_BPS
        bound = "flops" if t_c >= t_m else "bytes"
        rows.append({"kernel": name, "us": round(sec * 1e6, 1), "bound": bound,
                     "roofline_fraction": round(max(t_c, t_m) / sec, 4)})

    # ---- prefill attention: one prompt of T tokens
    nb = T // bs
    kc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    vc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    q = torch.randn(T, H, D, device=dev).to(bf)
    meta = AttnMetadata(q_start=torch.tensor([0, T], **i32), ctx_len=torch.tensor([T], **i32),
                        block_tables=(torch.arange(nb, **i32) + 1).view(1, nb), slot_mapping=torch.arange(T, **i32) + bs,
                        max_q_len=T, num_seqs=1, num_tokens=T, state_slots=torch.tensor([0], **i32))
    sinks = torch.zeros(H, device=dev)
    fl = 4.0 * T * T / 2 * H * D
    add("sink_attn_prefill", _timed(lambda: sink_attention(q, kc, vc, meta, 0.09, sinks)), flops=fl)
    add("qwen2 paged_attention prefill", _timed(lambda: paged_attention(q, kc, vc, meta, 0.09)), flops=fl)
    # ---- decode attention: B rows of ctx keys
    nbd = ctx // bs
    kd = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    vd_ = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    qd = torch.randn(B, H, D, device=dev).to(bf)
    part_o = torch.empty(8 * B * H * D, device=dev)
    part_ml = torch.empty(8 * B * H * 2, device=dev)
    dmeta = AttnMetadata(q_start=torch.arange(B + 1, **i32), ctx_len=torch.full((B,), ctx, **i32),
                         block_tables=(torch.arange(B * nbd, **i32) + 1).view(B, nbd), slot_mapping=None, max_q_len=1,
                         num_seqs=B, num_tokens=B, is_decode=True, num_splits=8, split_len=ctx // 8, part_o=part_o,
                         part_ml=part_ml, state_slots=torch.arange(B, **i32))
    by = 2.0 * B * ctx * G * D * 2
    add("sink_attn_decode", _timed(lambda: sink_attention(qd, kd, vd_, dmeta, 0.09, sinks)), bytes_=by)
    add("qwen2 paged_attention decode", _timed(lambda: paged_attention(qd, kd, vd_, dmeta, 0.09)), bytes_=by)
    # ---- rotary + K/V store
    proj = torch.randn(T, (H + 2 * G) * D, device=dev).to(bf)
    pos = torch.arange(T, **i32)
    tab = rope_table(T, D, 1e4, dev)
    cs = rope_cos_sin(T, D, 1e4, dev)
    by = T * (H + 2 * G) * D * 2 * 2.0
    add("rope_vnorm_store", _timed(lambda: rope_vnorm_store(proj, 0, H * D, (H + G) * D, pos, tab, meta.slot_mapping, kc, vc,
                                                            H, G, D, D, D, 1e-5)), bytes_=by)
    add("qwen2 qkv_rope_kvstore", _timed(lambda: qkv_rope_kvstore(proj, None, pos, cs, meta.slot_mapping, kc, vc, H, G, D)),
        bytes_=by)
    # ---- norms at a sublayer boundary
    resid = torch.randn(T, W, device=dev)
    y = torch.randn(T, W, device=dev).to(bf)
    w32, b32, wbf = torch.ones(W, device=dev), torch.zeros(W, device=dev), torch.ones(W, device=dev).to(bf)
    add("dyt_residual (fp32 stream)", _timed(lambda: dyt_residual(resid, y, (0.5, w32, b32), pre=(0.5, w32, b32))),
        bytes_=T * W * (2 + 4 + 4 + 2.0))
    rb = torch.randn(T, W, device=dev).to(bf)
    add("qwen2 add+rmsnorm (bf16 stream)", _timed(lambda: rmsnorm(y, wbf, 1e-6, residual=rb)), bytes_=T * W * 2 * 4.0)
    # ---- GLU
    gu = torch.randn(T, 2 * ff, device=dev).to(bf)
    add("clamped_glu", _timed(lambda: clamped_glu(gu, 7.0)), bytes_=T * ff * 2 * 3.0)
    add("qwen2 silu_mul", _timed(lambda: silu_mul(gu)), bytes_=T * ff * 2 * 3.0)
    # ---- recurrent mixers (no like kernel in Qwen2; fp32 vector flops / state bytes)
    pr = torch.randn(T, 4 * H * D, device=dev).to(bf)
    dec = torch.full((H,), 0.99, device=dev)
    S = torch.zeros(B + 1, H, D, D, device=dev)
    add("decay_attn_scan prefill", _timed(lambda: decay_attention(pr, 0, H * D, 2 * H * D, dec, S, meta, H, D, D), 3, 1),
        flops=4.0 * T * H * D * D, bytes_=T * 3 * H * D * 2.0, peak=VALU_F32)
    prd = torch.randn(B, 4 * H * D, device=dev).to(bf)
    add("decay_attn_scan decode", _timed(lambda: decay_attention(prd, 0, H * D, 2 * H * D, dec, S, dmeta, H, D, D)),
        bytes_=2.0 * B * H * D * D * 4)
    o = torch.randn(T, H * D, device=dev)
    out = torch.empty(T, H * D, device=dev, dtype=bf)
    add("gated_rmsnorm", _timed(lambda: gated_rmsnorm(o, w32[: H * D].contiguous(), pr, 3 * H * D, 1e-5, out)),
        bytes_=T * H * D * (4 + 2 + 2.0))
    gp = torch.randn(T, 3 * W, device=dev).to(bf)
    Sg = torch.zeros(B + 1, W, device=dev)
    add("mingru_scan prefill", _timed(lambda: mingru_scan(gp, 0, W, 2 * W, b32, b32, Sg, meta, W)), bytes_=T * W * 2 * 4.0)
    gpd = torch.randn(B, 3 * W, device=dev).to(bf)
    add("mingru_scan decode", _timed(lambda: mingru_scan(gpd, 0, W, 2 * W, b32, b32, Sg, dmeta, W)),
        bytes_=B * W * (2 * 4 + 8.0))
    return rows


def _namudra_kernel_table(dev, H=28, G=4, D=128, W=3584, T=2048, B=64, ctx=2048, bs=16, win=1024, R=192, r=64, S=2):
    """[(kernel, seconds, bound, fraction of roofline)] for Namudra's kernels and the like kernels of Zofesun."""
    from ..ops.attention import AttnMetadata, sigmoid_window_attention, sink_attention
    from ..ops.elementwise import latent_store, qk_norm_store, rope_table, rope_vnorm_store
    from ..ops.norm import dyt_residual, hyper_mix, rmsnorm_rows
    from ..ops.recurrent import decay_attention, gated_rmsnorm

    bf = torch.bfloat16
    i32 = dict(dtype=torch.int32, device=dev)
    rows = []

    def add(name, sec, flops=0.0, bytes_=0.0, peak=MFMA_BF16):
        t_c, t_m = flops / peak, bytes_ / HBM_BPS
        rows.append({"kernel": name, "us": round(sec * 1e6, 1), "bound": "flops" if t_c >= t_m else "bytes",
                     "roofline_fraction": round(max(t_c, t_m) / sec, 4)})

    nb = T // bs
    meta = AttnMetadata(q_start=torch.tensor([0, T], **i32), ctx_len=torch.tensor([T], **i32),
                        block_tables=(torch.arange(nb, **i32) + 1).view(1, nb), slot_mapping=torch.arange(T, **i32) + bs,
                        max_q_len=T, num_seqs=1, num_tokens=T, state_slots=torch.tensor([0], **i32))
    nbd = ctx // bs
    part_o = torch.empty(8 * B * H * max(D, R), device=dev)
    part_ml = torch.empty(8 * B * H * 2, device=dev)
    dmeta = AttnMetadata(q_start=torch.arange(B + 1, **i32), ctx_len=torch.full((B,), ctx, **i32),
                         block_tables=(torch.arange(B * nbd, **i32) + 1).view(B, nbd), slot_mapping=None, max_q_len=1,
                         num_seqs=B, num_tokens=B, is_decode=True, num_splits=8, split_len=ctx // 8, part_o=part_o,
                         part_ml=part_ml, state_slots=torch.arange(B, **i32))
    # ---- prefill attention, one prompt of T tokens: windowed sigmoid | latent (one kv head, key R + r, value R) | sink
    kc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    vc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    q = torch.randn(T, H, D, device=dev).to(bf)
    gate = torch.randn(T, H * D, device=dev).to(bf)
    pb = torch.zeros(H, device=dev)
    pairs = T * (T + 1) / 2 - (T - win) * (T - win + 1) / 2  # visible (query, key) pairs
    add("sigmoid_window_prefill (window 1024)", _timed(lambda: sigmoid_window_attention(q, kc, vc, meta, 0.09, pb, win, gate=gate)),
        flops=4.0 * pairs * H * D)
    add("zofesun sink_attn_prefill", _timed(lambda: sink_attention(q, kc, vc, meta, 0.09, pb)), flops=4.0 * T * T / 2 * H * D)
    kl = torch.randn(nb + 1, 1, bs, R + r, device=dev).to(bf)
    vl = kl[..., :R]
    ql = torch.randn(T, H, R + r, device=dev).to(bf)
    add("latent attention prefill (sink kernel, no sink)", _timed(lambda: sink_attention(ql, kl, vl, meta, 0.06, None)),
        flops=2.0 * T * T / 2 * H * (2 * R + r))
    # ---- decode attention: B rows of ctx keys
    kd = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    vd_ = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    qd = torch.randn(B, H, D, device=dev).to(bf)
    gd = torch.randn(B, H * D, device=dev).to(bf)
    add("sigmoid_window_decode (window 1024)", _timed(lambda: sigmoid_window_attention(qd, kd, vd_, dmeta, 0.09, pb, win, gate=gd)),
        bytes_=2.0 * B * win * G * D * 2)
    add("zofesun sink_attn_decode", _timed(lambda: sink_attention(qd, kd, vd_, dmeta, 0.09, pb)), bytes_=2.0 * B * ctx * G * D * 2)
    kld = torch.randn(B * nbd + 1, 1, bs, R + r, device=dev).to(bf)
    vld = kld[..., :R]
    qld = torch.randn(B, H, R + r, device=dev).to(bf)
    add("latent attention decode (sink kernel, no sink)", _timed(lambda: sink_attention(qld, kld, vld, dmeta, 0.06, None)),
        bytes_=B * ctx * (R + r) * 2.0)
    # ---- projection post-processing + cache stores
    proj = torch.randn(T, (2 * H + G) * D, device=dev).to(bf)
    ones = torch.ones(D, device=dev)
    add("qk_norm_store", _timed(lambda: qk_norm_store(proj, 0, H * D, ones, ones, meta.slot_mapping, kc, vc, H, G, D, 1e-6)),
        bytes_=T * (2 * H + 3 * G) * D * 2.0)
    pos = torch.arange(T, **i32)
    tab = rope_table(T, D, 1e4, dev)
    add("zofesun rope_vnorm_store", _timed(lambda: rope_vnorm_store(proj, 0, H * D, (H + G) * D, pos, tab, meta.slot_mapping, kc, vc,
                                                                    H, G, D, D, D, 1e-5)), bytes_=T * (H + 2 * G) * D * 2 * 2.0)
    ckv = torch.randn(T, R + r, device=dev).to(bf)
    tabr = rope_table(T, r, 1e4, dev)
    wR, wq4 = torch.ones(R, device=dev), torch.ones(W // 4, device=dev)
    add("latent_store", _timed(lambda: latent_store(ckv, wR, pos, tabr, meta.slot_mapping, ql, kl, 1e-6)),
        bytes_=T * ((R + r) * 2 + 2 * H * r) * 2.0)
    cq = torch.randn(T, 2 * (W // 4), device=dev).to(bf)
    add("rmsnorm_rows (query latent)", _timed(lambda: rmsnorm_rows(cq[:, : W // 4], wq4, 1e-6)),
        bytes_=T * (W // 4) * 2 * 2.0)
    # ---- sublayer boundary: S fp32 streams | one fp32 stream
    xs = torch.randn(S, T, W, device=dev)
    y = torch.randn(T, W, device=dev).to(bf)
    mix, oc, ic, w32 = torch.eye(S, device=dev), torch.ones(S, device=dev), torch.ones(S, device=dev) / S, torch.ones(W, device=dev)
    add(f"hyper_mix ({S} fp32 streams)", _timed(lambda: hyper_mix(xs, y, mix, oc, ic, w32, 1e-6)), bytes_=T * W * (2 + 8.0 * S + 2))
    resid = torch.randn(T, W, device=dev)
    b32 = torch.zeros(W, device=dev)
    add("zofesun dyt_residual (one fp32 stream)", _timed(lambda: dyt_residual(resid, y, (0.5, w32, b32), pre=(0.5, w32, b32))),
        bytes_=T * W * (2 + 4 + 4 + 2.0))
    # ---- retention scan (rotary, no activation) | decay scan (SiLU) ; per-head | whole-row gated norm
    pr = torch.randn(T, 4 * H * D, device=dev).to(bf)
    dec = torch.full((H,), 0.99, device=dev)
    St = torch.zeros(B + 1, H, D, D, device=dev)
    add("retention scan prefill", _timed(lambda: decay_attention(pr, 0, H * D, 2 * H * D, dec, St, meta, H, D, D, act=False,
                                                                positions=pos, rope=tab, k_scale=D ** -0.5), 3, 1),
        flops=4.0 * T * H * D * D, bytes_=T * 3 * H * D * 2.0, peak=VALU_F32)
    add("zofesun decay_attn_scan prefill", _timed(lambda: decay_attention(pr, 0, H * D, 2 * H * D, dec, St, meta, H, D, D), 3, 1),
        flops=4.0 * T * H * D * D, bytes_=T * 3 * H * D * 2.0, peak=VALU_F32)
    prd = torch.randn(B, 4 * H * D, device=dev).to(bf)
    posd = torch.full((B,), ctx - 1, **i32)
    add("retention scan decode", _timed(lambda: decay_attention(prd, 0, H * D, 2 * H * D, dec, St, dmeta, H, D, D, act=False,
                                                               positions=posd, rope=tab, k_scale=D ** -0.5)),
        bytes_=2.0 * B * H * D * D * 4)
    add("zofesun decay_attn_scan decode", _timed(lambda: decay_attention(prd, 0, H * D, 2 * H * D, dec, St, dmeta, H, D, D)),
        bytes_=2.0 * B * H * D * D * 4)
    o = torch.randn(T, H * D, device=dev)
    out = torch.empty(T, H * D, device=dev, dtype=bf)
    add("gated_rmsnorm per head, SiLU gate", _timed(lambda: gated_rmsnorm(o, None, pr, 3 * H * D, 1e-6, out, groups=H, gate="silu")),
        bytes_=T * H * D * (4 + 2 + 2.0))
    add("zofesun gated_rmsnorm whole row", _timed(lambda: gated_rmsnorm(o, w32[: H * D].contiguous(), pr, 3 * H * D, 1e-5, out)),
        bytes_=T * H * D * (4 + 2 + 2.0))
    return rows


def _leripel_models(name, dev):
    """Leripel at a bench size: per four layers retention, block-local attention (blocks of 1024), the state-space
    mixer, block-local attention; every layer beside a mixture of 16 experts (4 per token) plus a shared expert whose
    active width equals the dense decoders' feed-forward; beside the Namudra and Qwen2 stacks."""
    from ..models.configs import leripel_config
    from ..models.leripel import LeripelModel

    W, H, G, D, ff, nl, _ = SIZES[name]
    per = (ff // 5) // 64 * 64
    lc = leripel_config(f"leripel-{name}", VOCAB, W, ("rama" * nl)[:nl], heads=H, kv_heads=G, dim=D, chunk=1024,
                        ssm_vdim=64, ssm_state=128, experts=16, top=4, groups=(4, 2), ff=per, shared_ff=ff - 4 * per)
    mk_n, _, mk_q = _namudra_models(name, dev)
    return (lambda: LeripelModel(lc, device=dev, seed=1)), mk_n, mk_q


def _leripel_kernel_table(dev, H=28, G=4, D=128, W=3584, ff=18944, T=2048, B=64, ctx=2048, bs=16, chunk=1024, E=16,
                          top=4, P=64, N=128):
    """[(kernel, seconds, bound, fraction of roofline)] for Leripel's kernels and the like kernels of Namudra."""
    from ..ops.attention import AttnMetadata, sigmoid_window_attention, sink_attention
    from ..ops.elementwise import rope_table, rope_vnorm_store
    from ..ops.linear import linear
    from ..ops.moe import moe_experts, moe_route
    from ..ops.norm import hyper_mix, residual_rmsnorm
    from ..ops.recurrent import causal_conv, decay_attention, gated_rmsnorm, ssm_scan

    bf = torch.bfloat16
    i32 = dict(dtype=torch.int32, device=dev)
    rows = []

    def add(name, sec, flops=0.0, bytes_=0.0, peak=MFMA_BF16):
        t_c, t_m = flops / peak, bytes_ / HBM_BPS
        rows.append({"kernel": name, "us": round(sec * 1e6, 1), "bound": "flops" if t_c >= t_m else "bytes",
                     "roofline_fraction": round(max(t_c, t_m) / sec, 4)})

    nb = T // bs
    meta = AttnMetadata(q_start=torch.tensor([0, T], **i32), ctx_len=torch.tensor([T], **i32),
                        block_tables=(torch.arange(nb, **i32) + 1).view(1, nb), slot_mapping=torch.arange(T, **i32) + bs,
                        max_q_len=T, num_seqs=1, num_tokens=T, state_slots=torch.tensor([0], **i32))
    nbd = ctx // bs
    dmeta = AttnMetadata(q_start=torch.arange(B + 1, **i32), ctx_len=torch.full((B,), ctx, **i32),
                         block_tables=(torch.arange(B * nbd, **i32) + 1).view(B, nbd), slot_mapping=None, max_q_len=1,
                         num_seqs=B, num_tokens=B, is_decode=True, state_slots=torch.arange(B, **i32))
    # ---- attention: blocks of `chunk` positions, temperatures, head gates | sliding window of the same length
    kc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    vc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    q = torch.randn(T, H, D, device=dev).to(bf)
    temp, pb = torch.ones(H, device=dev), torch.zeros(H, device=dev)
    hg = torch.randn(T, H, device=dev).to(bf)
    gate = torch.randn(T, H * D, device=dev).to(bf)
    pairs_c = (T // chunk) * chunk * (chunk + 1) / 2
    pairs_w = T * (T + 1) / 2 - (T - chunk) * (T - chunk + 1) / 2
    add(f"block-local attention prefill (blocks of {chunk})",
        _timed(lambda: sink_attention(q, kc, vc, meta, 0.09, None, head_scale=temp, head_gate=hg, chunk=chunk)),
        flops=4.0 * pairs_c * H * D)
    add("namudra sigmoid_window_prefill (window 1024)",
        _timed(lambda: sigmoid_window_attention(q, kc, vc, meta, 0.09, pb, chunk, gate=gate)), flops=4.0 * pairs_w * H * D)
    kd = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    vd_ = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    qd = torch.randn(B, H, D, device=dev).to(bf)
    hgd = torch.randn(B, H, device=dev).to(bf)
    gd = torch.randn(B, H * D, device=dev).to(bf)
    dmeta.ctx_len = torch.full((B,), ctx, **i32)  # the last token closes a block: a full block of keys is read
    add(f"block-local attention decode ({chunk} keys)",
        _timed(lambda: sink_attention(qd, kd, vd_, dmeta, 0.09, None, head_scale=temp, head_gate=hgd, chunk=chunk)),
        bytes_=2.0 * B * chunk * G * D * 2)
    add("namudra sigmoid_window_decode (window 1024)",
        _timed(lambda: sigmoid_window_attention(qd, kd, vd_, dmeta, 0.09, pb, chunk, gate=gd)), bytes_=2.0 * B * chunk * G * D * 2)
    # ---- rotary + K/V store
    proj = torch.randn(T, (H + 2 * G) * D + 32, device=dev).to(bf)
    pos = torch.arange(T, **i32)
    tab, tabh = rope_table(T, D, 1e4, dev), rope_table(T, D // 2, 1e4, dev)
    by = T * (H + 2 * G) * D * 2 * 2.0
    add("rope store, adjacent pairs, half the head", _timed(lambda: rope_vnorm_store(
        proj, 0, H * D, (H + G) * D, pos, tabh, meta.slot_mapping, kc, vc, H, G, D, D, D // 2, 1e-5, interleaved=True,
        vnorm=False)), bytes_=by)
    add("zofesun rope_vnorm_store", _timed(lambda: rope_vnorm_store(proj, 0, H * D, (H + G) * D, pos, tab, meta.slot_mapping,
                                                                    kc, vc, H, G, D, D, D, 1e-5)), bytes_=by)
    # ---- layer boundary: mixer + shared + `top` weighted experts into one fp32 residual | two fp32 streams
    x = torch.randn(T, W, device=dev)
    a, b = torch.randn(T, W, device=dev).to(bf), torch.randn(T, W, device=dev).to(bf)
    e = torch.randn(T, top, W, device=dev).to(bf)
    ec, bc, w32 = torch.rand(T, top, device=dev), torch.rand(T, device=dev), torch.ones(W, device=dev)
    add(f"residual_rmsnorm (mixer + shared + {top} experts)", _timed(lambda: residual_rmsnorm(x, a, b, bc, e, ec, w32, 1e-5)),
        bytes_=T * W * (8 + 2.0 * (2 + top) + 2))
    xs = torch.randn(2, T, W, device=dev)
    mix, oc, ic = torch.eye(2, device=dev), torch.ones(2, device=dev), torch.ones(2, device=dev) / 2
    add("namudra hyper_mix (2 fp32 streams)", _timed(lambda: hyper_mix(xs, a, mix, oc, ic, w32, 1e-6)), bytes_=T * W * (2 + 16.0 + 2))
    # ---- state-space mixer | retention scan
    Hs = W // P
    inner, ch = Hs * P, Hs * P + 2 * N
    ld = 2 * inner + 2 * N + Hs
    pj = (torch.randn(T, ld, device=dev) * 0.5).to(bf)
    cw, cb = torch.randn(ch, 4, device=dev) * 0.5, torch.zeros(ch, device=dev)
    cst = torch.zeros(B + 1, 3, ch, device=dev, dtype=bf)
    sst = torch.zeros(B + 1, Hs, N, P, device=dev)
    dtb, alog, dsk = torch.zeros(Hs, device=dev), torch.zeros(Hs, device=dev), torch.ones(Hs, device=dev)
    add("causal_conv prefill (4 taps)", _timed(lambda: causal_conv(pj, inner, cw, cb, cst, meta)), bytes_=T * ch * 2 * 2.0)
    xbc = causal_conv(pj, inner, cw, cb, cst, meta)
    add("ssm_scan prefill", _timed(lambda: ssm_scan(xbc, pj, inner + ch, dtb, alog, dsk, sst, meta, Hs, 1, N, P), 3, 1),
        flops=4.0 * T * Hs * N * P, bytes_=T * ch * 2.0, peak=VALU_F32)
    pr = torch.randn(T, 4 * H * D, device=dev).to(bf)
    dec = torch.full((H,), 0.99, device=dev)
    St = torch.zeros(B + 1, H, D, D, device=dev)
    add("retention scan prefill (no rotary)", _timed(lambda: decay_attention(pr, 0, H * D, 2 * H * D, dec, St, meta, H, D, D, act=False,
                                                                             k_scale=D ** -0.5), 3, 1),
        flops=4.0 * T * H * D * D, bytes_=T * 3 * H * D * 2.0, peak=VALU_F32)
    pjd = (torch.randn(B, ld, device=dev) * 0.5).to(bf)
    add("causal_conv decode", _timed(lambda: causal_conv(pjd, inner, cw, cb, cst, dmeta)), bytes_=B * ch * 2 * (2 + 2 * 3.0))
    xbd = causal_conv(pjd, inner, cw, cb, cst, dmeta)
    add("ssm_scan decode", _timed(lambda: ssm_scan(xbd, pjd, inner + ch, dtb, alog, dsk, sst, dmeta, Hs, 1, N, P)),
        bytes_=2.0 * B * Hs * N * P * 4)
    prd = torch.randn(B, 4 * H * D, device=dev).to(bf)
    add("retention scan decode", _timed(lambda: decay_attention(prd, 0, H * D, 2 * H * D, dec, St, dmeta, H, D, D, act=False,
                                                               k_scale=D ** -0.5)), bytes_=2.0 * B * H * D * D * 4)
    o = torch.randn(T, inner, device=dev)
    out = torch.empty(T, inner, device=dev, dtype=bf)
    add("gated_rmsnorm, gate first, whole row", _timed(lambda: gated_rmsnorm(o, w32[:inner].contiguous(), pj, 0, 1e-5, out, gate="silu",
                                                                             gate_first=True)), bytes_=T * inner * (4 + 2 + 2.0))
    o2 = torch.randn(T, H * D, device=dev)
    out2 = torch.empty(T, H * D, device=dev, dtype=bf)
    add("namudra gated_rmsnorm per head", _timed(lambda: gated_rmsnorm(o2, None, pr, 3 * H * D, 1e-6, out2, groups=H, gate="silu")),
        bytes_=T * H * D * (4 + 2 + 2.0))
    # ---- experts: router, grouped GEMMs | dense GEMMs of the same active width through the engine's linear()
    F = (ff // 5) // 64 * 64
    h = torch.randn(T, W, device=dev).to(bf)
    wr = torch.randn(E + 1, W, device=dev) * 0.05
    add("moe_route (16 experts + gate row)", _timed(lambda: moe_route(h, wr, E, top, 4, 2)), flops=2.0 * T * (E + 1) * W,
        bytes_=T * W * 2.0, peak=VALU_F32)
    ids, _, _ = moe_route(h, wr, E, top, 4, 2)
    wgu = (torch.randn(E, 2 * F, W, device=dev) * 0.02).to(bf)
    wd = (torch.randn(E, W, F, device=dev) * 0.02).to(bf)
    add(f"moe experts prefill ({T} x {top} rows, align + 2 grouped GEMMs)", _timed(lambda: moe_experts(h, ids, wgu, wd)),
        flops=6.0 * T * top * F * W)
    wgd, wdd = (torch.randn(2 * top * F, W, device=dev) * 0.02).to(bf), (torch.randn(W, top * F, device=dev) * 0.02).to(bf)
    hh = torch.randn(T, top * F, device=dev).to(bf)
    add("dense gate|up + down GEMMs of the same active width (linear)",
        _timed(lambda: (linear(h, wgd), linear(hh, wdd))), flops=6.0 * T * top * F * W)
    hd = torch.randn(B, W, device=dev).to(bf)
    idd, _, _ = moe_route(hd, wr, E, top, 4, 2)
    add(f"moe experts decode ({B} x {top} rows)", _timed(lambda: moe_experts(hd, idd, wgu, wd)), bytes_=3.0 * E * F * W * 2)
    hhd = torch.randn(B, top * F, device=dev).to(bf)
    add("dense gate|up + down GEMMs, decode rows (linear)", _timed(lambda: (linear(hd, wgd), linear(hhd, wdd))),
        bytes_=3.0 * top * F * W * 2)
    return rows


def _pubulix_models(name, dev):
    """Pubulix at a bench size: per four layers capped sliding-window attention (window 1024), latent attention with
    its own cache (window 2048), attention again, latent attention over the same cache; every layer with 16
    table-routed experts (4 per token) whose active width equals the dense decoders' feed-forward, an input
    convolution of 4 taps and gated residual branches; beside the Leripel and Qwen2 stacks."""
    from ..models.configs import pubulix_config
    from ..models.pubulix import PubulixModel

    W, H, G, D, ff, nl, _ = SIZES[name]
    pc = pubulix_config(f"pubulix-{name}", VOCAB, W, ("alas" * nl)[:nl], heads=H, kv_heads=G, dim=D, window=1024,
                        lat_heads=H, kv_rank=192, rot_dim=64, lat_window=2048, experts=16, top=4, ff=(ff // 4) // 64 * 64)
    mk_l, _, mk_q = _leripel_models(name, dev)
    return (lambda: PubulixModel(pc, device=dev, seed=1)), mk_l, mk_q


def _pubulix_kernel_table(dev, H=28, G=4, D=128, W=3584, ff=18944, T=2048, B=64, ctx=2048, bs=16, win=1024, lwin=2048,
                          R=192, r=64, E=16, top=4, V=VOCAB):
    """[(kernel, seconds, bound, fraction of roofline)] for Pubulix's kernels and the like kernels of Leripel (attention,
    convolution, boundary, experts) and Namudra (latent attention)."""
    from ..ops.attention import AttnMetadata, sink_attention
    from ..ops.elementwise import latent_rope_store, latent_store, rope_table, tanh_cap_
    from ..ops.linear import linear
    from ..ops.moe import head_project, moe_experts, moe_route, moe_table_route
    from ..ops.norm import residual_rmsnorm
    from ..ops.recurrent import causal_conv

    bf = torch.bfloat16
    i32 = dict(dtype=torch.int32, device=dev)
    rows = []

    def add(name, sec, flops=0.0, bytes_=0.0, peak=MFMA_BF16):
        t_c, t_m = flops / peak, bytes_ / HBM_BPS
        rows.append({"kernel": name, "us": round(sec * 1e6, 1), "bound": "flops" if t_c >= t_m else "bytes",
                     "roofline_fraction": round(max(t_c, t_m) / sec, 4)})

    nb = T // bs
    meta = AttnMetadata(q_start=torch.tensor([0, T], **i32), ctx_len=torch.tensor([T], **i32),
                        block_tables=(torch.arange(nb, **i32) + 1).view(1, nb), slot_mapping=torch.arange(T, **i32) + bs,
                        max_q_len=T, num_seqs=1, num_tokens=T, state_slots=torch.tensor([0], **i32))
    nbd = ctx // bs
    dmeta = AttnMetadata(q_start=torch.arange(B + 1, **i32), ctx_len=torch.full((B,), ctx, **i32),
                         block_tables=(torch.arange(B * nbd, **i32) + 1).view(B, nbd), slot_mapping=None, max_q_len=1,
                         num_seqs=B, num_tokens=B, is_decode=True, state_slots=torch.arange(B, **i32))
    # ---- attention: a window of `win` positions with capped scores | leripel's blocks of the same length
    kc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    vc = torch.randn(nb + 1, G, bs, D, device=dev).to(bf)
    q = torch.randn(T, H, D, device=dev).to(bf)
    temp = torch.ones(H, device=dev)
    hg = torch.randn(T, H, device=dev).to(bf)
    pairs_w = T * (T + 1) / 2 - (T - win) * (T - win + 1) / 2
    pairs_c = (T // win) * win * (win + 1) / 2
    add(f"capped window attention prefill (window {win})",
        _timed(lambda: sink_attention(q, kc, vc, meta, 0.09, None, window=win, softcap=50.0)), flops=4.0 * pairs_w * H * D)
    add(f"leripel block-local attention prefill (blocks of {win})",
        _timed(lambda: sink_attention(q, kc, vc, meta, 0.09, None, head_scale=temp, head_gate=hg, chunk=win)),
        flops=4.0 * pairs_c * H * D)
    kd = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    vd_ = torch.randn(B * nbd + 1, G, bs, D, device=dev).to(bf)
    qd = torch.randn(B, H, D, device=dev).to(bf)
    hgd = torch.randn(B, H, device=dev).to(bf)
    add(f"capped window attention decode ({win} keys)",
        _timed(lambda: sink_attention(qd, kd, vd_, dmeta, 0.09, None, window=win, softcap=50.0)),
        bytes_=2.0 * B * win * G * D * 2)
    add(f"leripel block-local attention decode ({win} keys)",
        _timed(lambda: sink_attention(qd, kd, vd_, dmeta, 0.09, None, head_scale=temp, head_gate=hgd, chunk=win)),
        bytes_=2.0 * B * win * G * D * 2)
    # ---- latent attention: a window and a sink over latent | rotated rows | namudra's causal form on the same rows
    lk = torch.randn(nb + 1, 1, bs, R + r, device=dev).to(bf)
    lq = torch.randn(T, H, R + r, device=dev).to(bf)
    sink = torch.zeros(H, device=dev)
    pairs_l = T * (T + 1) / 2 - max(0, T - lwin) * (max(0, T - lwin) + 1) / 2
    add(f"latent attention prefill (window {lwin}, sink)",
        _timed(lambda: sink_attention(lq, lk, lk[..., :R], meta, 0.06, sink, window=lwin)),
        flops=2.0 * pairs_l * H * (2 * R + r))
    add("namudra latent attention prefill (causal)", _timed(lambda: sink_attention(lq, lk, lk[..., :R], meta, 0.06, None)),
        flops=2.0 * (T * (T + 1) / 2) * H * (2 * R + r))
    lkd = torch.randn(B * nbd + 1, 1, bs, R + r, device=dev).to(bf)
    lqd = torch.randn(B, H, R + r, device=dev).to(bf)
    add(f"latent attention decode ({min(ctx, lwin)} keys, sink)",
        _timed(lambda: sink_attention(lqd, lkd, lkd[..., :R], dmeta, 0.06, sink, window=lwin)),
        bytes_=1.0 * B * min(ctx, lwin) * (R + r) * 2)
    add(f"namudra latent attention decode ({ctx} keys)",
        _timed(lambda: sink_attention(lqd, lkd, lkd[..., :R], dmeta, 0.06, None)), bytes_=1.0 * B * ctx * (R + r) * 2)
    # ---- queries + cache row out of the fused projection | namudra's in-place form
    ld = H * (R + r) + (R + r) + H * D
    proj = torch.randn(T, ld, device=dev).to(bf)
    pos = torch.arange(T, **i32)
    tab = rope_table(T, r, 1e4, dev)
    cw = torch.ones(R, device=dev)
    add("latent_rope_store (queries copied and rotated, cache row)", _timed(lambda: latent_rope_store(
        proj, 0, H * (R + r), cw, pos, tab, meta.slot_mapping, lk, H, 1e-5, interleaved=True)),
        bytes_=T * (H + 1) * (R + r) * 2 * 2.0)
    ckv = torch.randn(T, R + r, device=dev).to(bf)
    add("namudra latent_store (queries rotated in place)", _timed(lambda: latent_store(ckv, cw, pos, tab, meta.slot_mapping,
                                                                                        lq, lk, 1e-5)),
        bytes_=T * (R + r) * 2 * 2.0 + T * H * r * 2 * 2.0)
    # ---- one value matrix per head + gate | one dense GEMM of the same flops through linear()
    o = torch.randn(T, H * R, device=dev).to(bf)
    wuv = (torch.randn(H, D, R, device=dev) * 0.05).to(bf)
    gcol = proj[:, H * (R + r) + (R + r):]
    add(f"head_project prefill ({H} matrices {D} x {R}, gate)", _timed(lambda: head_project(o, wuv, gate=gcol)),
        flops=2.0 * T * H * D * R, bytes_=T * H * (R + 2 * D) * 2.0)
    wdn = (torch.randn(D, H * R, device=dev) * 0.02).to(bf)
    add("dense GEMM of the same flops (linear)", _timed(lambda: linear(o, wdn)), flops=2.0 * T * H * D * R,
        bytes_=T * H * R * 2.0)
    od = torch.randn(B, H * R, device=dev).to(bf)
    gd = torch.randn(B, H * D, device=dev).to(bf)
    add("head_project decode rows", _timed(lambda: head_project(od, wuv, gate=gd)), bytes_=H * D * R * 2.0)
    add("dense GEMM of the same weight bytes, decode rows (linear)", _timed(lambda: linear(od, wdn)), bytes_=H * D * R * 2.0)
    # ---- sublayer boundary: gated branch | leripel's ungated sum of the same operands
    x = torch.randn(T, W, device=dev)
    a = torch.randn(T, W, device=dev).to(bf)
    gt = torch.randn(T, W, device=dev).to(bf)
    e = torch.randn(T, top, W, device=dev).to(bf)
    ec, gb, w32 = torch.rand(T, top, device=dev), torch.zeros(W, device=dev), torch.ones(W, device=dev)
    add("residual_rmsnorm (gated mixer branch)", _timed(lambda: residual_rmsnorm(x, a, w=w32, eps=1e-5, gate=gt, gbias=gb, mult=0.5)),
        bytes_=T * W * (8 + 2.0 * 2 + 2))
    add("leripel residual_rmsnorm (one branch)", _timed(lambda: residual_rmsnorm(x, a, w=w32, eps=1e-5)),
        bytes_=T * W * (8 + 2.0 + 2))
    add(f"residual_rmsnorm (gated sum of {top} experts)",
        _timed(lambda: residual_rmsnorm(x, e=e, ecoef=ec, w=w32, eps=1e-5, gate=gt, gbias=gb, mult=0.5)),
        bytes_=T * W * (8 + 2.0 * (1 + top) + 2))
    add(f"leripel residual_rmsnorm (sum of {top} experts)", _timed(lambda: residual_rmsnorm(x, e=e, ecoef=ec, w=w32, eps=1e-5)),
        bytes_=T * W * (8 + 2.0 * top + 2))
    # ---- input convolution (no activation, input added) | leripel's SiLU form over the same channels
    h = torch.randn(T, W, device=dev).to(bf)
    cwt = torch.randn(W, 4, device=dev) * 0.3
    cst = torch.zeros(B + 1, 3, W, device=dev, dtype=bf)
    add("input convolution prefill (4 taps, h + conv(h))", _timed(lambda: causal_conv(h, 0, cwt, None, cst, meta, act=False, residual=True)),
        bytes_=T * W * 2 * 2.0)
    add("leripel causal_conv prefill (4 taps, SiLU)", _timed(lambda: causal_conv(h, 0, cwt, None, cst, meta)), bytes_=T * W * 2 * 2.0)
    hd = torch.randn(B, W, device=dev).to(bf)
    add("input convolution decode", _timed(lambda: causal_conv(hd, 0, cwt, None, cst, dmeta, act=False, residual=True)),
        bytes_=B * W * 2 * (2 + 2 * 3.0))
    add("leripel causal_conv decode", _timed(lambda: causal_conv(hd, 0, cwt, None, cst, dmeta)), bytes_=B * W * 2 * (2 + 2 * 3.0))
    # ---- experts: table routing, clamped units | leripel's router and SiLU units on the same grouped GEMM
    F = (ff // 4) // 64 * 64
    table = torch.rand(V, E, device=dev).argsort(1)[:, :top].to(torch.int32).contiguous()
    tok = torch.randint(0, V, (T,), device=dev).to(torch.int32)
    wr = torch.randn(E, W, device=dev) * 0.05
    add("moe_table_route", _timed(lambda: moe_table_route(tok, table)), bytes_=T * (4 + top * 12.0))
    add("leripel moe_route (16 experts)", _timed(lambda: moe_route(h, wr, E, top, 4, 2)), flops=2.0 * T * E * W, bytes_=T * W * 2.0,
        peak=VALU_F32)
    ids, _ = moe_table_route(tok, table)
    wgu = (torch.randn(E, 2 * F, W, device=dev) * 0.02).to(bf)
    wd = (torch.randn(E, W, F, device=dev) * 0.02).to(bf)
    add(f"clamped experts prefill ({T} x {top} rows)", _timed(lambda: moe_experts(h, ids, wgu, wd, 7.0, 1.702, 1.0)),
        flops=6.0 * T * top * F * W)
    add(f"leripel SiLU experts prefill ({T} x {top} rows)", _timed(lambda: moe_experts(h, ids, wgu, wd)), flops=6.0 * T * top * F * W)
    idd, _ = moe_table_route(tok[:B].contiguous(), table)
    add(f"clamped experts decode ({B} x {top} rows)", _timed(lambda: moe_experts(hd, idd, wgu, wd, 7.0, 1.702, 1.0)),
        bytes_=3.0 * E * F * W * 2)
    add(f"leripel SiLU experts decode ({B} x {top} rows)", _timed(lambda: moe_experts(hd, idd, wgu, wd)), bytes_=3.0 * E * F * W * 2)
    # ---- logit cap
    lg = torch.randn(B, V, device=dev).to(bf)
    add(f"tanh_cap ({B} x {V} logits)", _timed(lambda: tanh_cap_(lg, 30.0)), bytes_=B * V * 2 * 2.0)
    return rows


def run_pubulix(args) -> dict:
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    sizes = {}
    for name in SIZES:
        makers = dict(zip(("pubulix", "leripel", "qwen2"), _pubulix_models(name, dev)))
        cell = {}
        for batch, plen, glen in ((8, 2048, 64), (64, 1024, 64)):
            key = f"B{batch}_P{plen}_G{glen}"
            cell[key] = {k: _engine_numbers(mk, dev, batch, plen, glen) for k, mk in makers.items()}
            print(json.dumps({"size": name, "shape": key, **cell[key]}), flush=True)
        sizes[name] = cell
    kernels = _pubulix_kernel_table(dev)
    for r in kernels:
        print(json.dumps(r), flush=True)
    return {"metric": "pubulix_vs_leripel_vs_qwen2_tokens_per_s", "unit": "tokens/s", "dtype": "bf16",
            "data": "synthetic", "sizes": sizes, "kernels": kernels}


def run_leripel(args) -> dict:
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    sizes = {}
    for name in SIZES:
        makers = dict(zip(("leripel", "namudra", "qwen2"), _leripel_models(name, dev)))
        cell = {}
        for batch, plen, glen in ((8, 2048, 64), (64, 1024, 64)):
            key = f"B{batch}_P{plen}_G{glen}"
            cell[key] = {k: _engine_numbers(mk, dev, batch, plen, glen) for k, mk in makers.items()}
            print(json.dumps({"size": name, "shape": key, **cell[key]}), flush=True)
        sizes[name] = cell
    kernels = _leripel_kernel_table(dev)
    for r in kernels:
        print(json.dumps(r), flush=True)
    return {"metric": "leripel_vs_namudra_vs_qwen2_tokens_per_s", "unit": "tokens/s", "dtype": "bf16",
            "data": "synthetic", "sizes": sizes, "kernels": kernels}


def run_namudra(args) -> dict:
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    sizes = {}
    for name in SIZES:
        makers = dict(zip(("namudra", "zofesun", "qwen2"), _namudra_models(name, dev)))
        cell = {}
        for batch, plen, glen in ((8, 2048, 64), (64, 1024, 64)):
            key = f"B{batch}_P{plen}_G{glen}"
            cell[key] = {k: _engine_numbers(mk, dev, batch, plen, glen) for k, mk in makers.items()}
            print(json.dumps({"size": name, "shape": key, **cell[key]}), flush=True)
        sizes[name] = cell
    kernels = _namudra_kernel_table(dev)
    for r in kernels:
        print(json.dumps(r), flush=True)
    return {"metric": "namudra_vs_zofesun_vs_qwen2_tokens_per_s", "unit": "tokens/s", "dtype": "bf16",
            "data": "synthetic", "sizes": sizes, "kernels": kernels}


def run(args) -> dict:
    if getattr(args, "hybrid", None) == "namudra":
        return run_namudra(args)
    if getattr(args, "hybrid", None) == "leripel":
        return run_leripel(args)
    if getattr(args, "hybrid", None) == "pubulix":
        return run_pubulix(args)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    sizes = {}
    for name in SIZES:
        mk_z, mk_q = _models(name, dev)
        cell = {}
        for batch, plen, glen in ((8, 2048, 64), (64, 1024, 64)):
            key = f"B{batch}_P{plen}_G{glen}"
            cell[key] = {"zofesun": _engine_numbers(mk_z, dev, batch, plen, glen),
                         "qwen2": _engine_numbers(mk_q, dev, batch, plen, glen)}
            print(json.dumps({"size": name, "shape": key, **cell[key]}), flush=True)
        sizes[name] = cell
    kernels = _kernel_table(dev)
    for r in kernels:
        print(json.dumps(r), flush=True)
    return {"metric": "hybrid_vs_qwen2_tokens_per_s", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
            "sizes": sizes, "kernels": kernels}
