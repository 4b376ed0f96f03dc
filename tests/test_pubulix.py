"""Pubulix on the engine, CPU tier: the engine's cache / state / scheduler logic and the ops' host paths against
the float64 oracle (tests/pubulix_oracle.py); the same scenarios run on the HIP kernels in test_pubulix_gpu.py."""
import json

import numpy as np
import pytest
import torch

import pubulix_cases as C
import pubulix_oracle as O

TOL = 2e-5


def _meta(dev, lens, ctxs, slots, decode=False):
    """AttnMetadata of one step: sequences of ``lens`` new tokens behind ``ctxs`` - ``lens`` cached ones."""
    from githubrepostorag_amd.ops.attention import AttnMetadata

    i32 = dict(dtype=torch.int32, device=dev)
    qs = np.concatenate([[0], np.cumsum(lens)])
    return AttnMetadata(q_start=torch.tensor(qs.tolist(), **i32), ctx_len=torch.tensor(list(ctxs), **i32),
                        block_tables=torch.zeros(len(lens), 1, **i32), slot_mapping=torch.zeros(int(qs[-1]), **i32),
                        max_q_len=max(lens), num_seqs=len(lens), num_tokens=int(qs[-1]), is_decode=decode,
                        state_slots=torch.tensor(list(slots), **i32))


# ------------------------------------------------------------------------------------------------ mechanisms alone
def gated_boundary_case(device, dtype, tol):
    """x <- x + mult * sigmoid(gate + bias) * (branch | sum_k weight_k expert_k), then the RMS norm with one number
    as its weight; gate rows that are a column slice of a wider tensor."""
    from githubrepostorag_amd.ops.norm import residual_rmsnorm

    g = torch.Generator().manual_seed(1)
    for T, H, K, mult in ((5, 48, 2, 0.5), (3, 200, 0, 1.0), (2, 4100, 3, 0.25), (4, 9, 1, 2.0)):
        x = torch.randn(T, H, generator=g)
        a = torch.randn(T, H, generator=g).to(dtype)
        wide = torch.randn(T, 2 * H + 8, generator=g).to(dtype)
        gate = wide[:, 8:8 + H]
        gb, w = torch.randn(H, generator=g), torch.full((H,), 1.3)
        e = torch.randn(T, K, H, generator=g).to(dtype) if K else None
        ec = torch.rand(T, K, generator=g) if K else None
        y = (ec.double()[:, :, None] * e.double()).sum(1) if K else a.double()
        want = x.double() + mult * torch.sigmoid(gate.double() + gb.double()) * y
        dv = lambda t: None if t is None else t.to(device)
        xd = x.clone().to(device)
        wd = wide.to(device)
        h = residual_rmsnorm(xd, None if K else dv(a), e=dv(e), ecoef=dv(ec), w=dv(w), eps=1e-5, out_dtype=dtype,
                             gate=wd[:, 8:8 + H], gbias=dv(gb), mult=mult)
        assert float((xd.cpu().double() - want).abs().max()) < 2e-5 * max(1.0, float(want.abs().max()))
        hn = want / torch.sqrt((want * want).mean(-1, keepdim=True) + 1e-5) * 1.3
        assert float((h.cpu().double() - hn).abs().max()) < tol
    # no gate, mult alone
    x = torch.randn(3, 16, generator=g)
    a = torch.randn(3, 16, generator=g).to(dtype)
    xd = x.clone().to(device)
    residual_rmsnorm(xd, a.to(device), out_dtype=dtype, mult=0.5)
    assert float((xd.cpu().double() - (x.double() + 0.5 * a.double())).abs().max()) < 1e-5


def input_conv_case(device, dtype, tol):
    """h + conv(h) without activation over portions and single tokens of two sequences that share steps; the pool
    rows of a slot are those of the sequence that uses it now (a fresh sequence ignores what the slot held)."""
    from githubrepostorag_amd.ops.recurrent import causal_conv

    g = torch.Generator().manual_seed(2)
    for C_, taps in ((40, 3), (300, 1), (24, 5), (7, 2)):
        w = (0.5 * torch.randn(C_, taps, generator=g)).float()
        la, lb = 23, 9
        xa, xb = torch.randn(la, C_, generator=g).to(dtype), torch.randn(lb, C_, generator=g).to(dtype)
        want = {k: O.input_conv(x.double(), w.double()) for k, x in (("a", xa), ("b", xb))}
        pool = torch.full((3, taps - 1, C_), 7.0, dtype=dtype, device=device)  # stale contents everywhere
        got = {"a": [], "b": []}
        ca = cb = 0
        for na, nb in ((6, 2), (1, 1), (11, 0), (1, 5), (4, 1)):
            lens, ctxs, slots, rows, who = [], [], [], [], []
            for k, n, x, c, slot in (("a", na, xa, ca, 2), ("b", nb, xb, cb, 0)):
                if n:
                    lens.append(n); ctxs.append(c + n); slots.append(slot); rows.append(x[c:c + n]); who.append((k, n))
            m = _meta(device, lens, ctxs, slots, decode=max(lens) == 1)
            out = causal_conv(torch.cat(rows, 0).to(device), 0, w.to(device), None, pool, m, act=False, residual=True)
            o = 0
            for k, n in who:
                got[k].append(out[o:o + n].cpu())
                o += n
            ca += na
            cb += nb
        for k in got:
            assert float((torch.cat(got[k], 0).double() - want[k]).abs().max()) < tol, (C_, taps, k)


def latent_rows_case(device, dtype, tol):
    """The latent layer's cache row (normed latent | rotated part) and rotated queries out of one fused projection,
    in both pair layouts; a layer that stores nothing leaves the cache alone."""
    from githubrepostorag_amd.ops.elementwise import latent_rope_store, rope_table

    g = torch.Generator().manual_seed(3)
    for H, R, r, il in ((3, 20, 6, True), (1, 9, 2, True), (2, 136, 8, False), (5, 16, 16, True)):
        T, bs, eps = 11, 4, 1e-5
        qoff, coff = 8, 8 + H * (R + r) + 3
        proj = torch.randn(T, coff + R + r + 5, generator=g).to(dtype)
        cw = 1.0 + 0.2 * torch.randn(R, generator=g)
        pos = torch.randint(0, 50, (T,), generator=g).to(torch.int32)
        table = rope_table(64, r, 30.0, device)
        slots = torch.randperm(4 * bs, generator=g)[:T].to(torch.int32)
        slots[2] = -1
        kc = torch.zeros(4, 1, bs, R + r, dtype=dtype, device=device)
        q = latent_rope_store(proj.to(device), qoff, coff, cw.to(device), pos.to(device), table, slots.to(device), kc, H,
                              eps, interleaved=il)
        rot = O.rotate_adjacent if il else O.rotate_halves
        x = proj.double()
        for t in range(T):
            for h in range(H):
                row = x[t, qoff + h * (R + r): qoff + (h + 1) * (R + r)]
                want = torch.cat([row[:R], rot(row[R:], int(pos[t]), r, 30.0)])
                assert float((q[t, h].cpu().double() - want).abs().max()) < tol, (H, R, r, t, h)
            s = int(slots[t])
            if s < 0:
                continue
            c = O.rms_unit(x[t, coff:coff + R], eps) * cw.double()
            want = torch.cat([c, rot(x[t, coff + R:coff + R + r], int(pos[t]), r, 30.0)])
            assert float((kc[s // bs, 0, s % bs].cpu().double() - want).abs().max()) < tol * 4, (H, R, r, t)
        before = kc.clone()
        latent_rope_store(proj.to(device), qoff, None, None, pos.to(device), table, slots.to(device), kc, H, eps,
                          interleaved=il)
        assert torch.equal(before, kc)


def table_experts_case(device, dtype, tol):
    """Experts named by a table row per token id, the clamped unit, weights 1 / top -- summed by the boundary."""
    from githubrepostorag_amd.ops.moe import moe_experts, moe_table_route
    from githubrepostorag_amd.ops.norm import residual_rmsnorm

    g = torch.Generator().manual_seed(4)
    for T, W, F, E, top, V, limit in ((9, 32, 24, 5, 2, 17, 1.2), (4, 40, 8, 3, 3, 5, 0.4), (70, 16, 16, 4, 1, 9, 7.0),
                                      (400, 64, 32, 3, 2, 11, 1.0)):
        h = torch.randn(T, W, generator=g).to(dtype)
        wgu = (torch.randn(E, 2 * F, W, generator=g) * 2.0 * W ** -0.5).to(dtype)
        wd = (torch.randn(E, W, F, generator=g) * F ** -0.5).to(dtype)
        table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
        tok = torch.randint(0, V, (T,), generator=g).to(torch.int32)
        ids, wts = moe_table_route(tok.to(device), table.to(device))
        assert torch.equal(ids.cpu(), table[tok.long()]) and float((wts.cpu() - 1.0 / top).abs().max()) < 1e-7
        both = torch.stack([table, table.flip(0)]).contiguous()  # two layers' tables in one call
        ids2, wts2 = moe_table_route(tok.to(device), both.to(device))
        assert torch.equal(ids2[0].cpu(), table[tok.long()]) and torch.equal(ids2[1].cpu(), table.flip(0)[tok.long()])
        assert torch.equal(wts2.cpu(), wts.cpu())
        e = moe_experts(h.to(device), ids, wgu.to(device), wd.to(device), limit, 1.702, 1.0)
        x = torch.zeros(T, W, device=device)
        residual_rmsnorm(x, e=e, ecoef=wts, out_dtype=dtype)
        want = torch.zeros(T, W, dtype=torch.float64)
        for t in range(T):
            for k in range(top):
                j = int(table[int(tok[t]), k])
                want[t] += O.expert(h[t].double(), wgu[j, :F].double(), wgu[j, F:].double(), wd[j].double(), limit) / top
        assert float((x.cpu().double() - want).abs().max()) < tol * max(1.0, float(want.abs().max())), (T, W, F)


def head_matrices_case(device, dtype, tol):
    """One value matrix per head on the attended latents, times the sigmoid of a gate slice."""
    from githubrepostorag_amd.ops.moe import head_project

    g = torch.Generator().manual_seed(5)
    for T, H, N, K in ((7, 3, 10, 20), (1, 1, 14, 9), (33, 4, 32, 128), (300, 2, 16, 24), (5, 5, 6, 70)):
        x = torch.randn(T, H * K, generator=g).to(dtype)
        w = (torch.randn(H, N, K, generator=g) * K ** -0.5).to(dtype)
        wide = torch.randn(T, H * N + 16, generator=g).to(dtype)
        got = head_project(x.to(device), w.to(device), gate=wide.to(device)[:, 8:8 + H * N])
        want = torch.einsum("thk,hnk->thn", x.double().view(T, H, K), w.double()).reshape(T, H * N)
        assert float((head_project(x.to(device), w.to(device)).cpu().double() - want).abs().max()) < tol
        want = want * torch.sigmoid(wide[:, 8:8 + H * N].double())
        assert float((got.cpu().double() - want).abs().max()) < tol, (T, H, N, K)


def caps_and_scale_case(device, dtype, tol):
    from githubrepostorag_amd.ops.elementwise import tanh_cap_
    from githubrepostorag_amd.ops.norm import embed_gather_f32

    g = torch.Generator().manual_seed(6)
    z = (40.0 * torch.randn(5, 77, generator=g)).to(dtype)
    wide = torch.cat([z, z], 1).to(device)
    out = tanh_cap_(wide[:, :77], 30.0)
    assert float((out.cpu().double() - 30.0 * torch.tanh(z.double() / 30.0)).abs().max()) < tol * 30
    assert torch.equal(wide[:, 77:].cpu(), z)  # the columns beside the slice are untouched
    assert tanh_cap_(wide[:, 77:], 0.0) is not None and torch.equal(wide[:, 77:].cpu(), z)
    table = torch.randn(20, 24, generator=g).to(dtype)
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32)
    x = embed_gather_f32(ids.to(device), table.to(device), 3.0)
    assert x.dtype == torch.float32 and float((x.cpu().double() - 3.0 * table[ids.long()].double()).abs().max()) < 1e-6


def test_gated_boundary_alone():
    gated_boundary_case("cpu", torch.float32, 1e-5)


def test_input_convolution_alone():
    input_conv_case("cpu", torch.float32, 1e-5)


def test_latent_rows_alone():
    latent_rows_case("cpu", torch.float32, 1e-5)


def test_table_experts_alone():
    table_experts_case("cpu", torch.float32, 1e-5)


def test_head_matrices_alone():
    head_matrices_case("cpu", torch.float32, 1e-5)


def test_caps_and_embedding_scale():
    caps_and_scale_case("cpu", torch.float32, 1e-6)


def test_window_edges_in_prompts_and_decoding():
    C.case_window_edges("cpu", 1e-5)
    C.case_window_edges("cpu", 1e-5, bs=4, latent=True)


# ------------------------------------------------------------------------------------------------ the engine
def test_whole_prompt_and_layer_taps():
    C.case_whole_and_layers("cpu", TOL)


@pytest.mark.parametrize("kinds", [("attention", "attention"), ("latent", "latent"), ("latent", "shared")])
def test_single_mixer_models(kinds):
    C.case_single_mixer("cpu", TOL, kinds)


def test_experts_behind_a_mixer():
    C.case_single_mixer("cpu", TOL, ("attention",), mlp=True, n=30)


def test_prefill_against_decode():
    C.case_prefill_vs_decode("cpu", TOL, n=44)


def test_portions():
    C.case_portions("cpu", TOL)


def test_unequal_batches():
    C.case_batches("cpu", TOL)


def test_pages_and_slots_used_again():
    C.case_reuse("cpu", TOL)


def test_other_sizes():
    C.case_other_sizes("cpu", TOL)


def test_first_tokens():
    C.case_first_tokens("cpu", TOL)


def test_long_decode():
    C.case_long_decode("cpu", TOL)


def test_sharp_softmax_picks_far_keys():
    C.case_sharp_far_keys("cpu", 2e-4)


def test_greedy_generation_through_the_scheduler():
    C.case_generate("cpu")
    C.case_generate("cpu", mixed=True, max_batched=16)


def test_config_round_trip_and_registry(tmp_path):
    from safetensors.torch import save_file

    from githubrepostorag_amd.models import load_decoder
    from githubrepostorag_amd.models.configs import (config_from_dir, decoder_config, pubulix_config_from_dict,
                                                     pubulix_config_to_dict)
    from githubrepostorag_amd.models.pubulix import init_state_dict

    cfg = O.make_config()
    assert pubulix_config_to_dict(pubulix_config_from_dict(cfg)) == cfg
    tiny = decoder_config("pubulix-tiny")
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(pubulix_config_to_dict(tiny)))
    sd = init_state_dict(tiny, seed=1)
    save_file({k: v.contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
    assert config_from_dir(d).layers == tiny.layers
    model = load_decoder(d, device="cpu", dtype=torch.float32)
    assert type(model).__name__ == "PubulixModel" and len(model.runs) == 4
    caches = model.allocate_kv_cache(3, 16)
    assert caches[3][0] is caches[1][0]  # the sharing layer attends to its source's cache tensor
    assert tiny.param_count() == sum(v.numel() for v in sd.values())
    # a tensor of the wrong shape is refused by name; so is a source layer that is none
    bad = dict(sd)
    bad["l1.mix.uk"] = bad["l1.mix.uk"][:-1]
    with pytest.raises(ValueError, match="l1.mix.uk"):
        type(model)(tiny, device="cpu", dtype=torch.float32, state_dict=bad)
    wrong = O.make_config()
    wrong["layers"][3]["mixer"]["kv_from"] = 0
    with pytest.raises(ValueError, match="kv_from"):
        pubulix_config_from_dict(wrong)


def test_trace_replay(tmp_path):
    """The replay command on a saved checkpoint: portions, a request that sits out a step, slots used again."""
    import io

    from safetensors.torch import save_file

    from githubrepostorag_amd.engine.trace import run_trace

    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=31)
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
    a, b = C.tokens(cfg, 30, 1), C.tokens(cfg, 12, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:11], "want": []}, {"id": "a", "tokens": a[17:18], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [11]}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "b", "tokens": b[11:], "want": [0]}], "end": ["b"]}]
    log = io.StringIO()
    out = tmp_path / "o"
    assert run_trace(str(d), "float32", str(out), 128, device="cpu", lines=[json.dumps(s) for s in steps], log=log) == 0
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2", "done", "3"]
    wa, wb = O.forward(cfg, sd, a), O.forward(cfg, sd, b)
    rd = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
    assert C.rel_err(rd(0), wa[[0, 16]]) < TOL and C.rel_err(rd(1), wa[[17]]) < TOL
    assert C.rel_err(rd(2), wa[[29]]) < TOL and C.rel_err(rd(3), wb[[11]]) < TOL
