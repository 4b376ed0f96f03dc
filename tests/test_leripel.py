"""Leripel on the engine, CPU tier: the engine's cache / state / scheduler logic and the ops' host paths against
the float64 oracle (tests/leripel_oracle.py); the same scenarios run on the HIP kernels in test_leripel_gpu.py."""
import json

import numpy as np
import pytest
import torch

import leripel_cases as C
import leripel_oracle as O

TOL = 2e-5


def _meta(dev, lens, ctxs, slots, bs=16, decode=False):
    """AttnMetadata of one step: sequences of ``lens`` new tokens behind ``ctxs`` - ``lens`` cached ones."""
    from githubrepostorag_amd.ops.attention import AttnMetadata

    i32 = dict(dtype=torch.int32, device=dev)
    qs = np.concatenate([[0], np.cumsum(lens)])
    return AttnMetadata(q_start=torch.tensor(qs.tolist(), **i32), ctx_len=torch.tensor(list(ctxs), **i32),
                        block_tables=torch.zeros(len(lens), 1, **i32), slot_mapping=torch.zeros(int(qs[-1]), **i32),
                        max_q_len=max(lens), num_seqs=len(lens), num_tokens=int(qs[-1]), is_decode=decode,
                        state_slots=torch.tensor(list(slots), **i32))


# ------------------------------------------------------------------------------------------------ mechanisms alone
def boundary_case(device, dtype, tol):
    """residual += mixer + gate * shared + sum_k weight_k expert_k, then the RMS norm; the replace form; the copy."""
    from githubrepostorag_amd.ops.norm import residual_rmsnorm

    g = torch.Generator().manual_seed(1)
    for T, H, K in ((5, 48, 2), (3, 200, 1), (2, 4100, 3), (4, 8, 0)):
        x = torch.randn(T, H, generator=g)
        a, b = torch.randn(T, H, generator=g).to(dtype), torch.randn(T, H, generator=g).to(dtype)
        bc, w = torch.rand(T, generator=g), 1.0 + 0.1 * torch.randn(H, generator=g)
        e = torch.randn(T, K, H, generator=g).to(dtype) if K else None
        ec = torch.rand(T, K, generator=g) if K else None
        want = x.double() + a.double() + bc.double()[:, None] * b.double()
        if K:
            want = want + (ec.double()[:, :, None] * e.double()).sum(1)
        xd = x.clone().to(device)
        raw = torch.zeros(T, 2 * H, dtype=dtype, device=device)
        dv = lambda t: None if t is None else t.to(device)
        h = residual_rmsnorm(xd, dv(a), dv(b), dv(bc), dv(e), dv(ec), dv(w), 1e-5, dtype, raw=raw[:, H:])
        assert float((xd.cpu().double() - want).abs().max()) < 1e-5
        hn = want / torch.sqrt((want * want).mean(-1, keepdim=True) + 1e-5) * w.double()
        assert float((h.cpu().double() - hn).abs().max()) < tol
        assert float((raw[:, H:].cpu().double() - want).abs().max()) < tol * 4 and float(raw[:, :H].abs().max()) == 0
        # replace: x <- a alone
        h2 = residual_rmsnorm(xd, dv(a), w=dv(w), eps=1e-5, out_dtype=dtype, keep=False)
        assert float((xd.cpu().double() - a.double()).abs().max()) == 0
        an = a.double() / torch.sqrt((a.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w.double()
        assert float((h2.cpu().double() - an).abs().max()) < tol


def router_case(device, dtype):
    """Group-limited choice: every token's experts, weights and shared gate against the oracle's rule, on logits
    with clear gaps; also a best expert that sits in a closed group and must not be chosen."""
    from githubrepostorag_amd.ops.moe import moe_route

    g = torch.Generator().manual_seed(2)
    # (37 tokens: the kernel of decode rows and short portions; 150: the tiled kernel of prompts)
    for E, top, groups, keep, W, T in ((6, 2, 3, 2, 40, 37), (20, 4, 5, 3, 64, 150), (8, 8, 1, 1, 24, 37), (9, 1, 9, 1, 16, 37),
                                       (12, 3, 4, 4, 33, 37), (12, 3, 4, 4, 33, 131), (24, 5, 6, 2, 264, 9)):
        h = torch.randn(T, W, generator=g).to(dtype)
        wr = (torch.randn(E + 1, W, generator=g) * 0.7).to(torch.bfloat16).float()
        ids, wts, gate = moe_route(h.to(device), wr.to(device), E, top, groups, keep)
        z = h.double() @ wr.double().T
        s = torch.softmax(z[:, :E], -1)
        per = E // groups
        for t in range(T):
            best = sorted(range(groups), key=lambda q: -float(s[t, q * per:(q + 1) * per].max()))[:keep]
            allowed = [e for e in range(E) if e // per in best]
            chosen = sorted(allowed, key=lambda e: -float(s[t, e]))[:top]
            assert ids[t].tolist()[:len(chosen)] == chosen, (E, t)
            assert float((wts[t, :len(chosen)].cpu().double() - s[t, chosen]).abs().max()) < 1e-5
        assert float((gate.cpu().double() - torch.sigmoid(z[:, E])).abs().max()) < 1e-5
    # two groups of two, one open: expert 3 has the second-best score overall but its group is closed
    wr = torch.zeros(4, 4)
    wr[0, 0], wr[1, 1], wr[2, 2], wr[3, 3] = 5.0, 1.0, 0.0, 4.0
    h = torch.ones(1, 4, dtype=dtype)
    ids, wts, gate = moe_route(h.to(device), wr.to(device), 4, 2, 2, 1)
    assert ids[0].tolist() == [0, 1] and gate is None


def experts_case(device, dtype, tol):
    from githubrepostorag_amd.ops.moe import moe_experts

    g = torch.Generator().manual_seed(3)
    for T, W, F, E, top in ((9, 48, 20, 6, 2), (70, 64, 40, 5, 3), (3, 40, 24, 4, 4), (1, 33, 7, 3, 1), (200, 136, 40, 3, 2)):
        h = torch.randn(T, W, generator=g).to(dtype)
        wgu = (torch.randn(E, 2 * F, W, generator=g) / W ** 0.5).to(dtype)
        wd = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(dtype)
        ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
        if T > 20:
            ids[:, 0] = 1  # one expert with more rows than a tile, another with none
            ids[ids == 4] = 0
        got = moe_experts(h.to(device), ids.to(device), wgu.to(device), wd.to(device)).cpu().double()
        for t in range(T):
            for k in range(top):
                e = int(ids[t, k])
                gu = wgu[e].double() @ h[t].double()
                want = wd[e].double() @ (O.silu(gu[:F]) * gu[F:])
                assert float((got[t, k] - want).abs().max()) < tol * max(1.0, float(want.abs().max())), (T, t, k)


def conv_scan_case(device, dtype, tol):
    """The convolution and the scan on two sequences at once, cut into steps at different places (inside the
    convolution's reach, across scan chunks), with stale contents in the slots: against one pass of the oracle's
    loop over each whole sequence."""
    from githubrepostorag_amd.ops.recurrent import causal_conv, gated_rmsnorm, ssm_scan

    g = torch.Generator().manual_seed(4)
    for H, P, N, G, taps, ng in ((4, 6, 10, 2, 4, 2), (2, 70, 33, 1, 2, 1), (3, 8, 130, 3, 1, 3)):
        inner, ch = H * P, H * P + 2 * G * N
        ld = 2 * inner + 2 * G * N + H
        m = {"heads": H, "vdim": P, "state": N, "groups": G, "norm_groups": ng, "conv": taps}
        Wt = {"in": torch.eye(ld), "conv": (torch.randn(ch, taps, generator=g) * 0.5).to(torch.bfloat16).float(),
              "conv.b": (torch.randn(ch, generator=g) * 0.2).to(torch.bfloat16).float(),
              "dt_bias": torch.randn(H, generator=g), "A_log": torch.rand(H, generator=g) * 2 - 1.5,
              "D": 1 + 0.3 * torch.randn(H, generator=g), "norm": 1 + 0.1 * torch.randn(inner, generator=g),
              "o": torch.eye(inner)}
        lens = (150, 71)
        seqs = [(torch.randn(n, ld, generator=g) * 0.8).to(dtype) for n in lens]
        want = [O.ssm(s.double(), lambda n: Wt[n].double(), m, 1e-5) for s in seqs]
        cstate = torch.randn(3, max(taps - 1, 0), ch, generator=g).to(dtype).to(device)   # stale
        sstate = torch.randn(3, H, N, P, generator=g).to(device)
        dv = lambda n: Wt[n].to(device)
        got = [[], []]
        cur = [0, 0]
        for step in ((2, 1), (1, 69), (80, 1), (66, 0), (1, 0)):
            parts, ls, cs, sl, who = [], [], [], [], []
            for i, n in enumerate(step):
                if n:
                    parts.append(seqs[i][cur[i]:cur[i] + n])
                    cur[i] += n
                    ls.append(n); cs.append(cur[i]); sl.append(2 - i); who.append(i)
            proj = torch.cat(parts, 0).to(device)
            meta = _meta(device, ls, cs, sl)
            xbc = causal_conv(proj, inner, dv("conv"), dv("conv.b"), cstate, meta)
            y = ssm_scan(xbc, proj, inner + ch, dv("dt_bias"), dv("A_log"), dv("D"), sstate, meta, H, G, N, P)
            out = torch.empty(proj.shape[0], inner, dtype=dtype, device=device)
            gated_rmsnorm(y, dv("norm"), proj, 0, 1e-5, out, groups=ng, gate="silu", gate_first=True)
            o = 0
            for i, n in zip(who, ls):
                got[i].append(out[o:o + n].cpu().double())
                o += n
        for i in range(2):
            assert cur[i] == lens[i]
            assert float((torch.cat(got[i], 0) - want[i]).abs().max()) < tol, (H, i)


def test_boundary_alone():
    boundary_case("cpu", torch.float32, 1e-5)


def test_router_alone():
    router_case("cpu", torch.float32)


def test_experts_alone():
    experts_case("cpu", torch.float32, 1e-5)


def test_conv_and_scan_alone():
    conv_scan_case("cpu", torch.float32, 1e-4)


def test_block_edges_in_prompts_and_decoding():
    C.case_block_edges("cpu", 1e-5)


# ------------------------------------------------------------------------------------------------ the engine
def test_whole_prompt_and_layer_taps():
    C.case_whole_and_layers("cpu", TOL)


@pytest.mark.parametrize("kind", ["retention", "attention", "mamba2"])
def test_single_mixer_models(kind):
    C.case_single_mixer("cpu", TOL, kind)


def test_experts_beside_a_mixer():
    C.case_single_mixer("cpu", TOL, "retention", mlp=True)


def test_prefill_against_decode():
    C.case_prefill_vs_decode("cpu", TOL, n=40)


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
    from githubrepostorag_amd.models.configs import (config_from_dir, decoder_config, leripel_config_from_dict,
                                                     leripel_config_to_dict)
    from githubrepostorag_amd.models.leripel import init_state_dict

    cfg = O.make_config()
    assert leripel_config_to_dict(leripel_config_from_dict(cfg)) == cfg
    tiny = decoder_config("leripel-tiny")
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(leripel_config_to_dict(tiny)))
    sd = init_state_dict(tiny, seed=1)
    save_file({k: v.contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
    assert config_from_dir(d).layers == tiny.layers
    model = load_decoder(d, device="cpu", dtype=torch.float32)
    assert type(model).__name__ == "LeripelModel" and len(model.runs) == 6
    n = sum(v.numel() for v in sd.values())
    assert tiny.param_count() == n
    # a tensor of the wrong shape is refused by name
    sd["l0.mix.q"] = sd["l0.mix.q"][:-1]
    with pytest.raises(ValueError, match="l0.mix.q"):
        type(model)(tiny, device="cpu", dtype=torch.float32, state_dict=sd)


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
