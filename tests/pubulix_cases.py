"""Scenarios that compare the engine serving a Pubulix model (kernels, paged cache, state slots, scheduler) with
the plain float64 oracle of pubulix_oracle.py.  Every scenario takes the device: the CPU tier runs the ops' host
paths, the GPU tier the HIP kernels, through the same engine code."""
from __future__ import annotations

import numpy as np
import torch

import pubulix_oracle as O


def build(cfg_dict, sd, device, dtype=torch.float32, slots=4, pool_tokens=512, block_size=16, graphs=False,
          max_batched=4096, mixed=False, window=1):
    from githubrepostorag_amd.engine.llm_engine import EngineConfig, LLMEngine
    from githubrepostorag_amd.models import build_decoder
    from githubrepostorag_amd.models.configs import pubulix_config_from_dict

    model = build_decoder(pubulix_config_from_dict(cfg_dict), device=device, dtype=dtype, state_dict=sd)
    eng = LLMEngine(model, None, EngineConfig(max_num_seqs=slots, max_model_len=max(pool_tokens, 64),
                                              block_size=block_size, num_blocks=pool_tokens // block_size + 1,
                                              use_cuda_graph=graphs, max_num_batched_tokens=max_batched,
                                              mixed_batches=mixed, decode_window=window))
    return model, eng


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(7000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def rel_err(got, want):
    """Mean-free RMS difference over the vocabulary, relative to the logits' own spread (the worst row)."""
    got = torch.as_tensor(np.asarray(got), dtype=torch.float64)
    want = torch.as_tensor(np.asarray(want), dtype=torch.float64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.std(-1)).max())


def feed_in_portions(eng, rid, toks, cuts, end=True):
    """Feed ``toks`` as portions of the sizes in ``cuts`` (cycled), asking for every place; -> logits [T, vocab]."""
    out, a, i = [], 0, 0
    while a < len(toks):
        n = min(cuts[i % len(cuts)], len(toks) - a)
        last = a + n == len(toks)
        out.append(eng.feed([(rid, toks[a:a + n], list(range(n)))], [rid] if last and end else []))
        a += n
        i += 1
    return np.concatenate(out, 0)


def case_whole_and_layers(device, tol, dtype=torch.float32, **cfg_kw):
    cfg = O.make_config(**cfg_kw)
    sd = O.make_weights(cfg, seed=3)
    toks = tokens(cfg, 37, 0)
    want, taps = O.logits_and_taps(cfg, sd, toks)
    model, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "a", toks, [len(toks)]), want) < tol
    # the residual after every layer, through the model's own step (one sequence, fresh cache / state)
    from githubrepostorag_amd.ops.attention import AttnMetadata

    T, bs = len(toks), 16
    nb = -(-T // bs)
    i32 = dict(dtype=torch.int32, device=model.device)
    meta = AttnMetadata(q_start=torch.tensor([0, T], **i32), ctx_len=torch.tensor([T], **i32),
                        block_tables=(torch.arange(nb, **i32) + 1).view(1, nb), slot_mapping=torch.arange(T, **i32) + bs,
                        max_q_len=T, num_seqs=1, num_tokens=T, state_slots=torch.tensor([1], **i32))
    mine = []
    model.forward(torch.tensor(toks, **i32), torch.arange(T, **i32), meta, model.allocate_kv_cache(nb + 1, bs),
                  state=model.allocate_state(2), taps=mine)
    assert len(mine) == taps.shape[0]
    for r, (a, b) in enumerate(zip(mine, taps)):
        err = float((a.double().cpu() - b).abs().max() / b.abs().max())
        assert err < tol, (r, err)


def case_single_mixer(device, tol, kinds, dtype=torch.float32, mlp=False, n=45, **kw):
    """A stack of one mixer kind (a shared-cache layer behind its source), with or without experts: the mechanism
    alone between embedding and head; whole, token by token, and in portions.  Windows shorter than the prompt."""
    cfg = O.make_config(kinds=kinds, no_mlp=() if mlp else tuple(range(len(kinds))), **kw)
    sd = O.make_weights(cfg, seed=21)
    toks = tokens(cfg, n, 5)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "w", toks, [n]), want) < tol
    assert rel_err(feed_in_portions(eng, "d", toks, [1]), want) < tol
    assert rel_err(feed_in_portions(eng, "c", toks, [6, 2, 19]), want) < tol


def case_prefill_vs_decode(device, tol, dtype=torch.float32, n=58, **cfg_kw):
    cfg = O.make_config(**cfg_kw)
    sd = O.make_weights(cfg, seed=5)
    toks = tokens(cfg, n, 1)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "p", toks, [n]), want) < tol
    assert rel_err(feed_in_portions(eng, "d", toks, [1]), want) < tol           # every token on the decode path
    assert rel_err(feed_in_portions(eng, "pd", toks, [n - 25] + [1] * 25), want) < tol  # windows pass over decoded tokens


def case_portions(device, tol, dtype=torch.float32):
    """Portions cut inside pages (16), windows (11 and 19) and the convolution's reach (3), down to two tokens."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=7)
    toks = tokens(cfg, 101, 2)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    for k, cuts in enumerate(([2], [3, 2, 17, 1, 16, 31], [16], [15, 1, 1, 33], [11, 19], [64, 2], [90, 9], [1, 2])):
        assert rel_err(feed_in_portions(eng, f"c{k}", toks, cuts), want) < tol, cuts


def case_batches(device, tol, dtype=torch.float32, alone=False):
    """Unequal requests in one batch -- portions beside single tokens, requests that sit out steps and end at
    different times -- give each request the logits it gets alone: the oracle's, or (``alone``) the same engine's
    when it serves the request whole and by itself."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=9)
    lens = {"a": 45, "b": 9, "c": 31, "d": 18}
    toks = {k: tokens(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    _, eng = build(cfg, sd, device, dtype, pool_tokens=192)
    if alone:
        want = {k: torch.as_tensor(feed_in_portions(eng, k + "0", t, [len(t)]), dtype=torch.float64) for k, t in toks.items()}
    else:
        want = {k: O.forward(cfg, sd, t) for k, t in toks.items()}
    plan = [  # (request, tokens) per step
        [("a", 20), ("b", 2)],
        [("a", 1), ("b", 1), ("c", 17)],
        [("a", 1), ("c", 1), ("d", 16)],
        [("b", 6), ("a", 3), ("d", 1), ("c", 13)],
        [("a", 20), ("d", 1)],
    ]
    cur = {k: 0 for k in toks}
    got = {k: [] for k in toks}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, toks[k][cur[k]:cur[k] + n], list(range(n))))
            cur[k] += n
            if cur[k] == lens[k]:
                end.append(k)
        out = eng.feed(entries, end)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
    for k in toks:
        assert cur[k] == lens[k]
        assert rel_err(np.concatenate(got[k], 0), want[k]) < tol, k
    assert eng.kv.num_free == eng.kv.num_blocks - 1 and len(eng.sched.free_slots) == 4


def case_reuse(device, tol, dtype=torch.float32):
    """Pages and state slots that were freed are used again: with one slot and a pool of one request's worth, later
    requests land on the earlier ones' pages and convolution inputs and still match their oracle."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=11)
    _, eng = build(cfg, sd, device, dtype, slots=1, pool_tokens=64)
    for i, n in enumerate((50, 7, 33, 64, 1)):
        toks = tokens(cfg, n, 20 + i)
        want = O.forward(cfg, sd, toks)
        cuts = [[n], [3, 1], [32, 1], [60, 2, 1, 1], [1]][i]
        assert rel_err(feed_in_portions(eng, f"r{i}", toks, cuts), want) < tol, i
        assert eng.kv.num_free == eng.kv.num_blocks - 1
    # a request that stops mid-way leaves nothing behind either
    eng.feed([("x", tokens(cfg, 40, 30), [])], [])
    eng.feed([], ["x"])
    toks = tokens(cfg, 21, 31)
    assert rel_err(feed_in_portions(eng, "y", toks, [20, 1]), O.forward(cfg, sd, toks)) < tol


def case_long_decode(device, tol, dtype=torch.float32):
    cfg = O.make_config(window=33, lat_window=70)
    sd = O.make_weights(cfg, seed=13)
    toks = tokens(cfg, 150, 3)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "l", toks, [6] + [1] * 144), want) < tol


def case_other_sizes(device, tol, dtype=torch.float32):
    """Sizes where things the usual configs make equal differ, or are 1."""
    variants = [
        # one kv head, whole-head rotary, value size above the key size, a window of one position (only itself);
        # one latent head, every expert chosen, a residual multiplier of 1, no embedding scale
        dict(width=40, vocab=33, kinds=("latent", "attention", "shared"), heads=3, kv_heads=1, dim=10, vdim=24,
             rot_dims=10, rot_base=7.0, scale=1.0, window=1, lat_heads=1, lat_dim=6, lat_vdim=14, kv_rank=9, rot_dim=2,
             lat_window=4, experts=3, top=3, residual_mult=1.0, embed_scale=1.0),
        # heads == kv heads, no rotary, windows longer than the prompt, no score cap and no logit cap; a convolution
        # of one tap; top 1; a latent value size above the latent size
        dict(width=48, vocab=50, kinds=("attention", "latent"), heads=2, kv_heads=2, dim=72, vdim=72, rot_dims=0,
             scale=0.1, window=500, softcap=0.0, logit_softcap=0.0, lat_heads=2, lat_dim=20, lat_vdim=40, kv_rank=12,
             rot_dim=4, lat_window=500, taps=1, experts=4, top=1, ff=8),
        # no convolution at all; two layers sharing one cache with different windows come out of make_config's default
        # window for both, so the second gets its own below; five taps in the next variant
        dict(width=56, vocab=64, kinds=("latent", "shared", "shared"), no_mlp=(1,), lat_heads=5, lat_dim=4, lat_vdim=6,
             kv_rank=70, rot_dim=10, lat_window=7, taps=0, experts=8, top=5),
        dict(taps=5, window=2, lat_window=2, kinds=("attention", "latent", "shared", "attention")),
        # a wide latent (more than 64 value columns per lane chunk) and a long head
        dict(width=64, kinds=("latent", "shared"), lat_heads=2, lat_dim=16, lat_vdim=8, kv_rank=136, rot_dim=8,
             lat_window=23, no_mlp=(0, 1)),
        # a width and a vocabulary that are multiples of nothing useful (rows of 60 and 72 bytes), odd head sizes
        dict(width=30, vocab=77, kinds=("attention", "latent", "shared"), heads=2, kv_heads=1, dim=10, vdim=6,
             rot_dims=6, lat_heads=2, lat_dim=5, lat_vdim=7, kv_rank=11, rot_dim=2, ff=9, experts=2, top=2, taps=4),
        dict(width=36, vocab=101, kinds=("latent", "attention"), heads=6, kv_heads=3, dim=6, vdim=10, rot_dims=2,
             lat_heads=4, lat_dim=6, lat_vdim=6, kv_rank=18, rot_dim=6, ff=20, experts=7, top=4, taps=2),
    ]
    for i, kw in enumerate(variants):
        cfg = O.make_config(**kw)
        if i == 2:  # the sharing layers look further back, and less far, than the layer that owns the cache
            cfg["layers"][1]["mixer"]["mask"]["size"] = 12
            cfg["layers"][2]["mixer"]["mask"]["size"] = 3
        sd = O.make_weights(cfg, seed=40 + i)
        toks = tokens(cfg, 29, 40 + i)
        want = O.forward(cfg, sd, toks)
        _, eng = build(cfg, sd, device, dtype)
        assert rel_err(feed_in_portions(eng, "w", toks, [29]), want) < tol, i
        assert rel_err(feed_in_portions(eng, "c", toks, [5, 1, 2]), want) < tol, i


def case_first_tokens(device, tol, dtype=torch.float32):
    """Position 0 alone (one key, a sink, a convolution that starts from zeros in a used slot), then 1, 2."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=17)
    _, eng = build(cfg, sd, device, dtype, slots=1)
    eng.feed([("warm", tokens(cfg, 30, 50), [])], ["warm"])  # leave convolution inputs and pages behind
    for n in (1, 2, 3, 5):
        toks = tokens(cfg, n, 60 + n)
        want = O.forward(cfg, sd, toks)
        assert rel_err(feed_in_portions(eng, f"f{n}", toks, [1]), want) < tol
        assert rel_err(feed_in_portions(eng, f"g{n}", toks, [n]), want) < tol


def case_sharp_far_keys(device, tol, dtype=torch.float32):
    """Softmax scales large enough (and a cap high enough) that every query picks out single keys of its window, many
    of them far back and across page borders: a key read from the wrong place changes the logits outright.  300
    tokens under windows of 150 and 210, the last 40 decoded one by one, portions cut off the page grid."""
    cfg = O.make_config(kinds=("attention", "latent", "shared"), no_mlp=(0, 1, 2), scale=6.0, softcap=200.0,
                        lat_scale=5.0, window=150, lat_window=210, kv_heads=1)
    sd = O.make_weights(cfg, seed=29)
    toks = tokens(cfg, 300, 6)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "s", toks, [300]), want) < tol
    assert rel_err(feed_in_portions(eng, "t", toks, [97, 130, 33] + [1] * 40), want) < tol


def case_window_edges(device, tol, dtype=torch.float32, bs=16, latent=False):
    """The attention op alone on crafted keys: key j is 30 e_j, so a query e_p scores 30 on position p and 0
    elsewhere, and the softmax weight of an asked-for visible key is ~1.  Head 0 asks for the oldest key of the
    query's window (just inside), head 1 for the key one before it (just outside: its weight must be spread over the
    visible keys instead, none of which carries the marker value), head 2 for the query's own position.  In a
    prompt's portion that follows cached context and for a decoded token; windows that end on, before and after
    page borders, pages out of order.  ``latent``: the values are the first columns of the key rows (one cache
    tensor); heads 0 and 2 carry a sink far below their scores, which must change nothing, head 1 a sink of 0 beside
    its n visible keys of score 0, which must take exactly 1 / (n + 1) of the weight."""
    from githubrepostorag_amd.ops.attention import AttnMetadata, sink_attention

    dev = torch.device(device)
    H, G, ctx = 3, 1, 75
    d, vd = 96, 16
    for window in (1, 2, 5, bs, bs + 1, 2 * bs - 1, 40, 64, 65, 75, 200):
        nb = -(-ctx // bs)
        g = torch.Generator().manual_seed(window)
        perm = (torch.randperm(nb, generator=g) + 1).to(torch.int32)
        kc = torch.zeros(nb + 1, G, bs, d, dtype=dtype, device=dev)
        vc = kc[..., :vd] if latent else torch.zeros(nb + 1, G, bs, vd, dtype=dtype, device=dev)
        for j in range(ctx):  # (latent: the value columns are key columns 0 .. vd - 1, so the markers sit at vd + j)
            kc[perm[j // bs], 0, j % bs, vd + j] = 30.0
            vc[perm[j // bs], 0, j % bs, 0] = j + 1.0  # the value names its position
        sinks = torch.tensor([-20.0, 0.0, -20.0], device=dev) if latent else None
        for qlen in (33, 9, 1):  # (33 queries in bf16: the matrix-core kernel)
            q = torch.zeros(qlen, H, d)
            for n, p in enumerate(range(ctx - qlen, ctx)):
                lo = max(0, p - window + 1)
                q[n, 0, vd + lo] = 1.0
                if lo > 0:
                    q[n, 1, vd + lo - 1] = 1.0
                q[n, 2, vd + p] = 1.0
            i32 = dict(dtype=torch.int32, device=dev)
            meta = AttnMetadata(q_start=torch.tensor([0, qlen], **i32), ctx_len=torch.tensor([ctx], **i32),
                                block_tables=perm.view(1, nb).to(dev), slot_mapping=torch.zeros(qlen, **i32),
                                max_q_len=qlen, num_seqs=1, num_tokens=qlen, is_decode=qlen == 1)
            got = sink_attention(q.to(dtype).to(dev), kc, vc, meta, 1.0, sinks, window=window,
                                 softcap=1000.0).float().cpu().view(qlen, H, vd)
            for n, p in enumerate(range(ctx - qlen, ctx)):
                lo = max(0, p - window + 1)
                assert abs(float(got[n, 0, 0]) - (lo + 1.0)) < tol * ctx, (window, qlen, p, "inside")
                assert abs(float(got[n, 2, 0]) - (p + 1.0)) < tol * ctx, (window, qlen, p, "self")
                if lo > 0:  # the key just outside gets nothing: head 1 sees a flat average of its window's values
                    want = float(torch.arange(lo, p + 1).double().mean()) + 1.0
                    if latent:
                        want *= (p + 1 - lo) / (p + 2 - lo)
                    assert abs(float(got[n, 1, 0]) - want) < tol * ctx, (window, qlen, p, "outside")
            if latent:
                continue
            # a cap of 2 on the scores: the asked-for key scores 2 tanh(15) = 2, the other visible keys 0
            got = sink_attention(q.to(dtype).to(dev), kc, vc, meta, 1.0, None, window=window,
                                 softcap=2.0).float().cpu().view(qlen, H, vd)
            e2 = float(np.exp(2.0))
            for n, p in enumerate(range(ctx - qlen, ctx)):
                lo = max(0, p - window + 1)
                others = float(torch.arange(lo, p).double().sum()) + (p - lo)  # sum of (j + 1) over the keys before p
                want = (e2 * (p + 1.0) + others) / (e2 + p - lo)
                assert abs(float(got[n, 2, 0]) - want) < tol * ctx, (window, qlen, p, "capped")


def case_generate(device, dtype=torch.float32, graphs=False, mixed=False, window=1, max_batched=4096, tol=2e-3,
                  **cfg_kw):
    """Greedy generation through LLMEngine.generate (scheduler, chunked prefill, sampler, decode steps): every
    generated token is the oracle's arg-max given the tokens before it (up to a near-tie)."""
    from githubrepostorag_amd.engine.sequence import SamplingParams

    cfg = O.make_config(**cfg_kw)
    sd = O.make_weights(cfg, seed=19)
    _, eng = build(cfg, sd, device, dtype, slots=3, pool_tokens=256, graphs=graphs, mixed=mixed, window=window,
                   max_batched=max_batched)
    prompts = [tokens(cfg, n, 70 + i) for i, n in enumerate((5, 23, 11, 2))]  # 4 prompts on 3 slots: one waits
    outs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True))
    for p, c in zip(prompts, outs):
        assert len(c.token_ids) == 14
        logits = O.forward(cfg, sd, p + c.token_ids[:-1])
        for j, t in enumerate(c.token_ids):
            row = logits[len(p) - 1 + j]
            assert float(row.max() - row[t]) < tol * float(row.std()), (len(p), j)
    assert eng.kv.num_free == eng.kv.num_blocks - 1
