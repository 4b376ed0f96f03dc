"""Leripel on the HIP kernels (cuda:0): every mechanism alone and the engine scenarios of leripel_cases.py against
the float64 oracle -- in fp32 (the kernels' 32-bit parts are then the whole computation: tight bounds) and in bf16
(the serving precision)."""
import numpy as np
import pytest
import torch

import leripel_cases as C
import leripel_oracle as O
import test_leripel as T

pytestmark = pytest.mark.gpu

F32 = 5e-5   # fp32 GEMMs + fp32 kernels against float64
BF16 = 0.06  # bf16 GEMMs and activations


@pytest.fixture(autouse=True)
def _true_fp32():
    torch.backends.cuda.matmul.allow_tf32 = False
    yield


def test_kernel_library_is_loaded():
    from githubrepostorag_amd.ops import _lib

    assert _lib.lib() is not None and _lib.loaded_path()
    for name in ("grag_causal_conv", "grag_ssm_scan", "grag_moe_route", "grag_moe_align", "grag_moe_gemm",
                 "grag_residual_rmsnorm", "grag_sink_attn_prefill", "grag_sink_attn_decode"):
        assert hasattr(_lib.lib(), name)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.03)])
def test_boundary_alone(dtype, tol):
    T.boundary_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_alone(dtype):
    T.router_case("cuda", dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.02)])
def test_experts_alone(dtype, tol):
    # fp32: the plain tiles; bf16: the matrix-core tiles where the sizes are multiples of 8, small and (the last case,
    # 400 rows over 3 experts) large ones
    T.experts_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 0.08)])
def test_conv_and_scan_alone(dtype, tol):
    T.conv_scan_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 5e-3)])
def test_block_edges_in_prompts_and_decoding(dtype, tol):
    C.case_block_edges("cuda", tol, dtype)  # (bf16: the stored output is rounded to 8 bits, 0.4 % of a marker up to 75; a wrong key is off by >= 1)
    C.case_block_edges("cuda", tol, dtype, bs=4)


@pytest.mark.parametrize("kind", ["retention", "attention", "mamba2"])
def test_single_mixer_models(kind):
    C.case_single_mixer("cuda", F32, kind)
    C.case_single_mixer("cuda", BF16, kind, torch.bfloat16)
    with C.near_ties(0.06):
        C.case_single_mixer("cuda", BF16, kind, torch.bfloat16, mlp=True)
    C.case_single_mixer("cuda", F32, kind, mlp=True)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_whole_prompt_and_layer_taps(dtype, tol):
    with C.near_ties(0.06 if dtype == torch.bfloat16 else 0.0):
        C.case_whole_and_layers("cuda", tol, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_prefill_against_decode(dtype, tol):
    with C.near_ties(0.06 if dtype == torch.bfloat16 else 0.0):
        C.case_prefill_vs_decode("cuda", tol, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_portions(dtype, tol):
    with C.near_ties(0.06 if dtype == torch.bfloat16 else 0.0):
        C.case_portions("cuda", tol, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_unequal_batches(dtype, tol):
    if dtype == torch.bfloat16:
        with C.near_ties(0.06):
            C.case_batches("cuda", 0.02, dtype, alone=True)
    else:
        C.case_batches("cuda", tol, dtype)


def test_pages_and_slots_used_again():
    C.case_reuse("cuda", F32)


def test_other_sizes():
    C.case_other_sizes("cuda", F32)
    with C.near_ties(0.1):
        C.case_other_sizes("cuda", 0.15, torch.bfloat16)  # (three passes and tiny widths amplify the rounding)


def test_first_tokens():
    C.case_first_tokens("cuda", F32)


def test_long_decode():
    C.case_long_decode("cuda", F32)


def test_sharp_softmax_picks_far_keys():
    C.case_sharp_far_keys("cuda", 5e-4)


def test_matrix_core_shapes_bf16():
    """Head sizes in multiples of 16, expert sizes in multiples of 8 and prompt portions of >= 16 queries: the bf16
    attention and expert kernels that run on the matrix cores, whole and in portions with decoded tokens at the end;
    blocks of 70 positions against 64-key tiles."""
    cfg = O.make_config(width=64, kinds=("attention", "mamba2", "retention"), loop=(0, 2, 2), no_mlp=(2,), heads=4,
                        kv_heads=2, dim=32, vdim=48, scale=0.2, chunk=70, rot_dims=16, ret_heads=2, ret_dim=16,
                        ret_vdim=32, decay=[0.95, 0.999], ssm_heads=4, ssm_vdim=16, ssm_state=32, ssm_groups=2,
                        ssm_norm_groups=2, experts=8, top=3, groups=(4, 3), ff=40, shared_ff=48)
    sd = O.make_weights(cfg, seed=51)
    toks = C.tokens(cfg, 200, 8)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "w", toks, [200]), want) < BF16
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [64, 70, 50] + [1] * 16), want) < BF16


def test_serving_head_sizes():
    """The head sizes of the bench presets (128-wide attention heads, state-space heads of 64 channels with a state of
    128) at a small width, blocks of 80, prompts and decoded tokens, both precisions."""
    cfg = O.make_config(width=128, vocab=128, kinds=("retention", "attention", "mamba2"), loop=(0, 0, 1), heads=4,
                        kv_heads=2, dim=128, vdim=128, scale=0.09, chunk=80, rot_dims=64, ret_heads=2, ret_dim=128,
                        ret_vdim=128, decay=[0.98, 0.999], ssm_heads=2, ssm_vdim=64, ssm_state=128, ssm_groups=1,
                        ssm_norm_groups=1, experts=4, top=2, groups=(2, 1), ff=64, shared_ff=64)
    sd = O.make_weights(cfg, seed=57)
    toks = C.tokens(cfg, 150, 11)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [70, 64] + [1] * 16), want) < BF16
    _, eng = C.build(cfg, sd, "cuda", torch.float32)
    assert C.rel_err(C.feed_in_portions(eng, "d", toks, [70, 64] + [1] * 16), want) < F32


def test_key_splits_with_blocks():
    """Blocks longer than the decode kernel's single-pass limit take the engine's key splits: splits that lie wholly
    before the query's block are empty, the split that holds the block's first key starts inside it."""
    cfg = O.make_config(width=64, kinds=("attention",), loop=(0, 0, 1), no_mlp=(0,), heads=4, kv_heads=2, dim=16,
                        vdim=16, scale=0.4, chunk=1100, rot_dims=8)
    sd = O.make_weights(cfg, seed=59)
    toks = C.tokens(cfg, 1300, 12)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16, pool_tokens=1408)
    assert C.rel_err(C.feed_in_portions(eng, "k", toks, [1090] + [1] * 20 + [170] + [1] * 20), want) < BF16


@pytest.mark.parametrize("graphs,mixed,window,max_batched", [(False, False, 1, 4096), (True, False, 1, 4096),
                                                             (True, False, 4, 4096), (False, True, 1, 8)])
def test_greedy_generation(graphs, mixed, window, max_batched):
    C.case_generate("cuda", graphs=graphs, mixed=mixed, window=window, max_batched=max_batched)


def test_bf16_batch_invariance():
    """bf16 serving: a request's logits beside other requests equal its logits alone (the same kernels see the
    same operands per row; only GEMM tiling may differ with the batch's row count)."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=37)
    a, b = C.tokens(cfg, 40, 1), C.tokens(cfg, 13, 2)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    alone = C.feed_in_portions(eng, "a", a, [40])
    o1 = eng.feed([("a2", a[:25], list(range(25))), ("b", b[:12], [])], [])
    o2 = eng.feed([("a2", a[25:], list(range(15))), ("b", b[12:], [0])], ["a2", "b"])
    assert C.rel_err(np.concatenate([o1, o2[:15]], 0), alone) < 0.02
