"""Pubulix on the HIP kernels (cuda:0): every mechanism alone and the engine scenarios of pubulix_cases.py against
the float64 oracle -- in fp32 (the kernels' 32-bit parts are then the whole computation: tight bounds) and in bf16
(the serving precision)."""
import numpy as np
import pytest
import torch

import pubulix_cases as C
import pubulix_oracle as O
import test_pubulix as T

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
    for name in ("grag_causal_conv", "grag_latent_rope_store", "grag_moe_table_route", "grag_moe_align", "grag_moe_gemm",
                 "grag_residual_rmsnorm", "grag_sink_attn_prefill", "grag_sink_attn_decode", "grag_tanh_cap"):
        assert hasattr(_lib.lib(), name)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.03)])
def test_gated_boundary_alone(dtype, tol):
    T.gated_boundary_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.05)])
def test_input_convolution_alone(dtype, tol):
    T.input_conv_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.03)])
def test_latent_rows_alone(dtype, tol):
    T.latent_rows_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.03)])
def test_table_experts_alone(dtype, tol):
    # fp32: the plain tiles; bf16: the matrix-core tiles, small and (the last case, 800 rows over 3 experts) large ones
    T.table_experts_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.03)])
def test_head_matrices_alone(dtype, tol):
    T.head_matrices_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 5e-3)])
def test_caps_and_embedding_scale(dtype, tol):
    T.caps_and_scale_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 5e-3)])
def test_window_edges_in_prompts_and_decoding(dtype, tol):
    # (bf16: the stored output is rounded to 8 bits, 0.4 % of a marker up to 75; a wrong key is off by >= 1)
    C.case_window_edges("cuda", tol, dtype)
    C.case_window_edges("cuda", tol, dtype, bs=4, latent=True)


@pytest.mark.parametrize("kinds", [("attention", "attention"), ("latent", "latent"), ("latent", "shared")])
def test_single_mixer_models(kinds):
    C.case_single_mixer("cuda", F32, kinds)
    C.case_single_mixer("cuda", BF16, kinds, torch.bfloat16)
    C.case_single_mixer("cuda", F32, kinds, mlp=True)
    C.case_single_mixer("cuda", BF16, kinds, torch.bfloat16, mlp=True)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_whole_prompt_and_layer_taps(dtype, tol):
    C.case_whole_and_layers("cuda", tol, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_prefill_against_decode(dtype, tol):
    C.case_prefill_vs_decode("cuda", tol, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_portions(dtype, tol):
    C.case_portions("cuda", tol, dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32), (torch.bfloat16, BF16)])
def test_unequal_batches(dtype, tol):
    C.case_batches("cuda", tol, dtype)


def test_pages_and_slots_used_again():
    C.case_reuse("cuda", F32)


def test_other_sizes():
    C.case_other_sizes("cuda", F32)
    C.case_other_sizes("cuda", 0.1, torch.bfloat16)  # (tiny widths amplify the rounding)


def test_first_tokens():
    C.case_first_tokens("cuda", F32)


def test_long_decode():
    C.case_long_decode("cuda", F32)
    C.case_long_decode("cuda", BF16, torch.bfloat16)


def test_sharp_softmax_picks_far_keys():
    C.case_sharp_far_keys("cuda", 5e-4)


def test_matrix_core_shapes_bf16():
    """Head and latent sizes in multiples of 16, expert sizes in multiples of 8 and prompt portions of >= 16 queries:
    the bf16 attention, expert and head-matrix kernels that run on the matrix cores, whole and in portions with
    decoded tokens at the end; windows of 70 and 100 positions against 64-key tiles."""
    cfg = O.make_config(width=64, kinds=("attention", "latent", "shared"), heads=4, kv_heads=2, dim=32, vdim=48,
                        scale=0.2, window=70, rot_dims=16, lat_heads=4, lat_dim=16, lat_vdim=32, kv_rank=64, rot_dim=16,
                        lat_window=100, experts=8, top=3, ff=40)
    sd = O.make_weights(cfg, seed=51)
    toks = C.tokens(cfg, 200, 8)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "w", toks, [200]), want) < BF16
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [64, 70, 50] + [1] * 16), want) < BF16


def test_serving_head_sizes():
    """The head sizes of the bench presets (128-wide attention heads, a latent of 192 with a rotated part of 64) at a
    small width, windows of 80 and 130, prompts and decoded tokens, both precisions."""
    cfg = O.make_config(width=128, vocab=128, kinds=("attention", "latent", "shared"), heads=4, kv_heads=2, dim=128,
                        vdim=128, scale=0.09, window=80, rot_dims=128, lat_heads=4, lat_dim=128, lat_vdim=128,
                        kv_rank=192, rot_dim=64, lat_window=130, lat_scale=0.07, experts=4, top=2, ff=64)
    sd = O.make_weights(cfg, seed=57)
    toks = C.tokens(cfg, 150, 11)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [70, 64] + [1] * 16), want) < BF16
    _, eng = C.build(cfg, sd, "cuda", torch.float32)
    assert C.rel_err(C.feed_in_portions(eng, "d", toks, [70, 64] + [1] * 16), want) < F32


def test_many_heads_on_one_latent():
    """More than 16 heads share the one cached row of a latent layer: the decode kernel packs them 16 to a
    workgroup; with a window, sinks and key splits, both precisions."""
    cfg = O.make_config(width=64, kinds=("latent", "shared"), no_mlp=(0, 1), lat_heads=20, lat_dim=16, lat_vdim=16,
                        kv_rank=32, rot_dim=16, lat_window=90)
    sd = O.make_weights(cfg, seed=61)
    toks = C.tokens(cfg, 160, 13)
    want = O.forward(cfg, sd, toks)
    for dtype, tol in ((torch.bfloat16, BF16), (torch.float32, F32)):
        _, eng = C.build(cfg, sd, "cuda", dtype)
        assert C.rel_err(C.feed_in_portions(eng, "m", toks, [100, 33] + [1] * 27), want) < tol


def test_key_splits_with_windows():
    """Windows longer than the decode kernel's single-pass limit take the engine's key splits: splits that lie wholly
    before the query's window are empty, the split that holds the window's oldest key starts inside it."""
    cfg = O.make_config(width=64, kinds=("attention", "latent"), no_mlp=(0, 1), heads=4, kv_heads=2, dim=16, vdim=16,
                        scale=0.4, window=1100, rot_dims=8, lat_heads=2, lat_dim=16, lat_vdim=16, kv_rank=32, rot_dim=16,
                        lat_window=1200)
    sd = O.make_weights(cfg, seed=59)
    toks = C.tokens(cfg, 1300, 12)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16, pool_tokens=1408)
    assert C.rel_err(C.feed_in_portions(eng, "k", toks, [1090] + [1] * 20 + [170] + [1] * 20), want) < BF16
    # windows below the single-pass limit take the splits too when few sequences decode: parts before the window are
    # empty, the window starts inside a part
    cfg = O.make_config(width=64, kinds=("attention", "latent"), no_mlp=(0, 1), heads=4, kv_heads=2, dim=16, vdim=16,
                        scale=0.4, window=700, rot_dims=8, lat_heads=2, lat_dim=16, lat_vdim=16, kv_rank=32, rot_dim=16,
                        lat_window=900)
    sd = O.make_weights(cfg, seed=60)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16, pool_tokens=1408)
    assert C.rel_err(C.feed_in_portions(eng, "s", toks, [1250] + [1] * 50), want) < BF16


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
