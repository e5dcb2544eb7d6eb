"""Namudra on the HIP kernels (cuda:0): every mechanism alone and the engine scenarios of namudra_cases.py against
the float64 oracle -- in fp32 (the kernels' 32-bit parts are then the whole computation: tight bounds) and in bf16
(the serving precision)."""
import numpy as np
import pytest
import torch

import namudra_cases as C
import namudra_oracle as O
import test_namudra as T

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
    for name in ("grag_hyper_mix", "grag_qk_norm_store", "grag_latent_store", "grag_sigmoid_window_prefill",
                 "grag_sigmoid_window_decode", "grag_rmsnorm_rows"):
        assert hasattr(_lib.lib(), name)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.03)])
def test_hyper_connection_boundary(dtype, tol):
    T.hyper_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 0.12)])
def test_retention_alone(dtype, tol):
    # (bf16: the projections are rounded before a recurrence that forgets nothing in one head; outputs are O(1))
    T.retention_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.05)])
def test_window_attention_alone(dtype, tol):
    T.window_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 0.05)])
def test_latent_attention_alone(dtype, tol):
    T.latent_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 0.01)])
def test_glu_alone(dtype, tol):
    T.glu_case("cuda", dtype, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-5)])
def test_window_edges_in_prompts_and_decoding(dtype, tol):
    C.case_window_edges("cuda", tol, dtype)  # (keys, queries and values are exact in bf16)
    C.case_window_edges("cuda", tol, dtype, bs=4)


@pytest.mark.parametrize("kind", ["retention", "attention", "latent_attention"])
def test_single_mixer_models(kind):
    C.case_single_mixer("cuda", F32, kind)
    C.case_single_mixer("cuda", BF16, kind, torch.bfloat16)


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
    C.case_other_sizes("cuda", 0.15, torch.bfloat16)  # (ranks of 4-8 and three passes amplify the rounding)
    C.case_inferred_rank("cuda", F32)


def test_first_tokens():
    C.case_first_tokens("cuda", F32)


def test_long_decode():
    C.case_long_decode("cuda", F32)


def test_sharp_softmax_picks_far_keys():
    C.case_sharp_far_keys("cuda", 5e-4)


def test_matrix_core_shapes_bf16():
    """Head sizes in multiples of 16 and prompt portions of >= 16 queries: the bf16 attention kernels that run on
    the matrix cores, against the oracle, whole and in portions with decoded tokens at the end."""
    cfg = O.make_config(width=64, kinds=("attention", "latent_attention", "retention"), loop=(0, 2, 2), no_mlp=(2,),
                        att=dict(heads=4, kv_heads=2, dim=32, vdim=32, scale=0.2, mask={"size": 70}),
                        lat=dict(heads=4, dim=16, rot_dim=16, vdim=16, kv_rank=48, q_rank=32, scale=0.25),
                        ret=dict(heads=2, dim=16, vdim=32, decay=[0.95, 0.999], rot={"dims": 16, "base": 1000.0}))
    sd = O.make_weights(cfg, seed=51)
    toks = C.tokens(cfg, 200, 8)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "w", toks, [200]), want) < BF16
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [64, 70, 50] + [1] * 16), want) < BF16


def test_serving_head_sizes_bf16():
    """The head sizes of the bench presets (128-wide heads, a latent of 192 + 64 rotated: key rows of 256) at a small
    width: the widest instantiations of the matrix-core kernels, prompts and decoded tokens."""
    cfg = O.make_config(width=128, vocab=128, kinds=("retention", "attention", "latent_attention"), loop=(0, 0, 1),
                        no_mlp=(0, 1, 2), ret=dict(heads=2, dim=128, vdim=128, decay=[0.98, 0.999], rot={"dims": 128, "base": 1e4}),
                        att=dict(heads=4, kv_heads=2, dim=128, vdim=128, scale=0.09, mask={"size": 80}),
                        lat=dict(heads=4, dim=128, rot_dim=64, vdim=128, kv_rank=192, q_rank=96, scale=0.07))
    sd = O.make_weights(cfg, seed=57)
    toks = C.tokens(cfg, 150, 11)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [70, 64] + [1] * 16), want) < BF16
    _, eng = C.build(cfg, sd, "cuda", torch.float32)
    assert C.rel_err(C.feed_in_portions(eng, "d", toks, [70, 64] + [1] * 16), want) < F32


def test_more_than_sixteen_heads_per_kv_head_bf16():
    """Decode kernels that pack the heads of one kv head into 16 matrix-core columns take them in groups: 18 heads
    on one kv head (windowed attention), 20 heads on the latent cache."""
    cfg = O.make_config(width=64, kinds=("attention", "latent_attention"), loop=(0, 0, 1), no_mlp=(0,),
                        att=dict(heads=18, kv_heads=1, dim=16, vdim=16, scale=0.3, mask={"size": 50}),
                        lat=dict(heads=20, dim=16, rot_dim=16, vdim=16, kv_rank=32, q_rank=32, scale=0.25))
    sd = O.make_weights(cfg, seed=53)
    toks = C.tokens(cfg, 120, 9)
    want = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "c", toks, [90] + [1] * 30), want) < BF16
    _, eng = C.build(cfg, sd, "cuda", torch.float32)
    assert C.rel_err(C.feed_in_portions(eng, "d", toks, [90] + [1] * 30), want) < F32


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
