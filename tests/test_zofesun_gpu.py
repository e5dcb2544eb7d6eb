"""Zofesun on the HIP kernels (cuda:0): every mechanism alone and the engine scenarios of zofesun_cases.py
against the float64 oracle -- in fp32 (the kernels' 32-bit parts are then the whole computation: tight bounds)
and in bf16 (the serving precision)."""
import pytest
import torch

import test_zofesun as T
import zofesun_cases as C

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
    assert hasattr(_lib.lib(), "grag_sink_attn_prefill") and hasattr(_lib.lib(), "grag_mingru_scan")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 0.03)])
def test_sink_attention_far_keys_and_page_borders(dtype, tol):
    T.sink_attention_case("cuda", dtype, tol)
    T.sink_attention_case("cuda", dtype, tol, T=67, far=(0, 3, 4, 63, 64), bs=4)


@pytest.mark.parametrize("d,vd", [(32, 48), (64, 16), (128, 128), (16, 256), (48, 32), (80, 112)])
def test_sink_attention_matrix_core_shapes(d, vd):
    """bf16 with head sizes in multiples of 16: prompt portions of >= 16 queries run on the matrix cores."""
    T.sink_attention_case("cuda", torch.bfloat16, 0.03, T=150, far=(0, 15, 16, 64, 131), d=d, vd=vd)
    T.sink_attention_case("cuda", torch.bfloat16, 0.03, T=200, far=(63, 128, 191), bs=4, d=d, vd=vd)


@pytest.mark.parametrize("H,G,d,vd", [(4, 2, 32, 48), (14, 2, 128, 128), (16, 1, 16, 32), (3, 3, 64, 16)])
def test_decode_key_splits(H, G, d, vd):
    """One decoded token over a long context cut into key splits that are merged afterwards: the sink counts once,
    empty splits (a context shorter than the plan) add nothing, heads that share a kv head ride in one block."""
    from githubrepostorag_amd.ops.attention import AttnMetadata, sink_attention
    import zofesun_oracle as O

    g = torch.Generator().manual_seed(5)
    bf = torch.bfloat16
    lens = [700, 65, 1, 256]
    B, bs = len(lens), 16
    i32 = dict(dtype=torch.int32, device="cuda")
    nbmax = -(-max(lens) // bs)
    kc = torch.zeros(B * nbmax + 1, G, bs, d, dtype=bf, device="cuda")
    vc = torch.zeros(B * nbmax + 1, G, bs, vd, dtype=bf, device="cuda")
    bt = torch.zeros(B, nbmax, dtype=torch.int32)
    sinks = torch.randn(H, generator=g)
    qs, want = [], []
    perm = torch.randperm(B * nbmax, generator=g) + 1
    for b, n in enumerate(lens):
        q = (torch.randn(n, H, d, generator=g) * 0.4).to(bf).float()
        k = (torch.randn(n, G, d, generator=g) * 0.4).to(bf).float()
        v = torch.randn(n, G, vd, generator=g).to(bf).float()
        k[n // 3, :, 1] = 5.0
        q[n - 1, :, 1] = 4.0  # a key far back that stands out
        want.append(O.sink_attention(q[n - 1:].double(), k.double(), v.double(), 0.7, sinks.double())[0]
                    if n == 1 else O.sink_attention(q.double(), k.double(), v.double(), 0.7, sinks.double())[n - 1])
        pages = perm[b * nbmax:(b + 1) * nbmax]
        bt[b] = pages.to(torch.int32)
        pos = torch.arange(n)
        kc[pages[pos // bs], :, pos % bs] = k.to(bf).cuda()
        vc[pages[pos // bs], :, pos % bs] = v.to(bf).cuda()
        qs.append(q[n - 1])
    qd = torch.stack(qs).to(bf).cuda().contiguous()
    for nsplit, split_len in ((1, 1 << 30), (4, 256), (16, 64), (8, 128)):
        meta = AttnMetadata(q_start=torch.arange(B + 1, **i32), ctx_len=torch.tensor(lens, **i32),
                            block_tables=bt.cuda(), slot_mapping=None, max_q_len=1, num_seqs=B, num_tokens=B,
                            is_decode=True, num_splits=nsplit, split_len=split_len,
                            part_o=torch.full((nsplit * B * H * vd,), float("nan"), device="cuda"),
                            part_ml=torch.full((nsplit * B * H * 2,), float("nan"), device="cuda"))
        got = sink_attention(qd, kc, vc, meta, 0.7, sinks.cuda(), out_scale=1.5).double().cpu().view(B, H, vd)
        for b in range(B):
            err = float((got[b] - 1.5 * want[b]).abs().max())
            assert err < 0.03, (nsplit, b, err)


def test_matrix_core_shapes_through_the_engine():
    kw = dict(dim=32, vdim=48, rot_dims=16, lin_dim=16, lin_vdim=32)
    C.case_whole_and_layers("cuda", BF16, torch.bfloat16, **kw)
    C.case_prefill_vs_decode("cuda", BF16, torch.bfloat16, n=150, **kw)
    C.case_prefill_vs_decode("cuda", F32, torch.float32, n=150, **kw)
    C.case_generate("cuda", torch.bfloat16, graphs=True, window=4, tol=0.05, **kw)


def test_sink_attention_wide_heads():
    """Head sizes past one 64-lane pass, and a key tile that does not fit 64 keys."""
    from githubrepostorag_amd.ops.attention import AttnMetadata, sink_attention
    import zofesun_oracle as O

    g = torch.Generator().manual_seed(4)
    for (H, G, d, vd, n) in ((2, 1, 200, 136, 70), (3, 3, 256, 256, 40)):
        q, k, v = (torch.randn(n, H, d, generator=g) * 0.2, torch.randn(n, G, d, generator=g) * 0.2,
                   torch.randn(n, G, vd, generator=g))
        sinks = torch.randn(H, generator=g)
        want = O.sink_attention(q.double(), k.double(), v.double(), 0.5, sinks.double())
        kc, vc, bt, _ = T._paged(k, v, 16)
        i32 = dict(dtype=torch.int32, device="cuda")
        for a in (0, n - 1):
            m = n - a
            meta = AttnMetadata(q_start=torch.tensor([0, m], **i32), ctx_len=torch.tensor([n], **i32),
                                block_tables=bt.cuda(), slot_mapping=None, max_q_len=m, num_seqs=1, num_tokens=m,
                                is_decode=(m == 1))
            got = sink_attention(q[a:].cuda().contiguous(), kc.cuda(), vc.cuda(), meta, 0.5, sinks.cuda())
            assert float((got.double().cpu().view(m, H, vd) - want[a:]).abs().max()) < 2e-5


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-5)])
def test_recurrent_mixers_alone(dtype, tol):
    T.recurrent_case("cuda", dtype, tol)  # (bf16 inputs are rounded before both sides: the recurrences are fp32)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 0.03)])
def test_elementwise_mechanisms_alone(dtype, tol):
    T.elementwise_case("cuda", dtype, tol)


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
    C.case_other_sizes("cuda", BF16, torch.bfloat16)


def test_first_tokens():
    C.case_first_tokens("cuda", F32)


def test_long_decode():
    C.case_long_decode("cuda", F32)


@pytest.mark.parametrize("graphs,mixed,window,max_batched", [(False, False, 1, 4096), (True, False, 1, 4096),
                                                             (True, False, 4, 4096), (False, True, 1, 8)])
def test_greedy_generation(graphs, mixed, window, max_batched):
    C.case_generate("cuda", graphs=graphs, mixed=mixed, window=window, max_batched=max_batched)


def test_bf16_batch_invariance():
    """bf16 serving: a request's logits beside other requests equal its logits alone (the same kernels see the
    same operands per row; only GEMM tiling may differ with the batch's row count)."""
    import numpy as np
    import zofesun_oracle as O

    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=37)
    a, b = C.tokens(cfg, 40, 1), C.tokens(cfg, 13, 2)
    _, eng = C.build(cfg, sd, "cuda", torch.bfloat16)
    alone = C.feed_in_portions(eng, "a", a, [40])
    o1 = eng.feed([("a2", a[:25], list(range(25))), ("b", b[:12], [])], [])
    o2 = eng.feed([("a2", a[25:], list(range(15))), ("b", b[12:], [0])], ["a2", "b"])
    assert C.rel_err(np.concatenate([o1, o2[:15]], 0), alone) < 0.02
