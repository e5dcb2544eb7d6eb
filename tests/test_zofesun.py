"""Zofesun on the engine, CPU tier: the engine's cache / state / scheduler logic and the ops' host paths against
the float64 oracle (tests/zofesun_oracle.py); the same scenarios run on the HIP kernels in test_zofesun_gpu.py."""
import json

import numpy as np
import pytest
import torch

import zofesun_cases as C
import zofesun_oracle as O

TOL = 2e-5


def test_whole_prompt_and_layer_taps():
    C.case_whole_and_layers("cpu", TOL)


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


@pytest.mark.parametrize("mixed,max_batched", [(False, 4096), (True, 8)])
def test_greedy_generation(mixed, max_batched):
    C.case_generate("cpu", mixed=mixed, max_batched=max_batched)


def test_generation_survives_preemption():
    """A KV pool too small for all running requests: the scheduler preempts one (pages and slot freed) and
    recomputes it later from its first token -- its recurrent state restarts from zero with it."""
    from githubrepostorag_amd.engine.sequence import SamplingParams

    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=41)
    _, eng = C.build(cfg, sd, "cpu", slots=3, pool_tokens=96)
    prompts = [C.tokens(cfg, 5, 90 + i) for i in range(3)]  # admitted together (a page each), then they grow
    outs = eng.generate(prompts, SamplingParams(max_tokens=40, temperature=0.0, ignore_eos=True))
    assert eng.sched.num_preemptions > 0
    for p, c in zip(prompts, outs):
        logits, _ = O.forward(cfg, sd, p + c.token_ids[:-1])
        for j, t in enumerate(c.token_ids):
            row = logits[len(p) - 1 + j]
            assert float(row.max() - row[t]) < 2e-3 * float(row.std())


def test_bf16_close_to_oracle():
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=23)
    toks = C.tokens(cfg, 33, 5)
    want, _ = O.forward(cfg, sd, toks)
    _, eng = C.build(cfg, sd, "cpu", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "a", toks, [9, 1]), want) < 0.05


def test_config_round_trip_and_layer_runs():
    from githubrepostorag_amd.models.configs import (decoder_config, hybrid_config_from_dict,
                                                     hybrid_config_to_dict)

    d = O.make_config(kinds=("parallel", "mingru", "parallel", "mingru"), loop=(1, 3, 3), no_mlp=(2,))
    cfg = hybrid_config_from_dict(d)
    assert hybrid_config_to_dict(cfg) == d
    assert [(i, t) for i, t, _ in cfg.layer_runs()] == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (3, 0)]
    assert [f for _, _, f in cfg.layer_runs()] == [False, True, False, True, False, True, False, False]
    assert decoder_config("zofesun-tiny").arch == "zofesun"
    with pytest.raises(ValueError):
        hybrid_config_from_dict({**d, "loop": {"start": 3, "stop": 2, "times": 1}}).layer_runs()
    bad = json.loads(json.dumps(d))
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        hybrid_config_from_dict(bad)


def test_checkpoint_directory_and_cli(tmp_path, capsys):
    """config.json + model.safetensors on disk -> the registry picks the class; the trace and generate commands
    run it through the engine."""
    from githubrepostorag_amd.cli import main
    from githubrepostorag_amd.engine.trace import run_trace
    from githubrepostorag_amd.models.weights import save_state_dict

    cfg = O.make_config(loop=(0, 2, 2))
    sd = O.make_weights(cfg, seed=29)
    (tmp_path / "m").mkdir()
    (tmp_path / "m" / "config.json").write_text(json.dumps(cfg))
    save_state_dict(sd, tmp_path / "m" / "model.safetensors")
    a, b = C.tokens(cfg, 21, 1), C.tokens(cfg, 6, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:19], "want": [0, 18]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[19:20], "want": []}, {"id": "b", "tokens": b, "want": [5]}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[20:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    assert run_trace(str(tmp_path / "m"), "float32", str(out), 128, device="cpu",
                     lines=[json.dumps(s) for s in steps]) == 0
    assert "done 0" in capsys.readouterr().out
    wa, wb = O.forward(cfg, sd, a)[0], O.forward(cfg, sd, b)[0]
    g0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    g1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)
    g2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    assert C.rel_err(g0, wa[[0, 18]]) < TOL and C.rel_err(g1, wb[[5]]) < TOL and C.rel_err(g2, wa[[20]]) < TOL
    assert main(["generate", "--model", str(tmp_path / "m"), "--dtype", "float32", "--device", "cpu", "--prompt-ids",
                 "1,2,3", "4", "--max-tokens", "3"]) == 0
    lines = [json.loads(x) for x in capsys.readouterr().out.strip().splitlines()]
    assert [len(x["token_ids"]) for x in lines] == [3, 3]


def test_plan_errors():
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=31)
    _, eng = C.build(cfg, sd, "cpu", slots=1, pool_tokens=32)
    eng.feed([("a", [1, 2, 3], [])], [])
    with pytest.raises(RuntimeError):
        eng.feed([("b", [1], [])], [])          # no slot left
    with pytest.raises(MemoryError):
        eng.feed([("a", list(range(40)), [])], [])  # pool too small
    with pytest.raises(ValueError):
        eng.feed([("a", [1], [3])], [])         # wanted place outside the entry


# ------------------------------------------------------------------------------------------------ mechanisms alone
def _paged(k, v, bs, perm_seed=0, extra=3):
    """Scatter k [T, G, d] / v [T, G, vd] over shuffled pages -> (k_cache, v_cache, block table row, slots)."""
    T, G, d = k.shape
    vd = v.shape[2]
    nb = -(-T // bs)
    g = torch.Generator().manual_seed(perm_seed)
    pages = (torch.randperm(nb + extra, generator=g)[:nb] + 1)
    kc = torch.full((nb + extra + 1, G, bs, d), 7.0)
    vc = torch.full((nb + extra + 1, G, bs, vd), -7.0)
    pos = torch.arange(T)
    slots = pages[pos // bs] * bs + pos % bs
    kc[pages[pos // bs], :, pos % bs] = k
    vc[pages[pos // bs], :, pos % bs] = v
    return kc, vc, pages.to(torch.int32).view(1, nb), slots.to(torch.int32)


def sink_attention_case(device, dtype, tol, T=150, far=(0, 15, 16, 17, 63, 64, 131), bs=16, d=12, vd=20):
    """One far key made to dominate (query and key scaled along one direction): the output is that key's value,
    wherever the key lies -- page borders, the first token -- for a prompt chunk and for a decoded token; the
    sink takes its share of the denominator."""
    from githubrepostorag_amd.ops.attention import AttnMetadata, sink_attention

    H, G = 4, 2
    g = torch.Generator().manual_seed(1)
    for key in far:
        q = torch.randn(T, H, d, generator=g) * 0.3 * (12.0 / d) ** 0.5
        k = torch.randn(T, G, d, generator=g) * 0.3 * (12.0 / d) ** 0.5
        v = torch.randn(T, G, vd, generator=g)
        k[key, :, 0] = 6.0
        q[T - 1, :, 0] = 6.0
        q[T - 2, :, 0] = 6.0
        sinks = torch.tensor([-2.0, 0.5, 3.0, 40.0])
        if dtype == torch.bfloat16:
            q, k, v = (t.to(dtype).float() for t in (q, k, v))
        want = O.sink_attention(q.double(), k.double(), v.double(), 1.0, sinks.double())
        assert float((want[T - 1, 0] - v[key, 0].double()).abs().max()) < 0.05      # the far key wins head 0
        assert float(want[T - 1, 3].abs().max()) < 0.05 * float(v[key, 1].abs().max())  # a huge sink drains head 3
        kc, vc, bt, _ = _paged(k, v, bs, perm_seed=key)
        i32 = dict(dtype=torch.int32, device=device)
        kc, vc = kc.to(device, dtype), vc.to(device, dtype)
        for a in (0, T - 2, T - 1):  # a whole prompt, a two-token portion, one decoded token
            n = T - a
            meta = AttnMetadata(q_start=torch.tensor([0, n], **i32), ctx_len=torch.tensor([T], **i32),
                                block_tables=bt.to(device), slot_mapping=None, max_q_len=n, num_seqs=1, num_tokens=n,
                                is_decode=(n == 1))
            got = sink_attention(q[a:].to(device, dtype).contiguous(), kc, vc, meta, 1.0, sinks.to(device))
            err = (got.double().cpu().view(n, H, vd) - want[a:]).abs().max()
            assert float(err) < tol, (key, a, float(err))


def test_sink_attention_far_keys_and_page_borders():
    sink_attention_case("cpu", torch.float32, 1e-5)


def recurrent_case(device, dtype, tol):
    """Decay linear attention and minGRU: portions of a sequence through carried state equal the oracle's single
    pass; decay 1.0 (nothing forgotten) and a tiny decay both hold; a far token still shows through decay 1."""
    from githubrepostorag_amd.ops.attention import AttnMetadata
    from githubrepostorag_amd.ops.recurrent import decay_attention, mingru_scan

    T, H, d, vd, W = 90, 4, 6, 10, 37
    g = torch.Generator().manual_seed(2)
    proj = torch.randn(T, H * (2 * d + vd) + 5, generator=g)
    proj[3, 2 * H * d + 5:] += 8.0  # a far token with a large value
    decay = torch.tensor([1.0, 0.05, 0.98, 1e-9])
    x = proj.to(dtype).double()
    q, k, v = (O.silu(x[:, 5:5 + H * d]).view(T, H, d), O.silu(x[:, 5 + H * d:5 + 2 * H * d]).view(T, H, d),
               O.silu(x[:, 5 + 2 * H * d:]).view(T, H, vd))
    want = O.decay_attention(q, k, v, decay.double().tolist()).reshape(T, -1)
    gp = torch.randn(T, 3 * W, generator=g) * 2
    bz, bx = torch.randn(W, generator=g), torch.randn(W, generator=g)
    y = gp.to(dtype).double()
    wg = O.mingru(y[:, :W] + bz.double(), y[:, W:2 * W] + bx.double()) * O.silu(y[:, 2 * W:])
    i32 = dict(dtype=torch.int32, device=device)
    for cuts in ([T], [1] * T, [7, 2, 1, 30, 50]):
        S = torch.full((3, H, d, vd), 9.0, device=device)  # a used slot: must not leak into a new sequence
        Sg = torch.full((3, W), 9.0, device=device)
        outs, outg, a = [], [], 0
        for n in cuts:
            meta = AttnMetadata(q_start=torch.tensor([0, n], **i32), ctx_len=torch.tensor([a + n], **i32),
                                block_tables=None, slot_mapping=None, max_q_len=n, num_seqs=1, num_tokens=n,
                                is_decode=(n == 1), state_slots=torch.tensor([2], **i32))
            outs.append(decay_attention(proj[a:a + n].to(device, dtype).contiguous(), 5, 5 + H * d, 5 + 2 * H * d,
                                        decay.to(device), S, meta, H, d, vd))
            outg.append(mingru_scan(gp[a:a + n].to(device, dtype).contiguous(), 0, W, 2 * W, bz.to(device),
                                    bx.to(device), Sg, meta, W))
            a += n
        err = (torch.cat(outs).double().cpu() - want).abs().max() / want.abs().max()
        assert float(err) < tol, (cuts, float(err))
        errg = (torch.cat(outg).double().cpu() - wg).abs().max() / wg.abs().max()
        assert float(errg) < (tol if dtype == torch.float32 else 0.01), (cuts, float(errg))  # (bf16 outputs)
        assert float(S[0].min()) == 9.0 and float(Sg[1].max()) == 9.0  # other slots untouched


def test_recurrent_mixers_alone():
    recurrent_case("cpu", torch.float32, 1e-5)


def elementwise_case(device, dtype, tol):
    from githubrepostorag_amd.ops.elementwise import clamped_glu, rope_table, rope_vnorm_store
    from githubrepostorag_amd.ops.norm import dyt_residual, embed_gather_f32
    from githubrepostorag_amd.ops.recurrent import gated_rmsnorm

    g = torch.Generator().manual_seed(3)
    T, Hd = 9, 50
    x = torch.randn(T, Hd, generator=g) * 3
    y = (torch.randn(T, Hd, generator=g) * 3).to(dtype)
    w1, b1, w2, b2 = (torch.randn(Hd, generator=g) for _ in range(4))
    rows, vec = torch.randn(T, Hd, generator=g), torch.randn(Hd, generator=g)
    want_x = x.double() + O.dyt(y.double(), 0.7, w1.double(), b1.double()) + rows.double() + vec.double()
    want_h = O.dyt(want_x, 1.3, w2.double(), b2.double())
    r = x.clone().to(device)
    h = dyt_residual(r, y.to(device), (0.7, w1.to(device), b1.to(device)), rows.to(device), vec.to(device),
                     (1.3, w2.to(device), b2.to(device)), out_dtype=dtype)
    assert float((r.double().cpu() - want_x).abs().max()) < 1e-5
    assert float((h.double().cpu() - want_h).abs().max()) < tol
    # clamped GLU: values on both sides of every clamp
    gu = torch.tensor([[-3.0, 0.2, 0.9, 5.0, -0.5, -4.0, 0.3, 7.0]]).to(dtype)
    got = clamped_glu(gu.to(device), 0.8)
    want = O.clamped_glu(gu[:, :4].double(), gu[:, 4:].double(), 0.8)
    assert float((got.double().cpu() - want).abs().max()) < tol
    # gated RMS norm over the whole row
    o = torch.randn(T, 24, generator=g)
    pr = torch.randn(T, 30, generator=g).to(dtype)
    wn = torch.randn(24, generator=g)
    out = torch.zeros(T, 40, dtype=dtype, device=device)
    gated_rmsnorm(o.to(device), wn.to(device), pr.to(device), 6, 1e-5, out[:, 16:], out_scale=1.7)
    want = 1.7 * O.unit_rms(o.double(), 1e-5) * wn.double() * torch.sigmoid(pr[:, 6:].double())
    assert float((out[:, 16:].double().cpu() - want).abs().max()) < tol and float(out[:, :16].abs().max()) == 0
    # rotary on the first dims only + value norm + paged store
    H, G, d, vd, rd, bs = 4, 2, 10, 6, 4, 4
    proj = torch.randn(T, 3 + H * d + G * d + G * vd, generator=g).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 4, 5, 6, 700, 701], dtype=torch.int32)
    tab = rope_table(1024, rd, 50.0, device)
    slots = torch.tensor([4, 5, 6, 7, 12, 13, 14, -1, 9], dtype=torch.int32)
    kc = torch.zeros(5, G, bs, d, dtype=dtype, device=device)
    vc = torch.zeros(5, G, bs, vd, dtype=dtype, device=device)
    q = rope_vnorm_store(proj.to(device), 3, 3 + H * d, 3 + H * d + G * d, pos.to(device), tab, slots.to(device), kc,
                         vc, H, G, d, vd, rd, 1e-5)
    pd = proj.double()
    for t in range(T):
        qt = pd[t, 3:3 + H * d].view(1, H, d)
        kt = pd[t, 3 + H * d:3 + H * d + G * d].view(1, G, d)
        full_q = torch.zeros(int(pos[t]) + 1, H, d, dtype=torch.float64)
        full_k = torch.zeros(int(pos[t]) + 1, G, d, dtype=torch.float64)
        full_q[-1], full_k[-1] = qt[0], kt[0]
        wq, wk = O.rotate(full_q, rd, 50.0)[-1], O.rotate(full_k, rd, 50.0)[-1]
        assert float((q[t].double().cpu() - wq).abs().max()) < tol
        wv = O.unit_rms(pd[t, 3 + H * d + G * d:].view(G, vd), 1e-5)
        s = int(slots[t])
        if s >= 0:
            assert float((kc[s // bs, :, s % bs].double().cpu() - wk).abs().max()) < tol
            assert float((vc[s // bs, :, s % bs].double().cpu() - wv).abs().max()) < tol
    assert float(kc[0].abs().max()) == 0 and float(kc[2, :, 0].abs().max()) == 0  # nothing stored for slot -1
    tbl = torch.randn(11, 7, generator=g).to(dtype)
    ids = torch.tensor([3, 0, 10], dtype=torch.int32)
    assert torch.equal(embed_gather_f32(ids.to(device), tbl.to(device)).cpu(), tbl[ids.long()].float())


def test_elementwise_mechanisms_alone():
    elementwise_case("cpu", torch.float32, 1e-5)
