"""Namudra on the engine, CPU tier: the engine's cache / state / scheduler logic and the ops' host paths against
the float64 oracle (tests/namudra_oracle.py); the same scenarios run on the HIP kernels in test_namudra_gpu.py."""
import json
import math

import numpy as np
import pytest
import torch

import namudra_cases as C
import namudra_oracle as O

TOL = 2e-5


def test_whole_prompt_and_layer_taps():
    C.case_whole_and_layers("cpu", TOL)


@pytest.mark.parametrize("kind", ["retention", "attention", "latent_attention"])
def test_single_mixer_models(kind):
    C.case_single_mixer("cpu", TOL, kind)


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
    C.case_inferred_rank("cpu", TOL)


def test_first_tokens():
    C.case_first_tokens("cpu", TOL)


def test_long_decode():
    C.case_long_decode("cpu", TOL)


def test_sharp_softmax_picks_far_keys():
    C.case_sharp_far_keys("cpu", 2e-4)


def test_window_edges_in_prompts_and_decoding():
    C.case_window_edges("cpu", 1e-5)


@pytest.mark.parametrize("mixed,max_batched", [(False, 4096), (True, 8)])
def test_greedy_generation(mixed, max_batched):
    C.case_generate("cpu", mixed=mixed, max_batched=max_batched)


def test_bf16_close_to_oracle():
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=23)
    toks = C.tokens(cfg, 33, 5)
    _, eng = C.build(cfg, sd, "cpu", torch.bfloat16)
    assert C.rel_err(C.feed_in_portions(eng, "a", toks, [9, 1]), O.forward(cfg, sd, toks)) < 0.06


def test_config_round_trip_and_registry():
    from githubrepostorag_amd.models import build_decoder
    from githubrepostorag_amd.models.configs import (decoder_config, namudra_config_from_dict,
                                                     namudra_config_to_dict)
    from githubrepostorag_amd.models.namudra import NamudraModel

    d = O.make_config(kinds=("retention", "attention", "latent_attention", "retention"), loop=(1, 3, 3), no_mlp=(0, 3))
    cfg = namudra_config_from_dict(d)
    assert namudra_config_to_dict(cfg) == d
    assert [(i, t) for i, t, _ in cfg.layer_runs()] == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (3, 0)]
    tiny = decoder_config("namudra-tiny")
    assert tiny.arch == "namudra" and isinstance(build_decoder(tiny, device="cpu", dtype=torch.float32), NamudraModel)
    bad = json.loads(json.dumps(d))
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        namudra_config_from_dict(bad)
    bad = json.loads(json.dumps(d))
    bad["layers"][1]["mixer"]["vdim"] = 12  # the values are the keys: no other size
    with pytest.raises(ValueError):
        namudra_config_from_dict(bad)
    sd = O.make_weights(d, seed=1)
    sd["l1.mix.pb"] = sd["l1.mix.pb"][:-1]
    with pytest.raises(ValueError):
        build_decoder(cfg, device="cpu", dtype=torch.float32, state_dict=sd)


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
    wa, wb = O.forward(cfg, sd, a), O.forward(cfg, sd, b)
    g0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    g1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)
    g2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)
    assert C.rel_err(g0, wa[[0, 18]]) < TOL and C.rel_err(g1, wb[[5]]) < TOL and C.rel_err(g2, wa[[20]]) < TOL
    assert main(["generate", "--model", str(tmp_path / "m"), "--dtype", "float32", "--device", "cpu", "--prompt-ids",
                 "1,2,3", "4", "--max-tokens", "3"]) == 0
    lines = [json.loads(x) for x in capsys.readouterr().out.strip().splitlines()]
    assert [len(x["token_ids"]) for x in lines] == [3, 3]


# ------------------------------------------------------------------------------------------------ mechanisms alone
def _meta(device, lens, ctxs, bs, nb_per_seq, slots=None, decode=False):
    """Metadata of a step over sequences with ``lens`` new tokens and ``ctxs`` keys each; sequence s owns pages
    1 + s * nb_per_seq ... in reverse order (so consecutive keys are not consecutive pages)."""
    from githubrepostorag_amd.ops.attention import AttnMetadata

    i32 = dict(dtype=torch.int32, device=device)
    n = len(lens)
    bt = torch.tensor([[1 + s * nb_per_seq + (nb_per_seq - 1 - j) for j in range(nb_per_seq)] for s in range(n)], **i32)
    slot_map = []
    for s in range(n):
        for p in range(ctxs[s] - lens[s], ctxs[s]):
            slot_map.append(int(bt[s, p // bs]) * bs + p % bs)
    return AttnMetadata(q_start=torch.tensor([0] + list(np.cumsum(lens)), **i32), ctx_len=torch.tensor(ctxs, **i32),
                        block_tables=bt, slot_mapping=torch.tensor(slot_map, **i32), max_q_len=max(lens), num_seqs=n,
                        num_tokens=sum(lens), is_decode=decode,
                        state_slots=torch.tensor(slots if slots is not None else list(range(n)), **i32))


def hyper_case(device, dtype, tol):
    """Stream update, read-out and norm against the formulas, S = 1, 3 and the kernel's maximum."""
    from githubrepostorag_amd.ops.norm import hyper_mix

    g = torch.Generator().manual_seed(2)
    for S, Hd in ((1, 40), (3, 96), (8, 33)):
        T = 5
        xs = torch.randn(S, T, Hd, generator=g)
        y = torch.randn(T, Hd, generator=g).to(dtype)
        mix, outc, inc = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
        w = torch.randn(Hd, generator=g)
        new = [sum(mix[s, t].double() * xs[s].double() for s in range(S)) + outc[t].double() * y.double()
               for t in range(S)]
        u = sum(inc[s].double() * new[s] for s in range(S))
        want_h = O.norm_one_plus(u, w.double() - 1.0, 1e-5)
        d = torch.device(device)
        xd = xs.clone().to(d)
        h, usum = hyper_mix(xd, y.to(d), mix.to(d), outc.to(d), inc.to(d), w.to(d), 1e-5, dtype, want_sum=True)
        assert float((torch.stack(new) - xd.double().cpu()).abs().max()) < 1e-4
        assert float((usum.double().cpu() - u).abs().max()) < 1e-4
        assert float((h.double().cpu() - want_h).abs().max()) < tol
        # read-out only (no sublayer output pending): the streams stay as they are
        before = xd.clone()
        h2, _ = hyper_mix(xd, None, None, None, inc.to(d), w.to(d), 1e-5, dtype)
        assert torch.equal(before, xd) and float((h2.double().cpu() - want_h).abs().max()) < tol


def retention_case(device, dtype, tol):
    """The scan with rotary and key scale, the per-head unit norm and the SiLU gate against the oracle's retention
    (identity output projection): two sequences in one launch, one continuing from a stored state across a chunk
    border of the scan, then single decoded tokens."""
    from githubrepostorag_amd.ops.elementwise import rope_table
    from githubrepostorag_amd.ops.recurrent import decay_attention, gated_rmsnorm

    H, d, vd, W = 3, 12, 20, 24
    m = dict(heads=H, dim=d, vdim=vd, decay=[1.0, 0.93, 0.4], rot={"dims": 6, "base": 30.0})
    g = torch.Generator().manual_seed(4)
    wt = {n: (torch.randn(r, W, generator=g) * W ** -0.5).to(torch.bfloat16).double()
          for n, r in (("q", H * d), ("k", H * d), ("v", H * vd), ("g", H * vd))}
    wt["o"] = torch.eye(H * vd, dtype=torch.float64)
    dev = torch.device(device)
    lens = (150, 71)
    hs = [torch.randn(n, W, generator=g).to(torch.bfloat16).double() for n in lens]
    want = [O.retention(h, lambda n: wt[n], m, 1e-6) for h in hs]
    wcat = torch.cat([wt["q"], wt["k"], wt["v"], wt["g"]], 0)
    table = rope_table(256, 6, 30.0, dev)
    decay = torch.tensor(m["decay"], dtype=torch.float32, device=dev)
    state = torch.full((3, H, d, vd), 7.0, dtype=torch.float32, device=dev)   # stale values in the slots
    got = [[], []]

    def step(parts):  # parts: [(sequence, first token, end token)]
        proj = torch.cat([hs[s][a:b] @ wcat.T for s, a, b in parts], 0).to(dtype).to(dev)
        pos = torch.cat([torch.arange(a, b) for _, a, b in parts]).to(torch.int32).to(dev)
        meta = _meta(dev, [b - a for _, a, b in parts], [b for _, _, b in parts], 16, 16, slots=[2 - s for s, _, _ in parts],
                     decode=all(b - a == 1 for _, a, b in parts))
        o = decay_attention(proj, 0, H * d, 2 * H * d, decay, state, meta, H, d, vd, act=False, positions=pos,
                            rope=table, k_scale=d ** -0.5)
        y = torch.empty(proj.shape[0], H * vd, dtype=dtype, device=dev)
        gated_rmsnorm(o, None, proj, 2 * H * d + H * vd, 1e-6, y, groups=H, gate="silu")
        r = 0
        for s, a, b in parts:
            got[s].append(y[r:r + b - a].double().cpu())
            r += b - a

    step([(0, 0, 100), (1, 0, 3)])
    step([(1, 3, 70), (0, 100, 149)])
    step([(0, 149, 150), (1, 70, 71)])
    for s in range(2):
        err = float((torch.cat(got[s]) - want[s]).abs().max())
        assert err < tol, (s, err)


def window_case(device, dtype, tol):
    """q / k norm + store + windowed sigmoid attention + gate against the oracle's mixer (identity output
    projection): a prompt in two portions over shuffled pages, then decoded tokens."""
    from githubrepostorag_amd.ops.attention import sigmoid_window_attention
    from githubrepostorag_amd.ops.elementwise import qk_norm_store

    H, G, d, W, bs = 6, 2, 20, 24, 4
    m = dict(heads=H, kv_heads=G, dim=d, vdim=d, scale=0.35, mask={"size": 11})
    g = torch.Generator().manual_seed(6)
    wt = {n: (torch.randn(r, W, generator=g) * W ** -0.5).to(torch.bfloat16).double()
          for n, r in (("q", H * d), ("k", G * d), ("g", H * d))}
    wt.update({"q.norm": 1 + 0.2 * torch.randn(d, generator=g).double(), "k.norm": 1 + 0.2 * torch.randn(d, generator=g).double(),
               "pb": torch.randn(H, generator=g).double() - 1, "o": torch.eye(H * d, dtype=torch.float64)})
    T = 45
    h = torch.randn(T, W, generator=g).to(torch.bfloat16).double()
    want = O.window_attention(h, lambda n: wt[n], m, 1e-6)
    dev = torch.device(device)
    kc = torch.zeros(14, G, bs, d, dtype=dtype, device=dev)
    vc = torch.zeros_like(kc)
    wcat = torch.cat([wt["q"], wt["k"], wt["g"]], 0)
    f32 = lambda t: t.float().to(dev)
    got = []
    for a, b in ((0, 17), (17, 39)) + tuple((i, i + 1) for i in range(39, T)):
        proj = (h[a:b] @ wcat.T).to(dtype).to(dev)
        meta = _meta(dev, [b - a], [b], bs, 12, decode=b - a == 1)
        q = qk_norm_store(proj, 0, H * d, f32(wt["q.norm"]), f32(wt["k.norm"]), meta.slot_mapping, kc, vc, H, G, d, 1e-6)
        got.append(sigmoid_window_attention(q, kc, vc, meta, 0.35, f32(wt["pb"]), 11,
                                            gate=proj[:, (H + G) * d:]).double().cpu())
    assert float((torch.cat(got) - want).abs().max()) < tol


def latent_case(device, dtype, tol):
    """Norm of the query latent, latent store, rotary, softmax attention over the latent cache against the oracle's
    mixer, with the key / value expansions folded into the projections the way the model folds them."""
    from githubrepostorag_amd.ops.attention import sink_attention
    from githubrepostorag_amd.ops.elementwise import latent_store, rope_table
    from githubrepostorag_amd.ops.norm import rmsnorm_rows

    H, d, r, vd, R, Q, W, bs = 3, 10, 6, 14, 32, 18, 24, 8
    m = dict(heads=H, dim=d, rot_dim=r, vdim=vd, kv_rank=R, q_rank=Q, scale=0.9, rot={"dims": r, "base": 20.0})
    g = torch.Generator().manual_seed(8)
    rnd = lambda *s: (torch.randn(*s, generator=g) * s[-1] ** -0.5).to(torch.bfloat16).double()
    wt = {"dq": rnd(Q, W), "uq": rnd(H * (d + r), Q), "dkv": rnd(R + r, W), "uk": rnd(H * d, R), "uv": rnd(H * vd, R),
          "dq.norm": 1 + 0.2 * torch.randn(Q, generator=g).double(), "dkv.norm": 1 + 0.2 * torch.randn(R, generator=g).double(),
          "o": torch.eye(H * vd, dtype=torch.float64)}
    T = 61
    h = torch.randn(T, W, generator=g).to(torch.bfloat16).double()
    want = O.latent_attention(h, lambda n: wt[n], m, 1e-6)
    uq, uk, uv = wt["uq"].view(H, d + r, Q), wt["uk"].view(H, d, R), wt["uv"].view(H, vd, R)
    wq = torch.cat([torch.einsum("hdr,hdq->hrq", uk, uq[:, :d]), uq[:, d:]], 1).reshape(H * (R + r), Q)
    dev = torch.device(device)
    kc = torch.zeros(10, 1, bs, R + r, dtype=dtype, device=dev)
    vc = kc[..., :R]  # the values are the latents: the head of the same rows
    table = rope_table(128, r, 20.0, dev)
    f32 = lambda t: t.float().to(dev)
    got = []
    for a, b in ((0, 23), (23, 50)) + tuple((i, i + 1) for i in range(50, T)):
        proj = (h[a:b] @ torch.cat([wt["dq"], wt["dkv"]], 0).T).to(dtype).to(dev)
        meta = _meta(dev, [b - a], [b], bs, 8, decode=b - a == 1)
        cq = rmsnorm_rows(proj[:, :Q], f32(wt["dq.norm"]), 1e-6)
        q = (cq.double().cpu() @ wq.T).to(dtype).to(dev).view(b - a, H, R + r).contiguous()
        latent_store(proj[:, Q:], f32(wt["dkv.norm"]), torch.arange(a, b, dtype=torch.int32, device=dev), table,
                     meta.slot_mapping, q, kc, 1e-6)
        o = sink_attention(q, kc, vc, meta, 0.9, None).double().cpu().view(b - a, H, R)
        got.append(torch.einsum("thr,hvr->thv", o, uv).reshape(b - a, H * vd))
    assert float((torch.cat(got) - want).abs().max()) < tol


def glu_case(device, dtype, tol):
    from githubrepostorag_amd.ops.elementwise import clamped_glu

    g = torch.Generator().manual_seed(10)
    gu = (3 * torch.randn(7, 2 * 36, generator=g)).to(dtype)
    want = O.silu(gu[:, :36].double()) * gu[:, 36:].double()
    got = clamped_glu(gu.to(device), None, 1.0, 0.0).double().cpu()
    assert float((got - want).abs().max()) < tol * 10


def test_mechanisms_alone():
    hyper_case("cpu", torch.float32, 1e-5)
    retention_case("cpu", torch.float32, 1e-4)
    window_case("cpu", torch.float32, 1e-5)
    latent_case("cpu", torch.float32, 1e-5)
    glu_case("cpu", torch.float32, 1e-6)
