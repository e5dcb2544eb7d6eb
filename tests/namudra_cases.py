"""Scenarios that compare the engine serving a Namudra model (kernels, paged cache, state slots, scheduler) with
the plain float64 oracle of namudra_oracle.py.  Every scenario takes the device: the CPU tier runs the ops' host
paths, the GPU tier the HIP kernels, through the same engine code."""
from __future__ import annotations

import numpy as np
import torch

import namudra_oracle as O


def build(cfg_dict, sd, device, dtype=torch.float32, slots=4, pool_tokens=512, block_size=16, graphs=False,
          max_batched=4096, mixed=False, window=1):
    from githubrepostorag_amd.engine.llm_engine import EngineConfig, LLMEngine
    from githubrepostorag_amd.models import build_decoder
    from githubrepostorag_amd.models.configs import namudra_config_from_dict

    model = build_decoder(namudra_config_from_dict(cfg_dict), device=device, dtype=dtype, state_dict=sd)
    eng = LLMEngine(model, None, EngineConfig(max_num_seqs=slots, max_model_len=max(pool_tokens, 64),
                                              block_size=block_size, num_blocks=pool_tokens // block_size + 1,
                                              use_cuda_graph=graphs, max_num_batched_tokens=max_batched,
                                              mixed_batches=mixed, decode_window=window))
    return model, eng


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(7000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def rel_err(got, want):
    """Mean-free RMS difference over the vocabulary, relative to the logits' own spread (per row, the worst)."""
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
    toks = tokens(cfg, 33, 0)
    want, taps = O.logits_and_taps(cfg, sd, toks)
    model, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "a", toks, [len(toks)]), want) < tol
    # the streams' sum after every layer run, through the model's own step (one sequence, fresh cache / state)
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


def case_single_mixer(device, tol, kind, dtype=torch.float32, **kw):
    """One layer of one mixer, one stream, no feed-forward: the mechanism alone between embedding and head."""
    cfg = O.make_config(kinds=(kind,), loop=(0, 0, 1), no_mlp=(0,), streams=1, **kw)
    sd = O.make_weights(cfg, seed=21, hc_tensors=False)
    toks = tokens(cfg, 41, 5)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "w", toks, [41]), want) < tol
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
    assert rel_err(feed_in_portions(eng, "pd", toks, [n - 20] + [1] * 20), want) < tol  # the window passes over decoded tokens


def case_portions(device, tol, dtype=torch.float32):
    """Portions cut inside pages (16), windows (7) and scan chunks (64), down to two tokens."""
    cfg = O.make_config(kinds=("retention", "attention", "latent_attention", "retention"), loop=(0, 2, 3), no_mlp=(1,))
    sd = O.make_weights(cfg, seed=7)
    toks = tokens(cfg, 139, 2)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    for k, cuts in enumerate(([2], [3, 2, 17, 1, 16, 31], [16], [15, 1, 1, 33], [64, 2], [65, 63, 11], [130, 9])):
        assert rel_err(feed_in_portions(eng, f"c{k}", toks, cuts), want) < tol, cuts


def case_batches(device, tol, dtype=torch.float32):
    """Unequal requests in one batch -- portions beside single tokens, requests that sit out steps and end at
    different times -- give each request the logits it gets alone."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=9)
    lens = {"a": 45, "b": 9, "c": 31, "d": 18}
    toks = {k: tokens(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg, sd, t) for k, t in toks.items()}
    _, eng = build(cfg, sd, device, dtype, pool_tokens=192)
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
    """Pages and state slots that were freed are used again: with one slot and a pool of two requests' worth,
    later requests land on the earlier ones' pages and state and still match their own oracle."""
    cfg = O.make_config(loop=(0, 0, 1))
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
    cfg = O.make_config(kinds=("retention", "latent_attention", "attention"), loop=(0, 2, 2),
                        ret=dict(heads=3, decay=[0.2, 0.9, 0.9995]), att=dict(mask={"size": 33}))
    sd = O.make_weights(cfg, seed=13)
    toks = tokens(cfg, 150, 3)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "l", toks, [6] + [1] * 144), want) < tol


def case_other_sizes(device, tol, dtype=torch.float32):
    """Sizes where things the usual configs make equal differ, or are 1."""
    variants = [
        # one stream that still has its coefficients; one kv head; one retention head with dim > vdim, whole-head rotary
        (dict(width=40, vocab=33, streams=1, kinds=("retention", "attention"), loop=(0, 2, 2), no_mlp=(),
              ret=dict(heads=1, dim=10, vdim=6, decay=[0.97], rot={"dims": 10, "base": 7.0}),
              att=dict(heads=3, kv_heads=1, dim=10, vdim=10, scale=1.0, mask={"size": 1})), True),
        # one stream, plain residual (no coefficient tensors); heads == kv heads; window longer than the prompt
        (dict(width=48, vocab=50, streams=1, kinds=("attention", "latent_attention"), loop=(0, 0, 1), no_mlp=(0, 1),
              att=dict(heads=2, kv_heads=2, dim=72, vdim=72, scale=0.1, mask={"size": 500}),
              lat=dict(heads=1, dim=6, rot_dim=2, vdim=20, kv_rank=80, q_rank=7, scale=0.5)), False),
        # four streams; decay 1 (nothing forgotten) and a fast one; value size above 64; the loop is the whole stack
        (dict(width=56, vocab=64, streams=4, kinds=("latent_attention", "retention"), loop=(0, 2, 3), no_mlp=(1,),
              ret=dict(heads=2, dim=20, vdim=70, decay=[1.0, 0.5], rot={"dims": 2, "base": 10000.0}),
              lat=dict(heads=5, dim=4, rot_dim=12, vdim=4, kv_rank=8, q_rank=24, scale=0.7)), True),
        # three streams, a loop that runs once, a window of two
        (dict(streams=3, loop=(1, 2, 1), att=dict(mask={"size": 2})), True),
        # a latent wider than the matrix-core kernels' rows (value row above 256)
        (dict(kinds=("latent_attention",), loop=(0, 0, 1), no_mlp=(),
              lat=dict(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=320, q_rank=16, scale=0.2)), True),
    ]
    for i, (kw, hc) in enumerate(variants):
        cfg = O.make_config(**kw)
        sd = O.make_weights(cfg, seed=40 + i, hc_tensors=hc)
        toks = tokens(cfg, 29, 40 + i)
        want = O.forward(cfg, sd, toks)
        _, eng = build(cfg, sd, device, dtype)
        assert rel_err(feed_in_portions(eng, "w", toks, [29]), want) < tol, i
        assert rel_err(feed_in_portions(eng, "c", toks, [5, 1, 2]), want) < tol, i


def case_inferred_rank(device, tol):
    """A config without q_rank: the query latent's size comes from the weight."""
    cfg = O.make_config(kinds=("latent_attention",), loop=(0, 0, 1), no_mlp=())
    sd = O.make_weights(cfg, seed=23)
    del cfg["layers"][0]["mixer"]["q_rank"]
    toks = tokens(cfg, 19, 9)
    _, eng = build(cfg, sd, device)
    assert rel_err(feed_in_portions(eng, "w", toks, [19]), O.forward(cfg, sd, toks)) < tol


def case_first_tokens(device, tol, dtype=torch.float32):
    """Position 0 alone (one key, a state that starts from zero in a used slot), then 1, 2."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=17)
    _, eng = build(cfg, sd, device, dtype, slots=1)
    eng.feed([("warm", tokens(cfg, 30, 50), [])], ["warm"])  # leave a state and pages behind
    for n in (1, 2, 3):
        toks = tokens(cfg, n, 60 + n)
        want = O.forward(cfg, sd, toks)
        assert rel_err(feed_in_portions(eng, f"f{n}", toks, [1]), want) < tol
        assert rel_err(feed_in_portions(eng, f"g{n}", toks, [n]), want) < tol


def case_sharp_far_keys(device, tol, dtype=torch.float32):
    """A softmax scale large enough that every query of the latent layer picks out single keys, many of them far
    back and across page borders: a key read from the wrong place changes the logits outright.  300 tokens,
    the last 40 decoded one by one, portions cut off the page grid."""
    cfg = O.make_config(kinds=("latent_attention",), loop=(0, 1, 2), no_mlp=(), lat=dict(scale=6.0))
    sd = O.make_weights(cfg, seed=29)
    toks = tokens(cfg, 300, 6)
    want = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "s", toks, [300]), want) < tol
    assert rel_err(feed_in_portions(eng, "t", toks, [97, 130, 33] + [1] * 40), want) < tol


def case_window_edges(device, tol, dtype=torch.float32, bs=16):
    """The windowed attention op alone on crafted keys: key j is the unit vector e_j, so a query 90 e_p scores 90
    on position p and 0 elsewhere; with a bias of -30 the weight is ~1 there and ~1e-13 on every other key.  Head 0
    asks for the key just inside the window (distance window - 1), head 1 for the key just outside it (distance
    window): the output must hold the inside key's value and nothing of the outside one -- in a prompt's portion
    that follows cached context and for a decoded token; windows that end on, before and after a page border,
    pages out of order."""
    from githubrepostorag_amd.ops.attention import AttnMetadata, sigmoid_window_attention

    dev = torch.device(device)
    H, G, ctx = 2, 1, 75
    d = 80
    for win in (1, 5, bs, bs + 1, 2 * bs - 1, 40):
        nb = -(-ctx // bs)
        g = torch.Generator().manual_seed(win)
        perm = (torch.randperm(nb, generator=g) + 1).to(torch.int32)
        kc = torch.zeros(nb + 1, G, bs, d, dtype=dtype, device=dev)
        vc = torch.zeros(nb + 1, G, bs, d, dtype=dtype, device=dev)
        V = torch.randn(ctx, d, generator=g).to(torch.bfloat16).float()
        for j in range(ctx):
            kc[perm[j // bs], 0, j % bs, j] = 1.0
            vc[perm[j // bs], 0, j % bs] = V[j].to(dtype)
        for qlen in (33, 9, 1):  # (33 queries in bf16: the matrix-core kernel)
            want = torch.zeros(qlen, H, d, dtype=torch.float64)
            q = torch.zeros(qlen, H, d)
            for n, p in enumerate(range(ctx - qlen, ctx)):
                for h, tgt in enumerate((p - win + 1, p - win)):  # head 0: inside edge, head 1: outside
                    if tgt >= 0:
                        q[n, h, tgt] = 90.0
                        if h == 0:
                            want[n, h] = V[tgt].double()
            i32 = dict(dtype=torch.int32, device=dev)
            meta = AttnMetadata(q_start=torch.tensor([0, qlen], **i32), ctx_len=torch.tensor([ctx], **i32),
                                block_tables=perm.view(1, nb).to(dev), slot_mapping=torch.zeros(qlen, **i32),
                                max_q_len=qlen, num_seqs=1, num_tokens=qlen, is_decode=qlen == 1)
            got = sigmoid_window_attention(q.to(dtype).to(dev), kc, vc, meta, 1.0,
                                           torch.full((H,), -30.0, device=dev), win).float().cpu().view(qlen, H, d)
            assert float((got.double() - want).abs().max()) < tol, (win, qlen)


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
    outs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    for p, c in zip(prompts, outs):
        assert len(c.token_ids) == 10
        logits = O.forward(cfg, sd, p + c.token_ids[:-1])
        for j, t in enumerate(c.token_ids):
            row = logits[len(p) - 1 + j]
            assert float(row.max() - row[t]) < tol * float(row.std()), (len(p), j)
    assert eng.kv.num_free == eng.kv.num_blocks - 1
