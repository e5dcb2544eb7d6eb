"""Scenarios that compare the engine serving a Zofesun model (kernels, paged cache, state slots, scheduler) with
the plain float64 oracle of zofesun_oracle.py.  Every scenario takes the device: the CPU tier runs the ops'
host paths, the GPU tier the HIP kernels, through the same engine code."""
from __future__ import annotations

import numpy as np
import torch

import zofesun_oracle as O


def build(cfg_dict, sd, device, dtype=torch.float32, slots=4, pool_tokens=512, block_size=16, graphs=False,
          max_batched=4096, mixed=False, window=1):
    from githubrepostorag_amd.engine.llm_engine import EngineConfig, LLMEngine
    from githubrepostorag_amd.models.configs import hybrid_config_from_dict
    from githubrepostorag_amd.models.zofesun import ZofesunModel

    model = ZofesunModel(hybrid_config_from_dict(cfg_dict), device=device, dtype=dtype, state_dict=sd)
    eng = LLMEngine(model, None, EngineConfig(max_num_seqs=slots, max_model_len=max(pool_tokens, 64),
                                              block_size=block_size, num_blocks=pool_tokens // block_size + 1,
                                              use_cuda_graph=graphs, max_num_batched_tokens=max_batched,
                                              mixed_batches=mixed, decode_window=window))
    return model, eng


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(1000 + seed)
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
    toks = tokens(cfg, 37, 0)
    want, taps = O.forward(cfg, sd, toks)
    model, eng = build(cfg, sd, device, dtype)
    got = feed_in_portions(eng, "a", toks, [len(toks)])
    assert rel_err(got, want) < tol
    # the residual stream after every layer run, through the model's own step (one sequence, fresh cache / state)
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


def case_prefill_vs_decode(device, tol, dtype=torch.float32, n=70, **cfg_kw):
    cfg = O.make_config(**cfg_kw)
    sd = O.make_weights(cfg, seed=5)
    toks = tokens(cfg, n, 1)
    want, _ = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "p", toks, [n]), want) < tol
    assert rel_err(feed_in_portions(eng, "d", toks, [1]), want) < tol           # every token on the decode path
    assert rel_err(feed_in_portions(eng, "pd", toks, [n - 20] + [1] * 20), want) < tol


def case_portions(device, tol, dtype=torch.float32):
    cfg = O.make_config(kinds=("mingru", "parallel", "parallel", "mingru"), loop=(0, 2, 3), no_mlp=(1,))
    sd = O.make_weights(cfg, seed=7)
    toks = tokens(cfg, 83, 2)
    want, _ = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    for k, cuts in enumerate(([2], [3, 2, 17, 1, 16, 31], [16], [15, 1, 1, 33], [64, 2])):
        assert rel_err(feed_in_portions(eng, f"c{k}", toks, cuts), want) < tol, cuts


def case_batches(device, tol, dtype=torch.float32):
    """Unequal requests in one batch -- portions beside single tokens, requests that sit out steps and end at
    different times -- give each request the logits it gets alone."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=9)
    lens = {"a": 45, "b": 9, "c": 31, "d": 18}
    toks = {k: tokens(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg, sd, t)[0] for k, t in toks.items()}
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
        want, _ = O.forward(cfg, sd, toks)
        cuts = [[n], [3, 1], [32, 1], [60, 2, 1, 1], [1]][i]
        assert rel_err(feed_in_portions(eng, f"r{i}", toks, cuts), want) < tol, i
        assert eng.kv.num_free == eng.kv.num_blocks - 1
    # a request that stops mid-way leaves nothing behind either
    eng.feed([("x", tokens(cfg, 40, 30), [])], [])
    eng.feed([], ["x"])
    toks = tokens(cfg, 21, 31)
    assert rel_err(feed_in_portions(eng, "y", toks, [20, 1]), O.forward(cfg, sd, toks)[0]) < tol


def case_long_decode(device, tol, dtype=torch.float32):
    cfg = O.make_config(kinds=("parallel", "mingru"), loop=(0, 2, 2), decay=(0.2, 0.9, 0.9995))
    sd = O.make_weights(cfg, seed=13)
    toks = tokens(cfg, 150, 3)
    want, _ = O.forward(cfg, sd, toks)
    _, eng = build(cfg, sd, device, dtype)
    assert rel_err(feed_in_portions(eng, "l", toks, [6] + [1] * 144), want) < tol


def case_other_sizes(device, tol, dtype=torch.float32):
    """Sizes where things the usual configs make equal differ, or are 1."""
    variants = [
        dict(width=40, vocab=33, heads=3, kv_heads=3, dim=10, vdim=6, rot_dims=10, lin_heads=1, lin_dim=5, lin_vdim=3,
             decay=(0.97,), gru_width=24, ff=24, kinds=("parallel",), loop=(0, 1, 2), left_scale=1.0, right_scale=0.25),
        dict(width=48, vocab=50, heads=6, kv_heads=1, dim=16, vdim=72, rot_dims=2, lin_heads=2, lin_dim=20, lin_vdim=70,
             decay=(1.0, 0.5), gru_width=80, ff=16, kinds=("mingru", "parallel"), loop=(0, 0, 1), limit=2.5),
        dict(kinds=("mingru",), loop=(0, 1, 3), no_mlp=(0,), gru_width=64),
        dict(rot_dims=0, kinds=("parallel", "parallel"), loop=(1, 2, 2), no_mlp=(0, 1)),
    ]
    for i, kw in enumerate(variants):
        cfg = O.make_config(**kw)
        sd = O.make_weights(cfg, seed=40 + i)
        toks = tokens(cfg, 29, 40 + i)
        want, _ = O.forward(cfg, sd, toks)
        _, eng = build(cfg, sd, device, dtype)
        assert rel_err(feed_in_portions(eng, "w", toks, [29]), want) < tol, i
        assert rel_err(feed_in_portions(eng, "c", toks, [5, 1, 2]), want) < tol, i


def case_first_tokens(device, tol, dtype=torch.float32):
    """Position 0 alone (one key beside the sink, a state that starts from zero in a used slot), then 1, 2."""
    cfg = O.make_config()
    sd = O.make_weights(cfg, seed=17)
    _, eng = build(cfg, sd, device, dtype, slots=1)
    eng.feed([("warm", tokens(cfg, 30, 50), [])], ["warm"])  # leave a state and pages behind
    for n in (1, 2, 3):
        toks = tokens(cfg, n, 60 + n)
        want, _ = O.forward(cfg, sd, toks)
        assert rel_err(feed_in_portions(eng, f"f{n}", toks, [1]), want) < tol
        assert rel_err(feed_in_portions(eng, f"g{n}", toks, [n]), want) < tol


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
        logits, _ = O.forward(cfg, sd, p + c.token_ids[:-1])
        for j, t in enumerate(c.token_ids):
            row = logits[len(p) - 1 + j]
            assert float(row.max() - row[t]) < tol * float(row.std()), (len(p), j)
    assert eng.kv.num_free == eng.kv.num_blocks - 1
