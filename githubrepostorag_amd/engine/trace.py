"""Replay of a recorded token schedule through the engine (``python -m githubrepostorag_amd trace``, bin/trace_run).

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Each step is ONE engine batch (LLMEngine.feed): every entry's tokens continue that request from the cache and
state earlier steps left -- prompt portions beside single next tokens, requests that sit out steps, requests
that end and whose pages and slot are then used again.  Nothing is sampled.  For a step that wants logits the
runner writes ``<out>/<step>.f32`` (little-endian fp32 [wanted, vocab], in entry / want order), and after every
step it prints ``done <step>``.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np
import torch

SLOTS = 4  # live requests a replay may hold at once


def run_trace(model_dir: str, dtype: str, out_dir: str, max_tokens: int, device: str | None = None,
              block_size: int = 16, lines=None, log=None) -> int:
    from ..models import load_decoder
    from .llm_engine import EngineConfig, LLMEngine

    log = sys.stdout if log is None else log  # (looked up per call: the caller may have swapped the stream)
    dt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    dev = device or ("cuda" if torch.cuda.is_available() else "cpu")
    if dt == torch.float32:  # true fp32 products: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    model = load_decoder(model_dir, device=dev, dtype=dt)
    # the pool holds max_tokens tokens (every live request rounded up to whole pages) plus the scratch block
    nblocks = -(-max_tokens // block_size) + SLOTS + 1
    eng = LLMEngine(model, None, EngineConfig(max_num_seqs=SLOTS, max_model_len=max(max_tokens, block_size),
                                              max_num_batched_tokens=max(max_tokens, block_size),
                                              block_size=block_size, num_blocks=nblocks, use_cuda_graph=False,
                                              enable_prefix_caching=False))
    os.makedirs(out_dir, exist_ok=True)
    for line in (sys.stdin if lines is None else lines):
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or []) for e in st.get("entries", []) if e.get("tokens")]
        logits = eng.feed(entries, st.get("end") or [])
        if logits is not None:
            tmp = os.path.join(out_dir, f".{st['step']}.f32.tmp")
            np.ascontiguousarray(logits, dtype="<f4").tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{st['step']}.f32"))
        print(f"done {st['step']}", file=log, flush=True)
    return 0
