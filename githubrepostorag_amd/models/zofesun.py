"""Zofesun: a hybrid decoder on the paged-KV engine.

The layer list is data (models/configs.py HybridConfig): every layer has a sequence mixer and an optional
clamped-GLU feed-forward, both wrapped in Dynamic-Tanh norms before and after (x += post(sublayer(pre(x)))), over
an fp32 residual stream.  A span of layers may run several times with shared weights; every run of a layer has
its own K/V cache and recurrent state, and every pass but the first re-adds the embedding output before its
first layer, every pass adds its own step vector.

Mixers:
  "parallel"  two mixers on the same input, summed with fixed weights:
              left   causal softmax attention with a per-head sink logit, GQA, rotary on the first dims of each
                     head, values RMS-normed per head before they are cached      [grag_rope_vnorm_store,
                     grag_sink_attn_prefill / grag_sink_attn_decode]
              right  linear attention with a fixed decay per head and an fp32 [dim, vdim] state per head,
                     q / k / v through SiLU; heads RMS-normed together, gated by a sigmoid projection
                                                                                   [grag_decay_attn_scan,
                                                                                    grag_gated_rmsnorm]
  "mingru"    gates from the current token only: S = (1 - z) S + z c, output gated by SiLU [grag_mingru_scan]

Per layer the mixer's input projections are ONE GEMM (left q | k | v | right q | k | v | gate, or z | x | g), the
two output projections of a parallel mixer are one GEMM over [left_scale * left | right_scale * right], gate and
up are one GEMM.  Every sublayer boundary is one kernel: residual += post-norm(sublayer), next pre-norm out
[grag_dyt_residual].  Activations are bf16 (or fp32 end to end with dtype=torch.float32: the GEMMs then run in
true fp32); norms, scores, softmax, decays and states are fp32 in both.
"""
from __future__ import annotations

import math

import torch

from ..ops.attention import AttnMetadata, sink_attention
from ..ops.elementwise import clamped_glu, rope_table, rope_vnorm_store
from ..ops.linear import linear
from ..ops.norm import dyt_residual, embed_gather_f32
from ..ops.recurrent import decay_attention, gated_rmsnorm, mingru_scan
from ..parallel.comm import Group
from .configs import HybridConfig

GLU_SIGMOID_SLOPE = 1.702


class _Norm(tuple):
    """(alpha, w fp32 [H], b fp32 [H]) of a Dynamic-Tanh norm."""


class _HLayer:
    __slots__ = ("spec", "norm1", "norm1b", "norm2", "norm2b", "wp", "wo", "off", "sinks", "decay", "rnorm", "bz",
                 "bx", "wgu", "wd", "rope")


def init_state_dict(cfg: HybridConfig, seed: int = 0, std: float | None = None) -> dict:
    """Random weights under the checkpoint's tensor names (bf16; benches and tests -- not a trained model)."""
    g = torch.Generator().manual_seed(seed * 1000003 + 41)
    H = cfg.hidden_size

    def r(*shape, s=None):
        s = (1.0 / math.sqrt(shape[-1])) if s is None else s
        return (torch.randn(*shape, generator=g) * (std or s)).to(torch.bfloat16)

    def norm(sd, name):
        sd[name] = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
        sd[name + ".b"] = (0.02 * torch.randn(H, generator=g)).to(torch.bfloat16)
        sd[name + ".alpha"] = torch.tensor(0.5 + 0.5 * torch.rand((), generator=g).item(), dtype=torch.bfloat16)

    sd = {"embed": r(cfg.vocab_size, H, s=1.0), "head": r(cfg.vocab_size, H),
          "loop.step": r(cfg.loop_times, H, s=0.1)}
    norm(sd, "final.norm")
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            norm(sd, p + n)
        m = L.mixer
        if m.kind == "mingru":
            W = m.width
            sd.update({p + "mix.z": r(W, H), p + "mix.z.b": r(W, s=0.5), p + "mix.x": r(W, H),
                       p + "mix.x.b": r(W, s=0.5), p + "mix.g": r(W, H), p + "mix.o": r(H, W)})
        else:
            l, q = m.left, m.right
            sd.update({p + "mix.left.q": r(l.heads * l.dim, H), p + "mix.left.k": r(l.kv_heads * l.dim, H),
                       p + "mix.left.v": r(l.kv_heads * l.vdim, H), p + "mix.left.sink": r(l.heads, s=1.0),
                       p + "mix.left.o": r(H, l.heads * l.vdim),
                       p + "mix.right.q": r(q.heads * q.dim, H), p + "mix.right.k": r(q.heads * q.dim, H),
                       p + "mix.right.v": r(q.heads * q.vdim, H), p + "mix.right.g": r(q.heads * q.vdim, H),
                       p + "mix.right.o": r(H, q.heads * q.vdim),
                       p + "mix.right.norm": (1.0 + 0.1 * torch.randn(q.heads * q.vdim, generator=g)).to(torch.bfloat16)})
        if L.mlp is not None:
            F = L.mlp.ff
            sd.update({p + "mlp.gate": r(F, H), p + "mlp.up": r(F, H), p + "mlp.down": r(H, F)})
    return sd


class ZofesunModel:
    has_state = True  # recurrent state per sequence slot: the engine allocates it and never reuses cached prefixes

    def __init__(self, cfg: HybridConfig, device="cuda", dtype=torch.bfloat16, tp: Group | None = None,
                 seed: int = 0, state_dict: dict | None = None, init_std: float | None = None):
        assert cfg.arch == "zofesun", cfg.arch
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or Group([0])
        if not self.tp.trivial:
            raise NotImplementedError("the hybrid decoder runs on one GPU per replica (no tensor parallelism)")
        # the engine sizes the decode attention's split-KV scratch (hq * head_dim floats per row and split) and
        # picks its split plan (hkv) from these: the widest attention among the layers
        att = [L.mixer.left for L in cfg.layers if L.mixer.kind == "parallel"]
        self.hq = max([a.heads for a in att], default=1)
        self.hkv = min([a.kv_heads for a in att], default=1)
        self.head_dim = max([a.vdim for a in att], default=1)
        self.runs = cfg.layer_runs()
        self._tables: dict = {}
        self._max_pos = 0
        self._load(state_dict if state_dict is not None else init_state_dict(cfg, seed, init_std))
        self.prepare(4096)

    # ------------------------------------------------------------------ weights
    def _load(self, sd: dict):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        H = cfg.hidden_size

        def act(*names):  # GEMM operands: the activation dtype, fused along the output rows
            ts = [sd[n] for n in names]
            return (torch.cat(ts, 0) if len(ts) > 1 else ts[0]).to(device=dev, dtype=dt).contiguous()

        def f32(name):
            return sd[name].to(device=dev, dtype=torch.float32).contiguous()

        def norm(name):
            if tuple(sd[name].shape) != (H,):
                raise ValueError(f"{name}: expected [{H}], found {tuple(sd[name].shape)}")
            return _Norm((float(sd[name + ".alpha"].float()), f32(name), f32(name + ".b")))

        def expect(name, *shape):
            if tuple(sd[name].shape) != shape:
                raise ValueError(f"{name}: expected {list(shape)}, found {list(sd[name].shape)}")

        expect("embed", cfg.vocab_size, H)
        expect("head", cfg.vocab_size, H)
        self.embed = act("embed")
        # LM head rows padded to a multiple of 8: the sampler reads logit rows 8 at a time (zero rows, cut off
        # again in compute_logits)
        pad = -cfg.vocab_size % 8
        self.head = act("head") if not pad else torch.cat(
            [act("head"), torch.zeros(pad, H, dtype=dt, device=dev)], 0).contiguous()
        self.final_norm = norm("final.norm")
        self.loop_step = None
        if cfg.loop_stop > cfg.loop_start:
            expect("loop.step", cfg.loop_times, H)
            self.loop_step = f32("loop.step")
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p = f"l{i}."
            L = _HLayer()
            L.spec = spec
            L.norm1, L.norm1b = norm(p + "norm1"), norm(p + "norm1b")
            m = spec.mixer
            L.sinks = L.decay = L.rnorm = L.bz = L.bx = L.rope = None
            if m.kind == "mingru":
                W = m.width
                for n in ("z", "x", "g"):
                    expect(p + "mix." + n, W, H)
                expect(p + "mix.o", H, W)
                L.wp = act(p + "mix.z", p + "mix.x", p + "mix.g")
                L.off = (0, W, 2 * W)
                L.bz, L.bx = f32(p + "mix.z.b"), f32(p + "mix.x.b")
                L.wo = act(p + "mix.o")
            else:
                l, r = m.left, m.right
                expect(p + "mix.left.q", l.heads * l.dim, H)
                expect(p + "mix.left.k", l.kv_heads * l.dim, H)
                expect(p + "mix.left.v", l.kv_heads * l.vdim, H)
                expect(p + "mix.left.o", H, l.heads * l.vdim)
                expect(p + "mix.right.q", r.heads * r.dim, H)
                expect(p + "mix.right.k", r.heads * r.dim, H)
                expect(p + "mix.right.v", r.heads * r.vdim, H)
                expect(p + "mix.right.g", r.heads * r.vdim, H)
                expect(p + "mix.right.o", H, r.heads * r.vdim)
                names = [p + "mix.left." + n for n in "qkv"] + [p + "mix.right." + n for n in "qkvg"]
                L.wp = act(*names)
                offs, o = [], 0
                for n in names:
                    offs.append(o)
                    o += sd[n].shape[0]
                L.off = tuple(offs)
                L.wo = torch.cat([sd[p + "mix.left.o"], sd[p + "mix.right.o"]], 1).to(device=dev, dtype=dt).contiguous()
                L.sinks = f32(p + "mix.left.sink")
                L.decay = torch.tensor(r.decay, dtype=torch.float32, device=dev)
                L.rnorm = f32(p + "mix.right.norm")
                L.rope = (l.rot_dims, l.rot_base)
            L.norm2 = L.norm2b = L.wgu = L.wd = None
            if spec.mlp is not None:
                F = spec.mlp.ff
                expect(p + "mlp.gate", F, H)
                expect(p + "mlp.up", F, H)
                expect(p + "mlp.down", H, F)
                L.norm2, L.norm2b = norm(p + "norm2"), norm(p + "norm2b")
                L.wgu = act(p + "mlp.gate", p + "mlp.up")
                L.wd = act(p + "mlp.down")
            self.layers.append(L)

    def prepare(self, max_len: int) -> None:
        """Rotary tables for positions below ``max_len`` (the engine calls this with its max_model_len before any
        step or graph capture; the design itself has no position limit)."""
        if max_len <= self._max_pos:
            return
        self._max_pos = max_len
        self._tables = {}
        for L in self.layers:
            if L.rope is not None and L.rope not in self._tables:
                self._tables[L.rope] = rope_table(max_len, L.rope[0], L.rope[1], self.device)

    def param_bytes(self) -> int:
        n = 0
        for t in [self.embed, self.head] + [x for L in self.layers for x in (L.wp, L.wo, L.wgu, L.wd) if x is not None]:
            n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ cache and state
    def kv_bytes_per_block(self, block_size: int) -> int:
        n = 0
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            if m.kind == "parallel":
                n += m.left.kv_heads * block_size * (m.left.dim + m.left.vdim)
        return max(1, n) * torch.finfo(self.dtype).bits // 8

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One (K [blocks, G, BS, dim], V [blocks, G, BS, vdim]) pair per run of a parallel layer (None for
        runs without attention); a looped layer has one pair per pass."""
        caches = []
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            if m.kind != "parallel":
                caches.append(None)
                continue
            l = m.left
            caches.append((torch.zeros(num_blocks, l.kv_heads, block_size, l.dim, dtype=self.dtype, device=self.device),
                           torch.zeros(num_blocks, l.kv_heads, block_size, l.vdim, dtype=self.dtype,
                                       device=self.device)))
        return caches

    def state_bytes_per_slot(self) -> int:
        n = 0
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            n += m.width if m.kind == "mingru" else m.right.heads * m.right.dim * m.right.vdim
        return 4 * n

    def allocate_state(self, num_slots: int):
        """One fp32 state pool per layer run: [slots, heads, dim, vdim] (linear attention) or [slots, width]."""
        pools = []
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            shape = (num_slots, m.width) if m.kind == "mingru" else (num_slots, m.right.heads, m.right.dim,
                                                                     m.right.vdim)
            pools.append(torch.zeros(shape, dtype=torch.float32, device=self.device))
        return pools

    # ------------------------------------------------------------------ forward
    def _mixer(self, L, h, positions, meta: AttnMetadata, kv, state):
        m = L.spec.mixer
        p = linear(h, L.wp)
        if m.kind == "mingru":
            zo, xo, go = L.off
            return linear(mingru_scan(p, zo, xo, go, L.bz, L.bx, state, meta, m.width), L.wo)
        l, r = m.left, m.right
        lq, lk, lv, rq, rk, rv, rg = L.off
        kc, vc = kv
        q = rope_vnorm_store(p, lq, lk, lv, positions, self._tables[L.rope], meta.slot_mapping, kc, vc, l.heads,
                             l.kv_heads, l.dim, l.vdim, l.rot_dims, self.cfg.norm_eps)
        nl, nr = l.heads * l.vdim, r.heads * r.vdim
        both = torch.empty(h.shape[0], nl + nr, dtype=h.dtype, device=h.device)
        sink_attention(q, kc, vc, meta, l.scale, L.sinks, out=both[:, :nl], out_scale=m.left_scale)
        o = decay_attention(p, rq, rk, rv, L.decay, state, meta, r.heads, r.dim, r.vdim)
        gated_rmsnorm(o, L.rnorm, p, rg, self.cfg.norm_eps, both[:, nl:], out_scale=m.right_scale)
        return linear(both, L.wo)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta: AttnMetadata, kv_caches,
                state=None, taps: list | None = None) -> torch.Tensor:
        """-> final-normed hidden [T, H].  ``state``: the pools of allocate_state (meta.state_slots names each
        sequence's slot).  ``taps``: if a list, a copy of the residual stream after every layer run is appended."""
        if state is None or meta.state_slots is None:
            raise ValueError("this model carries recurrent state: pass state pools and meta.state_slots")
        dt = self.dtype
        x = embed_gather_f32(input_ids, self.embed)
        emb = x.clone() if self.cfg.loop_times > 1 and self.loop_step is not None else None
        y = post = None
        for ri, (li, t, first) in enumerate(self.runs):
            L = self.layers[li]
            if taps is not None and ri > 0:  # the boundary below folds the previous layer's last sublayer in
                dyt_residual(x, y, post, out_dtype=dt)
                y = post = None
                taps.append(x.clone())
            h = dyt_residual(x, y, post, emb if first and t > 0 else None, self.loop_step[t] if first else None,
                             pre=L.norm1, out_dtype=dt)
            y, post = self._mixer(L, h, positions, meta, kv_caches[ri], state[ri]), L.norm1b
            if L.wgu is not None:
                h = dyt_residual(x, y, post, pre=L.norm2, out_dtype=dt)
                y, post = linear(clamped_glu(linear(h, L.wgu), L.spec.mlp.limit, GLU_SIGMOID_SLOPE), L.wd), L.norm2b
        if taps is not None and self.runs:
            dyt_residual(x, y, post, out_dtype=dt)
            y = post = None
            taps.append(x.clone())
        return dyt_residual(x, y, post, pre=self.final_norm, out_dtype=dt)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [B, H] -> logits [B, vocab] (a view of the padded GEMM output)."""
        return linear(hidden, self.head)[:, : self.cfg.vocab_size]
