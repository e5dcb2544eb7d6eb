"""Namudra: a decoder with several residual streams and three gated sequence mixers, on the paged-KV engine.

The layer list is data (models/configs.py HybridConfig, arch "namudra"): every layer names one mixer and an optional
SiLU-gated feed-forward.  A span of layers may run several times with shared weights; every run of a layer has its
own K/V cache or recurrent state.  The residual is ``streams`` fp32 copies x_1 .. x_S (hyper-connections): a
sublayer reads u = sum_s in[s] x_s through an RMS norm whose weight is stored around zero (multiplier 1 + w), and
its output y updates all streams at once, x_t <- sum_s mix[s, t] x_s + out[t] y.  The model's output is the final
norm of the streams' sum.  One stream with unit coefficients is the ordinary pre-norm residual.

Mixers:
  "retention"         linear attention with a fixed decay per head and an fp32 [dim, vdim] state per head: rotary on
                      q and k, k scaled by dim^-1/2, no softmax and no denominator; every head's output is divided
                      by its RMS and gated by SiLU of a projection          [grag_decay_attn_scan, grag_gated_rmsnorm]
  "attention"         sliding-window attention whose weights are sigmoid(score + bias_h), not normalised over keys;
                      q and k RMS-normed per head, the values are the un-normed keys, the heads gated by the sigmoid
                      of a projection              [grag_qk_norm_store, grag_sigmoid_window_prefill / _decode]
  "latent_attention"  causal softmax attention over a cached latent plus one rotated key part shared by the heads.
                      The key and value expansions are folded into the query and output projections when the
                      weights are loaded (W_q' = W_uk^T W_uq per head, W_o' = W_o W_uv per head), so a step attends
                      straight to the cache: one kv head whose key rows are latent | rotated part and whose value
                      rows are the head of the same rows  [grag_rmsnorm_rows, grag_latent_store, grag_sink_attn_*
                                                           without sink]

Per layer the mixer's input projections are one GEMM (q | k | v | g, q | k | g, or dq | dkv), gate and up are one
GEMM, and every sublayer boundary is one kernel: streams update, next read-out, next norm [grag_hyper_mix].
Activations are bf16 (or fp32 end to end with dtype=torch.float32: the GEMMs then run in true fp32); streams,
norms, positions, scores, attention weights, decays and states are fp32 in both.
"""
from __future__ import annotations

import math

import torch

from ..ops.attention import AttnMetadata, sigmoid_window_attention, sink_attention
from ..ops.elementwise import clamped_glu, latent_store, qk_norm_store, rope_table
from ..ops.linear import linear
from ..ops.norm import embed_gather_f32, hyper_mix, rmsnorm_rows
from ..ops.recurrent import decay_attention, gated_rmsnorm
from ..parallel.comm import Group
from .configs import HybridConfig


class _Layer:
    __slots__ = ("spec", "kind", "norm1", "norm2", "hc1", "hc2", "wp", "off", "wo", "wq", "decay", "qn", "kn", "pb",
                 "dqn", "ckn", "rope", "wgu", "wd")


def init_state_dict(cfg: HybridConfig, seed: int = 0, std: float | None = None) -> dict:
    """Random weights under the checkpoint's tensor names (bf16; benches and tests -- not a trained model)."""
    g = torch.Generator().manual_seed(seed * 1000003 + 77)
    W, S = cfg.hidden_size, cfg.streams

    def r(*shape, s=None):
        s = (1.0 / math.sqrt(shape[-1])) if s is None else s
        return (torch.randn(*shape, generator=g) * (std or s)).to(torch.bfloat16)

    def around(v, n, s=0.1):
        return (v + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    sd = {"embed": r(cfg.vocab_size, W, s=1.0), "head": r(cfg.vocab_size, W), "final.norm": around(0.0, W)}
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        a, kind = L.mixer.spec, L.mixer.kind
        for qi in (1, 2) if L.mlp is not None else (1,):
            sd[p + f"norm{qi}"] = around(0.0, W)
            if S > 1:
                sd[p + f"hc{qi}.in"] = around(1.0 / S, S, 0.2)
                sd[p + f"hc{qi}.out"] = around(1.0, S, 0.3)
                sd[p + f"hc{qi}.mix"] = (torch.eye(S) + 0.15 * torch.randn(S, S, generator=g)).to(torch.bfloat16)
        if kind == "retention":
            sd.update({p + "mix.q": r(a.heads * a.dim, W), p + "mix.k": r(a.heads * a.dim, W),
                       p + "mix.v": r(a.heads * a.vdim, W), p + "mix.g": r(a.heads * a.vdim, W),
                       p + "mix.o": r(W, a.heads * a.vdim)})
        elif kind == "attention":
            sd.update({p + "mix.q": r(a.heads * a.dim, W), p + "mix.k": r(a.kv_heads * a.dim, W),
                       p + "mix.q.norm": around(1.0, a.dim), p + "mix.k.norm": around(1.0, a.dim),
                       p + "mix.pb": r(a.heads, s=1.0) - 2.0, p + "mix.g": r(a.heads * a.vdim, W),
                       p + "mix.o": r(W, a.heads * a.vdim)})
        else:
            sd.update({p + "mix.dq": r(a.q_rank, W), p + "mix.dq.norm": around(1.0, a.q_rank),
                       p + "mix.uq": r(a.heads * (a.dim + a.rot_dim), a.q_rank),
                       p + "mix.dkv": r(a.kv_rank + a.rot_dim, W), p + "mix.dkv.norm": around(1.0, a.kv_rank),
                       p + "mix.uk": r(a.heads * a.dim, a.kv_rank), p + "mix.uv": r(a.heads * a.vdim, a.kv_rank),
                       p + "mix.o": r(W, a.heads * a.vdim)})
        if L.mlp is not None:
            F = L.mlp.ff
            sd.update({p + "mlp.gate": r(F, W), p + "mlp.up": r(F, W), p + "mlp.down": r(W, F)})
    return sd


class NamudraModel:
    has_state = True  # recurrent state per sequence slot: the engine allocates it and never reuses cached prefixes

    def __init__(self, cfg: HybridConfig, device="cuda", dtype=torch.bfloat16, tp: Group | None = None,
                 seed: int = 0, state_dict: dict | None = None, init_std: float | None = None):
        assert cfg.arch == "namudra", cfg.arch
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or Group([0])
        if not self.tp.trivial:
            raise NotImplementedError("the Namudra decoder runs on one GPU per replica (no tensor parallelism)")
        # the engine sizes the decode attention's split-KV scratch (hq * head_dim floats per row and split) and
        # picks its split plan (hkv) from these: only the latent layers split their keys (one kv head, values of
        # kv_rank); the windowed layers read at most a window
        lat = [L.mixer.spec for L in cfg.layers if L.mixer.kind == "latent_attention"]
        self.hq = max([a.heads for a in lat], default=1)
        self.hkv = 1
        self.head_dim = max([a.kv_rank for a in lat], default=1)
        self.runs = cfg.layer_runs()
        self._tables: dict = {}
        self._max_pos = 0
        self._load(state_dict if state_dict is not None else init_state_dict(cfg, seed, init_std))
        self.prepare(4096)

    # ------------------------------------------------------------------ weights
    def _load(self, sd: dict):
        cfg, dev, dt = self.cfg, self.device, self.dtype
        W, S = cfg.hidden_size, cfg.streams

        def expect(name, *shape):
            if name not in sd:
                raise KeyError(f"the checkpoint has no tensor {name!r}")
            if tuple(sd[name].shape) != shape:
                raise ValueError(f"{name}: expected {list(shape)}, found {list(sd[name].shape)}")

        def act(*names):  # GEMM operands: the activation dtype, fused along the output rows
            ts = [sd[n] for n in names]
            return (torch.cat(ts, 0) if len(ts) > 1 else ts[0]).to(device=dev, dtype=dt).contiguous()

        def f32(name, *shape):
            expect(name, *shape)
            return sd[name].to(device=dev, dtype=torch.float32).contiguous()

        def one_plus(name):  # a norm weight stored around zero: the multiplier is 1 + w
            return (1.0 + f32(name, W)).contiguous()

        def hyper(p):  # (mix [S, S] (from, to), out [S], in [S]); one stream without tensors: the plain residual
            if S == 1 and (p + ".in") not in sd:
                one = torch.ones(1, dtype=torch.float32, device=dev)
                return one.view(1, 1), one, one
            return f32(p + ".mix", S, S), f32(p + ".out", S), f32(p + ".in", S)

        expect("embed", cfg.vocab_size, W)
        expect("head", cfg.vocab_size, W)
        self.embed = act("embed")
        # LM head rows padded to a multiple of 8: the sampler reads logit rows 8 at a time (zero rows, cut off
        # again in compute_logits)
        pad = -cfg.vocab_size % 8
        self.head = act("head") if not pad else torch.cat(
            [act("head"), torch.zeros(pad, W, dtype=dt, device=dev)], 0).contiguous()
        self.final_norm = one_plus("final.norm")
        self.ones = torch.ones(S, dtype=torch.float32, device=dev)
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p = f"l{i}."
            L = _Layer()
            for n in _Layer.__slots__:
                setattr(L, n, None)
            L.spec, L.kind = spec, spec.mixer.kind
            a = spec.mixer.spec
            L.norm1, L.hc1 = one_plus(p + "norm1"), hyper(p + "hc1")
            m = p + "mix."
            if L.kind == "retention":
                for n, rows in (("q", a.heads * a.dim), ("k", a.heads * a.dim), ("v", a.heads * a.vdim),
                                ("g", a.heads * a.vdim)):
                    expect(m + n, rows, W)
                expect(m + "o", W, a.heads * a.vdim)
                L.wp = act(m + "q", m + "k", m + "v", m + "g")
                L.off = (0, a.heads * a.dim, 2 * a.heads * a.dim, 2 * a.heads * a.dim + a.heads * a.vdim)
                L.wo = act(m + "o")
                L.decay = torch.tensor(a.decay, dtype=torch.float32, device=dev)
                L.rope = (a.rot_dims, a.rot_base) if a.rot_dims else None
            elif L.kind == "attention":
                expect(m + "q", a.heads * a.dim, W)
                expect(m + "k", a.kv_heads * a.dim, W)
                expect(m + "g", a.heads * a.vdim, W)
                expect(m + "o", W, a.heads * a.vdim)
                L.wp = act(m + "q", m + "k", m + "g")
                L.off = (0, a.heads * a.dim, (a.heads + a.kv_heads) * a.dim)
                L.wo = act(m + "o")
                L.qn, L.kn, L.pb = f32(m + "q.norm", a.dim), f32(m + "k.norm", a.dim), f32(m + "pb", a.heads)
            else:
                H, d, r, vd, R = a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank
                qr = a.q_rank or sd[m + "dq"].shape[0]
                expect(m + "dq", qr, W)
                expect(m + "uq", H * (d + r), qr)
                expect(m + "dkv", R + r, W)
                expect(m + "uk", H * d, R)
                expect(m + "uv", H * vd, R)
                expect(m + "o", W, H * vd)
                L.wp = act(m + "dq", m + "dkv")
                L.off = (0, qr)
                L.dqn, L.ckn = f32(m + "dq.norm", qr), f32(m + "dkv.norm", R)
                # absorbed form, folded once in float64: per head the query's unrotated part goes through W_uk^T
                # (scores against the latent itself), the rotated part is kept; the output projection takes the
                # attention-weighted latents through W_uv
                uq = sd[m + "uq"].double().view(H, d + r, qr)
                uk = sd[m + "uk"].double().view(H, d, R)
                uv = sd[m + "uv"].double().view(H, vd, R)
                wo = sd[m + "o"].double().view(W, H, vd)
                wq = torch.cat([torch.einsum("hdr,hdq->hrq", uk, uq[:, :d]), uq[:, d:]], 1)  # [H, R + r, qr]
                L.wq = wq.reshape(H * (R + r), qr).to(device=dev, dtype=dt).contiguous()
                L.wo = torch.einsum("whv,hvr->whr", wo, uv).reshape(W, H * R).to(device=dev, dtype=dt).contiguous()
                L.rope = (r, a.rot_base)
            if spec.mlp is not None:
                F = spec.mlp.ff
                expect(p + "mlp.gate", F, W)
                expect(p + "mlp.up", F, W)
                expect(p + "mlp.down", W, F)
                L.norm2, L.hc2 = one_plus(p + "norm2"), hyper(p + "hc2")
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
        for t in [self.embed, self.head] + [x for L in self.layers for x in (L.wp, L.wq, L.wo, L.wgu, L.wd)
                                            if x is not None]:
            n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ cache and state
    def _kv_row(self, li: int) -> int:
        """Numbers cached per token by a layer (0: no cache)."""
        m = self.cfg.layers[li].mixer
        if m.kind == "attention":
            return 2 * m.spec.kv_heads * m.spec.dim
        if m.kind == "latent_attention":
            return m.spec.kv_rank + m.spec.rot_dim
        return 0

    def kv_bytes_per_block(self, block_size: int) -> int:
        n = sum(self._kv_row(li) for li, _, _ in self.runs) * block_size
        return max(1, n) * torch.finfo(self.dtype).bits // 8

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One (K, V) pair per run of a layer with attention (None for retention runs); a looped layer has one pair
        per pass.  Windowed layers: normed keys [blocks, G, BS, dim] and keys as projected, the values, in a
        tensor of their own.  Latent layers: one tensor [blocks, 1, BS, kv_rank + rot_dim] (latent | rotated part);
        its values are the latents, so V is a view of the first kv_rank columns of the same rows."""
        caches = []
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            a = m.spec
            z = dict(dtype=self.dtype, device=self.device)
            if m.kind == "attention":
                caches.append((torch.zeros(num_blocks, a.kv_heads, block_size, a.dim, **z),
                               torch.zeros(num_blocks, a.kv_heads, block_size, a.dim, **z)))
            elif m.kind == "latent_attention":
                k = torch.zeros(num_blocks, 1, block_size, a.kv_rank + a.rot_dim, **z)
                caches.append((k, k[..., : a.kv_rank]))
            else:
                caches.append(None)
        return caches

    def state_bytes_per_slot(self) -> int:
        n = 0
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            if m.kind == "retention":
                n += m.spec.heads * m.spec.dim * m.spec.vdim
        return 4 * n

    def allocate_state(self, num_slots: int):
        """One fp32 state pool [slots, heads, dim, vdim] per run of a retention layer (None for the others)."""
        pools = []
        for li, _, _ in self.runs:
            m = self.cfg.layers[li].mixer
            pools.append(torch.zeros(num_slots, m.spec.heads, m.spec.dim, m.spec.vdim, dtype=torch.float32,
                                     device=self.device) if m.kind == "retention" else None)
        return pools

    # ------------------------------------------------------------------ forward
    def _mixer(self, L, h, positions, meta: AttnMetadata, kv, state):
        a, eps = L.spec.mixer.spec, self.cfg.norm_eps
        p = linear(h, L.wp)
        T = h.shape[0]
        if L.kind == "retention":
            qo, ko, vo, go = L.off
            o = decay_attention(p, qo, ko, vo, L.decay, state, meta, a.heads, a.dim, a.vdim, act=False,
                                positions=positions, rope=self._tables[L.rope] if L.rope else None,
                                k_scale=a.dim ** -0.5)
            y = torch.empty(T, a.heads * a.vdim, dtype=h.dtype, device=h.device)
            gated_rmsnorm(o, None, p, go, eps, y, groups=a.heads, gate="silu")
            return linear(y, L.wo)
        kc, vc = kv
        if L.kind == "attention":
            qo, ko, go = L.off
            q = qk_norm_store(p, qo, ko, L.qn, L.kn, meta.slot_mapping, kc, vc, a.heads, a.kv_heads, a.dim, eps)
            y = sigmoid_window_attention(q, kc, vc, meta, a.scale, L.pb, a.window,
                                         gate=p[:, go:go + a.heads * a.vdim])
            return linear(y, L.wo)
        qr = L.off[1]
        cq = rmsnorm_rows(p[:, :qr], L.dqn, eps)
        q = linear(cq, L.wq).view(T, a.heads, a.kv_rank + a.rot_dim)
        latent_store(p[:, qr:], L.ckn, positions, self._tables[L.rope], meta.slot_mapping, q, kc, eps)
        return linear(sink_attention(q, kc, vc, meta, a.scale, None), L.wo)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, meta: AttnMetadata, kv_caches,
                state=None, taps: list | None = None) -> torch.Tensor:
        """-> final-normed hidden [T, W].  ``state``: the pools of allocate_state (meta.state_slots names each
        sequence's slot).  ``taps``: if a list, the sum of the streams after every layer run is appended."""
        if state is None or meta.state_slots is None:
            raise ValueError("this model carries recurrent state: pass state pools and meta.state_slots")
        dt, eps, S = self.dtype, self.cfg.norm_eps, self.cfg.streams
        x0 = embed_gather_f32(input_ids, self.embed)
        xs = x0.unsqueeze(0).repeat(S, 1, 1).contiguous() if S > 1 else x0.unsqueeze(0)
        y = hc = None  # the pending sublayer output and its stream coefficients, applied at the next boundary
        for ri, (li, _, _) in enumerate(self.runs):
            L = self.layers[li]
            if taps is not None and ri > 0:  # the boundary below folds the previous layer's last sublayer in
                taps.append(hyper_mix(xs, y, hc[0], hc[1], self.ones, None, eps, dt, want_sum=True)[1])
                y = hc = None
            h, _ = hyper_mix(xs, y, hc and hc[0], hc and hc[1], L.hc1[2], L.norm1, eps, dt)
            y, hc = self._mixer(L, h, positions, meta, kv_caches[ri], state[ri]), L.hc1
            if L.wgu is not None:
                h, _ = hyper_mix(xs, y, hc[0], hc[1], L.hc2[2], L.norm2, eps, dt)
                y, hc = linear(clamped_glu(linear(h, L.wgu), None, 1.0, 0.0), L.wd), L.hc2
        if taps is not None and self.runs:
            taps.append(hyper_mix(xs, y, hc[0], hc[1], self.ones, None, eps, dt, want_sum=True)[1])
            y = hc = None
        return hyper_mix(xs, y, hc and hc[0], hc and hc[1], self.ones, self.final_norm, eps, dt)[0]

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """final-normed hidden [B, W] -> logits [B, vocab] (a view of the padded GEMM output)."""
        return linear(hidden, self.head)[:, : self.cfg.vocab_size]
