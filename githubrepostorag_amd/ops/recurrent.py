"""Recurrent sequence mixers with a carried fp32 state per sequence (HIP on device tensors, plain fp32 loops on
CPU): linear attention with a fixed per-head decay, and the minGRU gated recurrence.

State lives in slot-indexed pools ([slots, ...] fp32) owned by the engine; ``meta.state_slots`` [nseq] names each
sequence's slot.  A sequence whose first token of the step is position 0 starts from a zero state (so a freed
slot needs no reset when it is used again); otherwise the step continues from the slot's state and leaves the
state after its last token there.  Tokens are consumed in order, so a prompt may be cut into steps anywhere.
"""
from __future__ import annotations

import torch

from ._lib import call, lib, ptr
from .attention import AttnMetadata


def _chunk_ws(kind: str, m: AttnMetadata, per_chunk: int, device) -> torch.Tensor | None:
    """fp32 scratch for the chunk-parallel passes of a long portion ([sequences * chunks, per_chunk]); None when
    every portion of the step fits one chunk (decode rows, short portions): the one-pass kernels take those."""
    chunk = getattr(lib(), "grag_decay_attn_chunk" if kind == "decay" else "grag_mingru_chunk")()
    if m.max_q_len <= chunk:
        return None
    return torch.empty(m.num_seqs * -(-m.max_q_len // chunk) * per_chunk, dtype=torch.float32, device=device)


def _dt(t: torch.Tensor) -> int:
    return 0 if t.dtype == torch.bfloat16 else 1


def _parts(meta: AttnMetadata):
    """(meta, first row, end row) of a step's parts: prefill chunks, then the decode rows of a mixed step."""
    dec = meta.extra.get("decode_rows")
    if dec is None:
        return [(meta, 0, meta.num_tokens)]
    Tp, dmeta = dec
    return [(meta, 0, Tp), (dmeta, Tp, Tp + dmeta.num_tokens)]


def decay_attention(proj: torch.Tensor, qoff: int, koff: int, voff: int, decay: torch.Tensor, state: torch.Tensor,
                    meta: AttnMetadata, H: int, d: int, vd: int, act: bool = True, positions: torch.Tensor | None = None,
                    rope: torch.Tensor | None = None, k_scale: float = 1.0) -> torch.Tensor:
    """Linear attention with decay.  From the fused projection ``proj`` [T, ld]: q, k = columns qoff / koff (H x d),
    v = columns voff (H x vd), each through SiLU when ``act``.  With ``rope`` (a rope_table [positions, rd]) the
    first rd dims of q and k are rotated by ``positions`` (dim i paired with i + rd/2) in fp32 inside the scan, and
    k is multiplied by ``k_scale`` after the rotation.  Per head S_t = decay_h S_(t-1) + k_t v_t^T (state
    [slots, H, d, vd] fp32), o_t = S_t^T q_t.  Returns o [T, H*vd] fp32."""
    T = proj.shape[0]
    out = torch.empty(T, H * vd, dtype=torch.float32, device=proj.device)
    rd = 0 if rope is None else rope.shape[1]
    if rd and (positions is None or positions.dtype != torch.int32 or rope.dtype != torch.float32 or rd > d or rd % 2):
        raise ValueError("rotary needs int32 positions and an fp32 table of an even width <= the head size")
    for m, r0, r1 in _parts(meta):
        if r1 <= r0:
            continue
        pos = positions[r0:r1] if rd else None
        if not proj.is_cuda:
            _decay_attention_cpu(proj[r0:r1], qoff, koff, voff, decay, state, m, H, d, vd, out[r0:r1], act, pos, rope,
                                 k_scale)
            continue
        assert proj.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous()
        x = proj[r0:r1]
        ws = _chunk_ws("decay", m, H * d * vd, proj.device)
        call("grag_decay_attn_scan", ptr(x), proj.stride(0), qoff, koff, voff, ptr(decay), ptr(state),
             ptr(m.state_slots), ptr(m.q_start), ptr(m.ctx_len), ptr(out[r0:r1]), m.num_seqs, H, d, vd,
             state.shape[0], _dt(proj), ptr(ws), m.max_q_len, 1 if act else 0, ptr(pos), ptr(rope), rd,
             rope.shape[0] if rd else 0, float(k_scale))
    return out


def _decay_attention_cpu(x, qoff, koff, voff, decay, state, m, H, d, vd, out, act=True, pos=None, rope=None,
                         k_scale=1.0):
    F = torch.nn.functional
    qs, cl, sl = m.q_start.tolist(), m.ctx_len.tolist(), m.state_slots.tolist()
    x = x.float()
    f = F.silu if act else (lambda t: t)
    for s in range(m.num_seqs):
        a, b = qs[s], qs[s + 1]
        if b <= a:
            continue
        S = torch.zeros(H, d, vd) if cl[s] - (b - a) == 0 else state[sl[s]].clone()
        q = f(x[a:b, qoff:qoff + H * d]).view(-1, H, d).clone()
        k = f(x[a:b, koff:koff + H * d]).view(-1, H, d).clone()
        v = f(x[a:b, voff:voff + H * vd]).view(-1, H, vd)
        if rope is not None:
            rd = rope.shape[1]
            h2 = rd // 2
            cs = rope[pos[a:b].long()]
            c, sn = cs[:, None, :h2], cs[:, None, h2:]
            for t in (q, k):
                u, w = t[..., :h2].clone(), t[..., h2:rd].clone()
                t[..., :h2] = u * c - w * sn
                t[..., h2:rd] = w * c + u * sn
        k = k * k_scale
        lam = decay.float().view(H, 1, 1)
        for t in range(b - a):
            S = lam * S + k[t, :, :, None] * v[t, :, None, :]
            out[a + t] = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1)
        state[sl[s]] = S


def gated_rmsnorm(x: torch.Tensor, w: torch.Tensor | None, proj: torch.Tensor, goff: int, eps: float,
                  out: torch.Tensor, out_scale: float = 1.0, groups: int = 1, gate: str = "sigmoid") -> torch.Tensor:
    """out = out_scale * x / rms(x) * w * gate(g): x [T, N] fp32 normalised over each of ``groups`` equal column
    groups (1: the whole row; the head count: per head), ``w`` [N] optional, g read from columns goff.. of the
    fused projection, gate "sigmoid" or "silu"; ``out`` [T, N] may be a column slice of a wider buffer."""
    T, N = x.shape
    if gate not in ("sigmoid", "silu") or N % groups:
        raise ValueError("gate is 'sigmoid' or 'silu', and the groups divide the row")
    if not x.is_cuda:
        g = proj[:, goff:goff + N].float()
        g = torch.sigmoid(g) if gate == "sigmoid" else torch.nn.functional.silu(g)
        xg = x.view(T, groups, N // groups)
        y = (xg / torch.sqrt(xg.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, N)
        out.copy_(y * (1.0 if w is None else w.float()) * g * out_scale)
        return out
    assert x.is_contiguous() and out.stride(1) == 1 and out.dtype == proj.dtype
    call("grag_gated_rmsnorm", ptr(x), ptr(w), ptr(proj), proj.stride(0), goff, ptr(out), out.stride(0), T, N,
         float(eps), float(out_scale), _dt(proj), groups, 1 if gate == "silu" else 0)
    return out


def mingru_scan(proj: torch.Tensor, zoff: int, xoff: int, goff: int, bz: torch.Tensor, bx: torch.Tensor,
                state: torch.Tensor, meta: AttnMetadata, W: int) -> torch.Tensor:
    """minGRU over a step's tokens.  From the fused projection [T, ld]: z = sigmoid(columns zoff + bz),
    u = columns xoff + bx, candidate = u + 1/2 where u >= 0 else sigmoid(u);
    S_t = (1 - z) S_(t-1) + z candidate (state [slots, W] fp32); returns S_t * silu(columns goff) [T, W]."""
    T = proj.shape[0]
    out = torch.empty(T, W, dtype=proj.dtype, device=proj.device)
    for m, r0, r1 in _parts(meta):
        if r1 <= r0:
            continue
        if not proj.is_cuda:
            _mingru_cpu(proj[r0:r1].float(), zoff, xoff, goff, bz, bx, state, m, W, out[r0:r1])
            continue
        assert proj.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous()
        ws = _chunk_ws("mingru", m, 2 * W, proj.device)
        call("grag_mingru_scan", ptr(proj[r0:r1]), proj.stride(0), zoff, xoff, goff, ptr(bz), ptr(bx), ptr(state),
             ptr(m.state_slots), ptr(m.q_start), ptr(m.ctx_len), ptr(out[r0:r1]), m.num_seqs, W, state.shape[0],
             _dt(proj), ptr(ws), m.max_q_len)
    return out


def _mingru_cpu(x, zoff, xoff, goff, bz, bx, state, m, W, out):
    qs, cl, sl = m.q_start.tolist(), m.ctx_len.tolist(), m.state_slots.tolist()
    z = torch.sigmoid(x[:, zoff:zoff + W] + bz.float())
    u = x[:, xoff:xoff + W] + bx.float()
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = torch.nn.functional.silu(x[:, goff:goff + W])
    for s in range(m.num_seqs):
        a, b = qs[s], qs[s + 1]
        if b <= a:
            continue
        S = torch.zeros(W) if cl[s] - (b - a) == 0 else state[sl[s]].clone()
        for t in range(a, b):
            S = (1.0 - z[t]) * S + z[t] * c[t]
            out[t] = (S * g[t]).to(out.dtype)
        state[sl[s]] = S
