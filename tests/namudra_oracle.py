"""A plain float64 implementation of the Namudra decoder, one function per mechanism, written from the
design's equations with loops over tokens.  Slow on purpose; it shares no code with the engine.

Weights: a dict name -> tensor (any float dtype; used as float64).  Config: the config.json dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def rotate(vec, pos, dims, base):
    """Rotary position on the first ``dims`` entries of ``vec`` (1-D): entry i pairs with entry i + dims/2."""
    out = vec.clone()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = float(vec[i]), float(vec[i + half])
        out[i] = u * math.cos(a) - v * math.sin(a)
        out[i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def silu(z):
    return z * torch.sigmoid(z)


def retention(h, W, m, eps):
    """h [T, width] -> [T, width].  m: the layer's mixer dict; W(name) -> weight."""
    T = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    rd, base = m["rot"]["dims"], m["rot"]["base"]
    q = (h @ W("q").T).view(T, H, d)
    k = (h @ W("k").T).view(T, H, d)
    v = (h @ W("v").T).view(T, H, vd)
    gate = silu(h @ W("g").T)
    out = torch.zeros(T, H * vd, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, vd, dtype=F64)
        lam = float(m["decay"][hh])
        for t in range(T):
            qt = rotate(q[t, hh], t, rd, base)
            kt = rotate(k[t, hh], t, rd, base) * d ** -0.5
            S = lam * S + torch.outer(kt, v[t, hh])
            o = S.T @ qt
            out[t, hh * vd:(hh + 1) * vd] = rms_unit(o, eps)
    return (out * gate) @ W("o").T


def window_attention(h, W, m, eps):
    """Sliding-window attention with sigmoid weights, keys as values, q / k norms, a per-head bias and an
    output gate."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    assert m["vdim"] == d
    win, scale = m["mask"]["size"], m["scale"]
    q = (h @ W("q").T).view(T, H, d)
    k = (h @ W("k").T).view(T, G, d)
    v = k.clone()
    qn = norm_plain(q, W("q.norm"), eps)
    kn = norm_plain(k, W("k.norm"), eps)
    pb = W("pb")
    out = torch.zeros(T, H, d, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            for j in range(max(0, i - win + 1), i + 1):
                s = float(qn[i, hh] @ kn[j, g]) * scale + float(pb[hh])
                out[i, hh] += v[j, g] / (1.0 + math.exp(-s))
    gate = torch.sigmoid(h @ W("g").T)
    return (out.reshape(T, H * d) * gate) @ W("o").T


def latent_attention(h, W, m, eps):
    """Causal softmax attention whose keys and values are expanded from a cached latent; one rotated key part
    is shared by the heads."""
    T = h.shape[0]
    H, d, r, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, scale = m["rot"]["base"], m["scale"]
    assert m["rot"]["dims"] == r
    cq = norm_plain(h @ W("dq").T, W("dq.norm"), eps)
    q = (cq @ W("uq").T).view(T, H, d + r)
    ckv = h @ W("dkv").T
    c = norm_plain(ckv[:, :R], W("dkv.norm"), eps)
    kr = torch.stack([rotate(ckv[t, R:], t, r, base) for t in range(T)])
    kn = (c @ W("uk").T).view(T, H, d)
    v = (c @ W("uv").T).view(T, H, vd)
    out = torch.zeros(T, H, vd, dtype=F64)
    for hh in range(H):
        for i in range(T):
            qr = rotate(q[i, hh, d:], i, r, base)
            s = torch.tensor([float(q[i, hh, :d] @ kn[j, hh]) + float(qr @ kr[j]) for j in range(i + 1)], dtype=F64)
            p = torch.softmax(s * scale, 0)
            out[i, hh] = (p[:, None] * v[:i + 1, hh]).sum(0)
    return out.reshape(T, H * vd) @ W("o").T


def glu(h, W):
    return (silu(h @ W("gate").T) * (h @ W("up").T)) @ W("down").T


MIXERS = {"retention": retention, "attention": window_attention, "latent_attention": latent_attention}


def layer_runs(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = list(range(a))
    for _ in range(times if b > a else 0):
        runs += list(range(a, b))
    return runs + list(range(b, n))


def forward(cfg, weights, tokens, taps=None):
    """tokens [T] -> logits [T, vocab] float64.  ``taps``: a list that receives the sum of the streams after
    every layer run."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    S = int(cfg.get("streams", 1))
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    xs = [x0.clone() for _ in range(S)]
    for li in layer_runs(cfg):
        L = cfg["layers"][li]
        p = f"l{li}."
        subs = [(1, lambda u: MIXERS[L["type"]](u, lambda n: w[p + "mix." + n], L["mixer"], eps))]
        if L.get("mlp") is not None:
            assert L["mlp"]["kind"] == "dense"
            subs.append((2, lambda u: glu(u, lambda n: w[p + "mlp." + n])))
        for qi, fn in subs:
            if S > 1 or (p + f"hc{qi}.in") in w:
                cin, cout, mix = w[p + f"hc{qi}.in"], w[p + f"hc{qi}.out"], w[p + f"hc{qi}.mix"]
            else:
                cin, cout, mix = torch.ones(1, dtype=F64), torch.ones(1, dtype=F64), torch.ones(1, 1, dtype=F64)
            u = sum(cin[s] * xs[s] for s in range(S))
            y = fn(norm_one_plus(u, w[p + f"norm{qi}"], eps))
            xs = [sum(mix[s, t] * xs[s] for s in range(S)) + cout[t] * y for t in range(S)]
        if taps is not None:
            taps.append(sum(xs))
    x = sum(xs)
    return norm_one_plus(x, w["final.norm"], eps) @ w["head"].T


# ------------------------------------------------------------------------------------------------ test models
def make_config(width=48, vocab=96, streams=2, kinds=("retention", "attention", "latent_attention"), loop=(1, 3, 2),
                no_mlp=(0,), ff=40, eps=1e-5, ret=None, att=None, lat=None):
    """A small config.json dict.  ``ret`` / ``att`` / ``lat`` override the mixers' sizes."""
    r = dict(heads=2, dim=8, vdim=12, decay=[0.9, 0.99], rot={"dims": 4, "base": 100.0})
    a = dict(heads=4, kv_heads=2, dim=8, vdim=8, scale=0.4, mask={"size": 7})
    l = dict(heads=3, dim=8, rot_dim=4, vdim=10, kv_rank=16, q_rank=12, scale=0.3, rot={"dims": 4, "base": 50.0})
    r.update(ret or {})
    a.update(att or {})
    l.update(lat or {})
    if "rot_dim" in (lat or {}) and "rot" not in (lat or {}):
        l["rot"] = {"dims": l["rot_dim"], "base": 50.0}
    mix = {"retention": r, "attention": a, "latent_attention": l}
    layers = [{"type": k, "mixer": dict(mix[k]), "mlp": None if i in no_mlp else {"kind": "dense", "ff": ff}}
              for i, k in enumerate(kinds)]
    return {"architecture": "Namudra", "vocab": vocab, "width": width, "streams": streams, "norm": {"eps": eps},
            "layers": layers, "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}


def make_weights(cfg, seed=0, hc_tensors=True):
    """Random weights whose values are exact in bfloat16, under the checkpoint's tensor names."""
    g = torch.Generator().manual_seed(4242 + seed)
    W, S = cfg["width"], cfg["streams"]

    def r(*shape, s=None):
        s = shape[-1] ** -0.5 if s is None else s
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    sd = {"embed": r(cfg["vocab"], W, s=1.0), "head": r(cfg["vocab"], W), "final.norm": r(W, s=0.2)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for qi in (1, 2) if L["mlp"] is not None else (1,):
            sd[p + f"norm{qi}"] = r(W, s=0.2)
            if S > 1 or hc_tensors:
                sd[p + f"hc{qi}.in"] = (1.0 / S + r(S, s=0.2).float()).to(torch.bfloat16)
                sd[p + f"hc{qi}.out"] = (1.0 + r(S, s=0.3).float()).to(torch.bfloat16)
                sd[p + f"hc{qi}.mix"] = (torch.eye(S) + r(S, S, s=0.2).float()).to(torch.bfloat16)
        if L["type"] == "retention":
            H, d, vd = m["heads"], m["dim"], m["vdim"]
            sd.update({p + "mix.q": r(H * d, W), p + "mix.k": r(H * d, W), p + "mix.v": r(H * vd, W),
                       p + "mix.g": r(H * vd, W), p + "mix.o": r(W, H * vd)})
        elif L["type"] == "attention":
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            sd.update({p + "mix.q": r(H * d, W), p + "mix.k": r(G * d, W),
                       p + "mix.q.norm": (1.0 + r(d, s=0.2).float()).to(torch.bfloat16),
                       p + "mix.k.norm": (1.0 + r(d, s=0.2).float()).to(torch.bfloat16),
                       p + "mix.pb": (r(H, s=1.0).float() - 1.0).to(torch.bfloat16),
                       p + "mix.g": r(H * d, W), p + "mix.o": r(W, H * d)})
        else:
            H, d, rr, vd, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            sd.update({p + "mix.dq": r(Q, W), p + "mix.dq.norm": (1.0 + r(Q, s=0.2).float()).to(torch.bfloat16),
                       p + "mix.uq": r(H * (d + rr), Q), p + "mix.dkv": r(R + rr, W),
                       p + "mix.dkv.norm": (1.0 + r(R, s=0.2).float()).to(torch.bfloat16),
                       p + "mix.uk": r(H * d, R), p + "mix.uv": r(H * vd, R), p + "mix.o": r(W, H * vd)})
        if L["mlp"] is not None:
            F = L["mlp"]["ff"]
            sd.update({p + "mlp.gate": r(F, W), p + "mlp.up": r(F, W), p + "mlp.down": r(W, F)})
    return sd


def logits_and_taps(cfg, sd, toks):
    taps = []
    return forward(cfg, sd, toks, taps), torch.stack(taps)
