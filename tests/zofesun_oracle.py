"""A plain, slow float64 implementation of the Zofesun design, one function per mechanism, written from the
design's equations with explicit loops.  It shares no code with the package: the tests compare the engine
(kernels, paged cache, state slots, scheduler) against it.

Notation: T tokens, positions 0..T-1 of ONE sequence; weights are [out, in] and applied as W x; ``sd`` maps the
checkpoint's tensor names to tensors; ``cfg`` is the config.json dictionary.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def dyt(x, alpha, w, b):
    """Dynamic Tanh: every element on its own, no statistics."""
    return torch.tanh(float(alpha) * x) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rotate(x, rot_dims, base):
    """x [T, heads, dim]: within the first rot_dims dims, dim i and dim i + rot_dims/2 form a pair turned by the
    angle position * base^(-2i/rot_dims); the other dims pass."""
    T, _, _ = x.shape
    out = x.clone()
    half = rot_dims // 2
    for p in range(T):
        for i in range(half):
            ang = p * base ** (-2.0 * i / rot_dims)
            c, s = math.cos(ang), math.sin(ang)
            u, v = x[p, :, i], x[p, :, i + half]
            out[p, :, i] = u * c - v * s
            out[p, :, i + half] = v * c + u * s
    return out


def sink_attention(q, k, v, scale, sinks):
    """q [T, H, d], k [T, G, d], v [T, G, vd] -> [T, H, vd].  Query head h reads kv head h // (H/G); token t sees
    tokens 0..t; the softmax denominator holds one extra term exp(sinks[h]) with no value."""
    T, H, _ = q.shape
    G, vd = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, vd, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for t in range(T):
            sc = (k[: t + 1, g] @ q[t, h]) * scale
            m = max(float(sc.max()), float(sinks[h]))
            e = torch.exp(sc - m)
            den = e.sum() + math.exp(float(sinks[h]) - m)
            out[t, h] = (e / den) @ v[: t + 1, g]
    return out


def decay_attention(q, k, v, decay):
    """q, k [T, H, d], v [T, H, vd]: S <- decay_h S + k_t v_t^T, o_t = S^T q_t."""
    T, H, d = q.shape
    vd = v.shape[2]
    out = torch.zeros(T, H, vd, dtype=F64)
    for h in range(H):
        S = torch.zeros(d, vd, dtype=F64)
        for t in range(T):
            S = decay[h] * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


def mingru(z_pre, u_pre):
    """Pre-activations [T, W] -> states [T, W]: z = sigmoid, candidate = u + 1/2 (u >= 0) or sigmoid(u) (u < 0)."""
    T, W = z_pre.shape
    S = torch.zeros(W, dtype=F64)
    out = torch.zeros(T, W, dtype=F64)
    for t in range(T):
        z = torch.sigmoid(z_pre[t])
        u = u_pre[t]
        cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        S = (1 - z) * S + z * cand
        out[t] = S
    return out


def clamped_glu(gate, up, limit):
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1)


def silu(x):
    return x * torch.sigmoid(x)


def mixer_parallel(h, sd, p, m, eps):
    l, r = m["left"], m["right"]
    T = h.shape[0]
    W = lambda n: sd[p + n].to(F64)
    q = (h @ W("left.q").T).view(T, l["heads"], l["dim"])
    k = (h @ W("left.k").T).view(T, l["kv_heads"], l["dim"])
    v = (h @ W("left.v").T).view(T, l["kv_heads"], l["vdim"])
    q = rotate(q, l["rot"]["dims"], l["rot"]["base"])
    k = rotate(k, l["rot"]["dims"], l["rot"]["base"])
    v = unit_rms(v, eps)
    left = sink_attention(q, k, v, l["scale"], W("left.sink")).reshape(T, -1) @ W("left.o").T
    rq = silu(h @ W("right.q").T).view(T, r["heads"], r["dim"])
    rk = silu(h @ W("right.k").T).view(T, r["heads"], r["dim"])
    rv = silu(h @ W("right.v").T).view(T, r["heads"], r["vdim"])
    o = decay_attention(rq, rk, rv, r["decay"]).reshape(T, -1)
    o = unit_rms(o, eps) * W("right.norm") * torch.sigmoid(h @ W("right.g").T)
    right = o @ W("right.o").T
    return m["left_scale"] * left + m["right_scale"] * right


def mixer_mingru(h, sd, p):
    W = lambda n: sd[p + n].to(F64)
    S = mingru(h @ W("z").T + W("z.b"), h @ W("x").T + W("x.b"))
    return (S * silu(h @ W("g").T)) @ W("o").T


def forward(cfg, sd, tokens):
    """-> (logits [T, vocab], residual stream after every layer run [runs, T, width])."""
    eps = cfg["norm"]["eps"]
    N = lambda x, n: dyt(x, sd[n + ".alpha"].to(F64), sd[n].to(F64), sd[n + ".b"].to(F64))
    x = sd["embed"].to(F64)[torch.tensor(tokens)]
    e0 = x.clone()
    taps = []

    def layer(x, i):
        L, p = cfg["layers"][i], f"l{i}."
        h = N(x, p + "norm1")
        y = mixer_mingru(h, sd, p + "mix.") if L["type"] == "mingru" else mixer_parallel(h, sd, p + "mix.", L["mixer"], eps)
        x = x + N(y, p + "norm1b")
        if L["mlp"] is not None:
            h = N(x, p + "norm2")
            y = clamped_glu(h @ sd[p + "mlp.gate"].to(F64).T, h @ sd[p + "mlp.up"].to(F64).T, L["mlp"]["limit"])
            x = x + N(y @ sd[p + "mlp.down"].to(F64).T, p + "norm2b")
        taps.append(x.clone())
        return x

    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    for i in range(lp["start"]):
        x = layer(x, i)
    if lp["stop"] > lp["start"]:
        for t in range(lp["times"]):
            if t > 0:
                x = x + e0
            x = x + sd["loop.step"].to(F64)[t]
            for i in range(lp["start"], lp["stop"]):
                x = layer(x, i)
    for i in range(lp["stop"], len(cfg["layers"])):
        x = layer(x, i)
    return N(x, "final.norm") @ sd["head"].to(F64).T, (torch.stack(taps) if taps else None)


# ------------------------------------------------------------------------------------------------ test material
def make_config(width=64, vocab=97, kinds=("parallel", "mingru", "parallel"), heads=4, kv_heads=2, dim=24, vdim=40,
                rot_dims=8, rot_base=1000.0, scale=0.31, lin_heads=3, lin_dim=8, lin_vdim=16,
                decay=(0.5, 0.93, 0.999), gru_width=48, ff=80, limit=0.75, no_mlp=(), loop=(1, 3, 2),
                left_scale=0.6, right_scale=1.3, eps=1e-5):
    layers = []
    for i, kind in enumerate(kinds):
        if kind == "parallel":
            mixer = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                              "rot": {"dims": rot_dims, "base": rot_base}},
                     "left_scale": left_scale,
                     "right": {"heads": lin_heads, "dim": lin_dim, "vdim": lin_vdim, "decay": list(decay)},
                     "right_scale": right_scale}
        else:
            mixer = {"width": gru_width}
        mlp = None if i in no_mlp else {"kind": "dense", "ff": ff, "limit": limit}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Zofesun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
            "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}


def make_weights(cfg, seed=0, gain=1.0):
    """Random bf16 weights under the checkpoint's names, scaled so every mixer and norm matters."""
    g = torch.Generator().manual_seed(seed)
    H = cfg["width"]
    bf = torch.bfloat16

    def r(*shape, s=None):
        s = gain / math.sqrt(shape[-1]) if s is None else s
        return (torch.randn(*shape, generator=g) * s).to(bf)

    def norm(sd, n):
        sd[n] = (1.0 + 0.2 * torch.randn(H, generator=g)).to(bf)
        sd[n + ".b"] = (0.05 * torch.randn(H, generator=g)).to(bf)
        sd[n + ".alpha"] = torch.tensor(0.6 + 0.5 * float(torch.rand((), generator=g)), dtype=bf)

    sd = {"embed": r(cfg["vocab"], H, s=1.0), "head": r(cfg["vocab"], H, s=2.0 / math.sqrt(H)),
          "loop.step": r(cfg["loop"]["times"], H, s=0.3)}
    norm(sd, "final.norm")
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            norm(sd, p + n)
        m = L["mixer"]
        if L["type"] == "mingru":
            W = m["width"]
            sd.update({p + "mix.z": r(W, H), p + "mix.z.b": r(W, s=0.5), p + "mix.x": r(W, H),
                       p + "mix.x.b": r(W, s=0.5), p + "mix.g": r(W, H), p + "mix.o": r(H, W)})
        else:
            l, q = m["left"], m["right"]
            sd.update({p + "mix.left.q": r(l["heads"] * l["dim"], H, s=2.0 / math.sqrt(H)),
                       p + "mix.left.k": r(l["kv_heads"] * l["dim"], H, s=2.0 / math.sqrt(H)),
                       p + "mix.left.v": r(l["kv_heads"] * l["vdim"], H),
                       p + "mix.left.sink": r(l["heads"], s=1.5), p + "mix.left.o": r(H, l["heads"] * l["vdim"]),
                       p + "mix.right.q": r(q["heads"] * q["dim"], H), p + "mix.right.k": r(q["heads"] * q["dim"], H),
                       p + "mix.right.v": r(q["heads"] * q["vdim"], H), p + "mix.right.g": r(q["heads"] * q["vdim"], H),
                       p + "mix.right.o": r(H, q["heads"] * q["vdim"]),
                       p + "mix.right.norm": (1.0 + 0.2 * torch.randn(q["heads"] * q["vdim"], generator=g)).to(bf)})
        if L["mlp"] is not None:
            Fd = L["mlp"]["ff"]
            sd.update({p + "mlp.gate": r(Fd, H, s=1.5 / math.sqrt(H)), p + "mlp.up": r(Fd, H, s=1.5 / math.sqrt(H)),
                       p + "mlp.down": r(H, Fd)})
    return sd
