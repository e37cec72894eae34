"""Slow, plain oracle of the Vibunex design: one function per mechanism, written from the equations with
explicit loops over positions, float64 by default.  It shares no code with the package: the configuration is
the nested dict a ``config.json`` of this design holds, the weights a ``{name: tensor}`` dict with the
checkpoint's tensor names.

A layer adds ``m * (gate1 * mixer(n1) + gate2 * ff(n2))`` to the stream ``x``, where ``n1``/``n2`` are two
scalar-gain RMS norms of the same ``x`` and ``gate_i = sigmoid(R_i n_i + b_i)``.  The mixer is the weighted sum of
a softmax attention (whole-projection q/k norm, partial rotation with stretched frequencies, a sink in the
denominator, weights mixed across heads, output gate) and a recurrent time mix with per-channel,
per-token decay.  The feed-forward is a sigmoid-routed mixture of squared-ReLU experts plus a gated shared one.
"""
from __future__ import annotations

import math

import torch


def scalar_rms_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


# ------------------------------------------------------------------------------------ rotation
def stretched_frequencies(rot):
    """Per pair ``i`` of the ``dims`` rotated entries: ``base**(-2i/dims)``, divided by ``factor`` for the slow pairs, kept
    for the fast ones, blended linearly between the two corner pairs.  Returns (list of frequencies, magnitude)."""
    dims, base = rot["dims"], rot["base"]
    sc = rot.get("scaling")
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not sc:
        return f, 1.0

    def corner(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(corner(sc["fast"])), 0)
    hi = min(math.ceil(corner(sc["slow"])), dims - 1)
    out = []
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / sc["factor"] * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(v, t, freqs, mag, dims):
    """Entries ``i`` and ``i + dims/2`` of the last axis (``i < dims/2``) are a pair turned by ``t * freqs[i]``; cosine and
    sine are scaled by ``mag``; entries from ``dims`` on pass through."""
    out = v.clone()
    half = dims // 2
    for i in range(half):
        a = t * freqs[i]
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, w = v[..., i], v[..., i + half]
        out[..., i] = u * c - w * s
        out[..., i + half] = w * c + u * s
    return out


# ------------------------------------------------------------------------------------ left mixer
def sink_talk_attention(h, P, m, eps):
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ P["q"].T, h @ P["k"].T, (h @ P["v"].T).view(n, G, Dv)
    q = (q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * P["q.norm"]).view(n, H, D)
    k = (k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * P["k.norm"]).view(n, G, D)
    freqs, mag = stretched_frequencies(m["rot"])
    dims = m["rot"]["dims"]
    q = torch.stack([rotate_half(q[t], t, freqs, mag, dims) for t in range(n)])
    k = torch.stack([rotate_half(k[t], t, freqs, mag, dims) for t in range(n)])
    out = torch.zeros(n, H, Dv, dtype=h.dtype)
    for i in range(n):
        wts = torch.zeros(H, i + 1, dtype=h.dtype)
        for hd in range(H):
            s = (k[:i + 1, hd // (H // G)] @ q[i, hd]) * m["scale"]
            top = max(float(s.max()), float(P["sink"][hd]))
            e = torch.exp(s - top)
            wts[hd] = e / (e.sum() + math.exp(float(P["sink"][hd]) - top))
        mixed = P["talk"] @ wts
        for hd in range(H):
            out[i, hd] = mixed[hd] @ v[:i + 1, hd // (H // G)]
    gate = sigmoid(h @ P["g"].T)
    return (out.reshape(n, H * Dv) * gate) @ P["o"].T


# ------------------------------------------------------------------------------------ right mixer
def time_mix(h, P, m, eps):
    n = h.shape[0]
    H, D = m["heads"], m["dim"]
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    mixes = {s: h + (prev - h) * P["mu." + s] for s in "rkvgw"}
    r = (mixes["r"] @ P["r"].T).view(n, H, D)
    k = (mixes["k"] @ P["k"].T).view(n, H, D)
    v = (mixes["v"] @ P["v"].T).view(n, H, D)
    gate = silu(mixes["g"] @ P["g"].T)
    w = torch.exp(-torch.exp(torch.tanh(mixes["w"] @ P["w1"].T) @ P["w2"].T + P["w0"])).view(n, H, D)
    out = torch.zeros(n, H, D, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(D, D, dtype=h.dtype)
        for t in range(n):
            kv = torch.outer(k[t, hd], v[t, hd])
            o = (S + P["u"][hd][:, None] * kv).T @ r[t, hd]
            out[t, hd] = o / torch.sqrt((o * o).mean() + eps)
            S = w[t, hd][:, None] * S + kv
    return (out.reshape(n, H * D) * P["norm"] * gate) @ P["o"].T


def parallel_mixer(h, P, m, eps):
    left = sink_talk_attention(h, {k[5:]: v for k, v in P.items() if k.startswith("left.")}, m["left"], eps)
    right = time_mix(h, {k[6:]: v for k, v in P.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ------------------------------------------------------------------------------------ feed-forward
def relu2_expert(h, up, down):
    return (torch.clamp(h @ up.T, min=0.0) ** 2) @ down.T


def routed_ff(h, P, mlp):
    n = h.shape[0]
    r = mlp["router"]
    s = sigmoid(h @ P["router"].T)
    out = torch.zeros_like(h)
    for t in range(n):
        order = sorted(range(r["experts"]), key=lambda e: -float(s[t, e]))[:r["top"]]
        for e in order:
            out[t] += s[t, e] * r["scale"] * relu2_expert(h[t], P[f"e{e}.up"], P[f"e{e}.down"])
    if mlp.get("shared"):
        out = out + sigmoid(h @ P["shared.sg"].T) * relu2_expert(h, P["shared.up"], P["shared.down"])
    return out


# ------------------------------------------------------------------------------------ the stack
def _sub(W, prefix):
    return {k[len(prefix):]: v for k, v in W.items() if k.startswith(prefix)}


def forward(cfg, W, tokens, dtype=torch.float64):
    """Logits ``[n, vocab]`` of one sequence, and the stream after every layer ``[layers, n, width]``."""
    W = {k: v.to(dtype) for k, v in W.items()}
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        n1 = scalar_rms_norm(x, W[p + "norm1"], eps)
        add = sigmoid(n1 @ W[p + "rg1"].T + W[p + "rg1.b"]) * parallel_mixer(n1, _sub(W, p + "mix."), layer["mixer"], eps)
        if layer.get("mlp"):
            n2 = scalar_rms_norm(x, W[p + "norm2"], eps)
            add = add + sigmoid(n2 @ W[p + "rg2"].T + W[p + "rg2.b"]) * routed_ff(n2, _sub(W, p + "mlp."), layer["mlp"])
        x = x + mult * add
        streams.append(x)
    logits = scalar_rms_norm(x, W["final.norm"], eps) @ W["head"].T
    return logits, torch.stack(streams)


def random_weights(cfg, seed=0, dtype=torch.float32, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def mat(o, i, gain=1.0):
        return torch.randn(o, i, generator=g, dtype=dtype) * (gain * spread / math.sqrt(i))

    def vec(n, mean=0.0, std=0.3):
        return mean + std * torch.randn(n, generator=g, dtype=dtype)

    W = {"embed": torch.randn(V, Wd, generator=g, dtype=dtype), "head": mat(V, Wd), "final.norm": vec((), 1.0, 0.1)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        W[p + "norm1"] = vec((), 1.0, 0.1)
        W[p + "rg1"], W[p + "rg1.b"] = mat(Wd, Wd), vec(Wd)
        a, b = layer["mixer"]["left"], layer["mixer"]["right"]
        H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        q = p + "mix.left."
        W[q + "q"], W[q + "k"], W[q + "v"] = mat(H * D, Wd), mat(G * D, Wd), mat(G * Dv, Wd)
        W[q + "q.norm"], W[q + "k.norm"] = vec(H * D, 1.0), vec(G * D, 1.0)
        W[q + "talk"] = torch.eye(H, dtype=dtype) + 0.3 * torch.randn(H, H, generator=g, dtype=dtype)
        W[q + "sink"] = vec(H, 0.0, 1.0)
        W[q + "g"], W[q + "o"] = mat(H * Dv, Wd), mat(Wd, H * Dv)
        q = p + "mix.right."
        Hr, Dr = b["heads"], b["dim"]
        lora = b.get("lora", 8)
        for s in "rkvgw":
            W[q + "mu." + s] = torch.rand(Wd, generator=g, dtype=dtype)
        for s in "rkvg":
            W[q + s] = mat(Hr * Dr, Wd)
        W[q + "w1"], W[q + "w2"] = mat(lora, Wd), mat(Hr * Dr, lora)
        W[q + "w0"] = vec(Hr * Dr, -1.0, 1.0)
        W[q + "u"] = vec((Hr, Dr), 0.3, 0.5)
        W[q + "norm"] = vec(Hr * Dr, 1.0)
        W[q + "o"] = mat(Wd, Hr * Dr)
        mlp = layer.get("mlp")
        if mlp:
            q = p + "mlp."
            W[p + "norm2"] = vec((), 1.0, 0.1)
            W[p + "rg2"], W[p + "rg2.b"] = mat(Wd, Wd), vec(Wd)
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                W[q + f"e{e}.up"], W[q + f"e{e}.down"] = mat(ff, Wd), mat(Wd, ff)
            W[q + "router"] = mat(mlp["router"]["experts"], Wd, 2.0)
            if mlp.get("shared"):
                fs = mlp["shared"]["ff"]
                W[q + "shared.up"], W[q + "shared.down"], W[q + "shared.sg"] = mat(fs, Wd), mat(Wd, fs), mat(1, Wd)
    return W
