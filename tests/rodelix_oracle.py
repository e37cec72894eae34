"""Slow, plain oracle of the Rodelix design: one function per mechanism, written straight from the
equations with explicit loops over positions, in float64 by default.  It shares no code with the
package: it takes the configuration as the nested dict a ``config.json`` of this design holds and
the weights as a ``{name: tensor}`` dict with the checkpoint's tensor names.

Notation: ``x`` residual stream ``[n, W]``; ``h`` what a mixer reads; ``t`` a position counted
from 0; ``eps`` the configuration's ``norm.eps``.
"""
from __future__ import annotations

import math

import torch


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def token_shift(h, mix):
    """``h[t] + (h[t-1] - h[t]) * mix`` with ``h[-1] = 0``; the unshifted rows are the ones looked back at."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mix


def rotate_pairs(v, t, base, dims):
    """Rotate the first ``dims`` entries of ``v`` (last axis) for position ``t``: entries (2i, 2i+1) form a pair
    turned by the angle ``t * base**(-2i/dims)``."""
    out = v.clone()
    for i in range(dims // 2):
        a = t * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


def softmax_rows(scores):
    m = scores.max()
    e = torch.exp(scores - m)
    return e / e.sum()


def window_attention(h, P, m, eps):
    """Grouped-query attention with per-head unit-RMS queries and keys, a per-head temperature, a logarithmic distance
    penalty and a sliding window.  ``P``: the mixer's tensors by short name; ``m``: its ``mixer`` dict."""
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    win = m["mask"]["size"]
    q = (h @ P["q"].T).view(n, H, D)
    k = (h @ P["k"].T).view(n, G, D)
    v = (h @ P["v"].T).view(n, G, Dv)
    q = unit_rms(q, eps) * P["q.norm"]
    k = unit_rms(k, eps) * P["k.norm"]
    out = torch.zeros(n, H, Dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(n):
            lo = max(0, i - win + 1)
            js = torch.arange(lo, i + 1)
            s = (k[lo:i + 1, g] @ q[i, hd]) * m["scale"] * P["temp"][hd]
            s = s - P["r1"][hd] * torch.log(1.0 + P["r2"][hd] * (i - js).to(h.dtype))
            out[i, hd] = softmax_rows(s) @ v[lo:i + 1, g]
    return out.reshape(n, H * Dv) @ P["o"].T


def latent_attention(h, P, m, eps):
    """Attention whose keys and values are expanded from one low-rank latent per token; a small rotated key part is
    shared by all heads.  Causal, plain softmax."""
    n = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q = (h @ P["q"].T).view(n, H, D + R)
    dkv = h @ P["dkv"].T
    c = unit_rms(dkv[:, :C], eps) * P["dkv.norm"]
    kr = dkv[:, C:]
    ku = (c @ P["uk"].T).view(n, H, D)
    v = (c @ P["uv"].T).view(n, H, Dv)
    qu, qr = q[..., :D], q[..., D:]
    qr = torch.stack([rotate_pairs(qr[t], t, base, dims) for t in range(n)])
    kr = torch.stack([rotate_pairs(kr[t], t, base, dims) for t in range(n)])
    out = torch.zeros(n, H, Dv, dtype=h.dtype)
    for hd in range(H):
        for i in range(n):
            s = (ku[:i + 1, hd] @ qu[i, hd] + kr[:i + 1] @ qr[i, hd]) * m["scale"]
            out[i, hd] = softmax_rows(s) @ v[:i + 1, hd]
    return out.reshape(n, H * Dv) @ P["o"].T


def silu(z):
    return z / (1.0 + torch.exp(-z))


def lightning(h, P, m, eps):
    """Linear attention with a per-head scalar decay: a ``[D, Dv]`` state per head, updated token by token."""
    n = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ P["q"].T).view(n, H, D)
    k = silu(h @ P["k"].T).view(n, H, D)
    v = silu(h @ P["v"].T).view(n, H, Dv)
    out = torch.zeros(n, H, Dv, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(n):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    o = unit_rms(out.reshape(n, H * Dv), eps) * P["norm"]
    o = o * (1.0 / (1.0 + torch.exp(-(h @ P["g"].T))))
    return o @ P["o"].T


def dense_ff(h, P):
    z = torch.clamp(h @ P["up"].T, min=0.0)
    return (z * z) @ P["down"].T


MIXERS = {"attention": window_attention, "latent_attention": latent_attention, "lightning": lightning}


def layer_runs(cfg):
    """Indices of the layers in execution order, and for each whether a new pass of the loop starts there (not the first)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order, restart = [], []
    for i in range(a):
        order.append(i), restart.append(False)
    for p in range(times if b > a else 0):
        for i in range(a, b):
            order.append(i), restart.append(p > 0 and i == a)
    for i in range(b if b > a else a, n):
        order.append(i), restart.append(False)
    return order, restart


def forward(cfg, W, tokens, dtype=torch.float64):
    """Logits ``[n, vocab]`` of one whole sequence and the residual stream after every layer run ``[runs, n, W]``."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    trail = []
    order, restart = layer_runs(cfg)
    for i, again in zip(order, restart):
        spec = cfg["layers"][i]
        pre = f"l{i}."
        if again:
            x = x + x0
        h = layer_norm(x, W[pre + "norm1"], W[pre + "norm1.b"], eps)
        h = token_shift(h, W[pre + "shift"])
        P = {k[len(pre) + 4:]: v for k, v in W.items() if k.startswith(pre + "mix.")}
        y = MIXERS[spec["type"]](h, P, spec["mixer"], eps)
        x = x + mult * layer_norm(y, W[pre + "norm1b"], W[pre + "norm1b.b"], eps)
        if spec.get("mlp"):
            h = layer_norm(x, W[pre + "norm2"], W[pre + "norm2.b"], eps)
            P = {k[len(pre) + 4:]: v for k, v in W.items() if k.startswith(pre + "mlp.")}
            y = dense_ff(h, P)
            x = x + mult * layer_norm(y, W[pre + "norm2b"], W[pre + "norm2b.b"], eps)
        trail.append(x.clone())
    h = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    logits = h @ W["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(trail)


def random_weights(cfg, seed=0, dtype=torch.float32, spread=1.0):
    """A full set of tensors for ``cfg`` with the checkpoint's names; norm weights near one, biases and the rest small."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std):
        return (torch.randn(*shape, generator=g) * std * spread).to(dtype)

    def lin(o, i):
        return rnd(o, i, std=1.0 / math.sqrt(i))

    W = {"embed": rnd(V, Wd, std=1.0), "head": lin(V, Wd),
         "final.norm": (1 + rnd(Wd, std=0.1)), "final.norm.b": rnd(Wd, std=0.1)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        for nm in ("norm1", "norm2", "norm1b", "norm2b"):
            W[p + nm] = 1 + rnd(Wd, std=0.1)
            W[p + nm + ".b"] = rnd(Wd, std=0.1)
        W[p + "shift"] = torch.rand(Wd, generator=g).to(dtype)
        t = spec["type"]
        if t == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = lin(H * D, Wd), lin(G * D, Wd), lin(G * Dv, Wd)
            W[p + "mix.q.norm"], W[p + "mix.k.norm"] = 1 + rnd(D, std=0.1), 1 + rnd(D, std=0.1)
            W[p + "mix.r1"] = torch.rand(H, generator=g).to(dtype)
            W[p + "mix.r2"] = torch.rand(H, generator=g).to(dtype)
            W[p + "mix.temp"] = (0.5 + torch.rand(H, generator=g)).to(dtype)
            W[p + "mix.o"] = lin(Wd, H * Dv)
        elif t == "latent_attention":
            H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[p + "mix.q"], W[p + "mix.dkv"] = lin(H * (D + R), Wd), lin(C + R, Wd)
            W[p + "mix.dkv.norm"] = 1 + rnd(C, std=0.1)
            W[p + "mix.uk"], W[p + "mix.uv"] = lin(H * D, C), lin(H * Dv, C)
            W[p + "mix.o"] = lin(Wd, H * Dv)
        elif t == "lightning":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            W[p + "mix.q"], W[p + "mix.k"] = lin(H * D, Wd), lin(H * D, Wd)
            W[p + "mix.v"], W[p + "mix.g"] = lin(H * Dv, Wd), lin(H * Dv, Wd)
            W[p + "mix.norm"] = 1 + rnd(H * Dv, std=0.1)
            W[p + "mix.o"] = lin(Wd, H * Dv)
        else:
            raise ValueError(t)
        if spec.get("mlp"):
            W[p + "mlp.up"], W[p + "mlp.down"] = lin(spec["mlp"]["ff"], Wd), lin(Wd, spec["mlp"]["ff"])
    return W
