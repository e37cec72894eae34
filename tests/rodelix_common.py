"""Shared pieces of the Rodelix tests: small configurations, checkpoints written from the oracle's random weights,
a rig that replays step schedules through the engine (``dli_amd.engine.trace.TraceReplayer``: the engine's own runner,
block manager, kernels) and the comparison with ``rodelix_oracle``.  The same cases run on the CPU path
(``test_rodelix.py``) and on the GPU kernels (``test_rodelix_gpu.py``)."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

import rodelix_oracle as oracle

ATTN = {"type": "attention", "mlp": {"kind": "dense", "ff": 96},
        "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.35, "mask": {"size": 37}}}
LIGHT = {"type": "lightning", "mlp": {"kind": "dense", "ff": 80},
         "mixer": {"heads": 3, "dim": 16, "vdim": 40, "decay": [0.55, 0.93, 0.999]}}
LATENT = {"type": "latent_attention", "mlp": None,
          "mixer": {"heads": 3, "dim": 20, "rot_dim": 12, "vdim": 28, "kv_rank": 48, "scale": 0.3,
                    "rot": {"base": 5000.0, "dims": 8}}}


def make_cfg(layers, width=80, vocab=211, loop=None, mult=0.4, cap=12.0, eps=1e-5):
    cfg = {"architecture": "Rodelix", "vocab": vocab, "width": width, "residual_mult": mult, "logit_softcap": cap,
           "norm": {"eps": eps}, "layers": copy.deepcopy(list(layers))}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


FULL = make_cfg([ATTN, LIGHT, LATENT, LIGHT], loop=(1, 3, 2))


def write_checkpoint(path, cfg, seed=0, bf16=False, edit=None):
    """Writes config.json + model.safetensors under ``path``; returns the weights (as stored, fp32 values) for the oracle."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    W = oracle.random_weights(cfg, seed)
    if edit:
        edit(W)
    if bf16:
        W = {k: v.to(torch.bfloat16) for k, v in W.items()}
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return {k: v.float() for k, v in W.items()}


class Rig:
    def __init__(self, model_dir, dtype="float32", device="cpu", max_tokens=1024, max_seqs=4):
        from dli_amd.engine.trace import TraceReplayer
        self.rep = TraceReplayer(str(model_dir), dtype, max_tokens, max_seqs, device)

    def run(self, requests, schedule):
        """``requests``: id → token list; ``schedule``: list of steps, each a list of (id, count).  Every position's logits
        are collected; a request ends with its last token.  Returns id → fp32 ``[n, vocab]``."""
        at = {i: 0 for i in requests}
        got = {i: [] for i in requests}
        for step in schedule:
            entries, end = [], []
            for i, n in step:
                lo, hi = at[i], at[i] + n
                assert hi <= len(requests[i])
                entries.append({"id": i, "tokens": requests[i][lo:hi], "want": list(range(n))})
                at[i] = hi
                if hi == len(requests[i]):
                    end.append(i)
            out = self.rep.step(entries, end)
            r = 0
            for e in entries:
                n = len(e["tokens"])
                got[e["id"]].append(out[r:r + n])
                r += n
        return {i: np.concatenate(v) if v else np.zeros((0, 0)) for i, v in got.items()}


def chunks(n, sizes):
    """Cut ``n`` tokens into portions cycling through ``sizes``."""
    out, k = [], 0
    while n > 0:
        c = min(sizes[k % len(sizes)], n)
        out.append(c)
        n -= c
        k += 1
    return out


def alone(i, n, sizes):
    return [[(i, c)] for c in chunks(n, sizes)]


def rel_err(got, want):
    """Root mean square of the difference over the root mean square of the expected logits (means taken off), per row; max."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))).max())


def expect(cfg, W, tokens):
    return oracle.forward(cfg, W, tokens)[0].numpy()


def tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


TOL = {"float32": 2e-4, "bfloat16": 6e-2}
