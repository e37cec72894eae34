"""Sequence mixers and the layer skeleton of heterogeneous decoder stacks.

Each mixer is a module with its sizes and constants as ``MixerSpec`` parameters, its own slice of the
runner's cache (token-major pages or per-sequence state rows, ``LayerCache``) and one ``forward(h, meta,
cache)`` that serves prefill chunks and decode rows of a mixed step alike:

* ``WindowAttention``   – grouped-query softmax attention, unit-RMS queries / keys, per-head temperature,
  logarithmic distance penalty, sliding window;
* ``LatentAttention``   – low-rank latent + shared rotated key cached per token; the key expansion is folded
  into the query and the value expansion applied after the softmax, so the cache is all the kernel reads;
* ``LightningAttention`` – linear attention with a per-head decay: a ``[D, Dv]`` fp32 state per head and sequence.

``MixerLayer`` wraps one of them (and an optional dense feed-forward) in the sandwich
``x += m · norm_b(sublayer(norm(x)))`` with token shift in front of the mixer.  The residual stream ``x`` is
fp32; GEMM operands are the model dtype.  Tensor parallelism is not implemented for these stacks.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..config import KV_BLOCK_SIZE, MixerSpec
from ..ops import seqmix
from ..parallel.state import ParallelContext
from .layers import Weight


@dataclass
class LayerCache:
    """What one layer run keeps between steps: token-major pages (``k`` / ``v``; latent attention: ``k`` only), the
    recurrent ``state`` rows and the token-shift rows ``shift`` (previous token's normed input) — the latter two indexed
    by state slot."""
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None
    shift: Optional[torch.Tensor] = None


def _param(shape, ctx, device) -> Weight:
    """Small fp32 parameter (norm weights / biases, per-head constants): these enter fp32 arithmetic only."""
    return Weight(tuple(shape), None, ctx, torch.float32, device)


def _matrix(out_f: int, in_f: int, ctx, dtype, device) -> Weight:
    return Weight((out_f, in_f), None, ctx, dtype, device)


class Norm(nn.Module):
    """Layer norm parameters (weight and bias over ``n`` features)."""

    def __init__(self, n: int, ctx, device):
        super().__init__()
        self.w, self.b = _param((n,), ctx, device), _param((n,), ctx, device)


class WindowAttention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, G, D, Dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        assert H % G == 0, "query heads must be a multiple of the key/value heads"
        self.qkv = _matrix(H * D + G * D + G * Dv, width, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.q_norm, self.k_norm = _param((D,), ctx, device), _param((D,), ctx, device)
        self.r1, self.r2, self.temp = (_param((H,), ctx, device) for _ in range(3))

    def weights(self, p):
        yield p + "qkv", self.qkv, "normal", [p + "q", p + "k", p + "v"]
        yield p + "o", self.o, "normal", None
        yield p + "q.norm", self.q_norm, "ones", None
        yield p + "k.norm", self.k_norm, "ones", None
        yield p + "r1", self.r1, "small", None
        yield p + "r2", self.r2, "small", None
        yield p + "temp", self.temp, "ones", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.dim, dtype=dtype, device=device),
                          v=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_heads * s.vdim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, G, D, Dv = s.heads, s.kv_heads, s.dim, s.vdim
        T = h.shape[0]
        qkv = ops.linear(h, self.qkv.data)
        seqmix.qk_norm_cache(qkv, self.q_norm.data, self.k_norm.data, self.eps, meta.slot_mapping, cache.k, cache.v, H, G, D, Dv)
        out = torch.empty(T, H, Dv, dtype=h.dtype, device=h.device)
        seqmix.token_attention(out, qkv[:, :H * D].view(T, H, D), None, cache.k, cache.v, meta, G, Dv, s.scale, s.window,
                               self.temp.data, self.r1.data, self.r2.data)
        return ops.linear(out.view(T, H * Dv), self.o.data)


class LatentAttention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D, R, Dv, C = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank
        assert spec.rot_dims <= R and spec.rot_dims % 2 == 0
        self.q_dkv = _matrix(H * (D + R) + C + R, width, ctx, dtype, device)
        self.c_norm = _param((C,), ctx, device)
        self.uk = _matrix(H * D, C, ctx, dtype, device)
        self.uv = _matrix(H * Dv, C, ctx, dtype, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.register_buffer("inv_freq", seqmix.rotary_inv_freq(spec.rot_base, spec.rot_dims, device), persistent=False)

    def weights(self, p):
        yield p + "q_dkv", self.q_dkv, "normal", [p + "q", p + "dkv"]
        yield p + "dkv.norm", self.c_norm, "ones", None
        yield p + "uk", self.uk, "normal", None
        yield p + "uv", self.uv, "normal", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(k=torch.zeros(num_blocks, KV_BLOCK_SIZE, s.kv_rank + s.rot_dim, dtype=dtype, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, D, R, Dv, C = s.heads, s.dim, s.rot_dim, s.vdim, s.kv_rank
        T = h.shape[0]
        both = ops.linear(h, self.q_dkv.data)
        q, dkv = both[:, :H * (D + R)], both[:, H * (D + R):]
        seqmix.latent_prep(q, dkv, self.c_norm.data, self.eps, meta.positions, self.inv_freq, s.rot_dims, meta.slot_mapping,
                           cache.k, H, D, R, C)
        q3 = q.view(T, H, D + R) if q.is_contiguous() else q.unflatten(1, (H, D + R))
        # key expansion folded into the query: (W_uk c) · q = c · (W_ukᵀ q) — one [D] → [C] product per head and token
        q_lat = torch.bmm(q3[:, :, :D].transpose(0, 1), self.uk.data.view(H, D, C))                  # [H, T, C]
        o_lat = torch.empty(H, T, C, dtype=h.dtype, device=h.device)
        seqmix.token_attention(o_lat.transpose(0, 1), q_lat.transpose(0, 1), q3[:, :, D:], cache.k, None, meta, 1, C, s.scale)
        # value expansion after the softmax: Σ p_j (W_uv c_j) = W_uv (Σ p_j c_j)
        out = torch.bmm(o_lat, self.uv.data.view(H, Dv, C).transpose(1, 2))                          # [H, T, Dv]
        return ops.linear(out.transpose(0, 1).reshape(T, H * Dv), self.o.data)


class LightningAttention(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.s, self.eps = spec, eps
        H, D, Dv = spec.heads, spec.dim, spec.vdim
        assert len(spec.decay) == H, "one decay per head"
        self.qkvg = _matrix(2 * H * D + 2 * H * Dv, width, ctx, dtype, device)
        self.norm = _param((H * Dv,), ctx, device)
        self.o = _matrix(width, H * Dv, ctx, dtype, device)
        self.register_buffer("decay", torch.tensor(spec.decay, dtype=torch.float32, device=device), persistent=False)

    def weights(self, p):
        yield p + "qkvg", self.qkvg, "normal", [p + "q", p + "k", p + "v", p + "g"]
        yield p + "norm", self.norm, "ones", None
        yield p + "o", self.o, "normal", None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        s = self.s
        return LayerCache(state=torch.zeros(num_slots, s.heads, s.dim, s.vdim, dtype=torch.float32, device=device))

    def forward(self, h, meta, cache: LayerCache):
        s = self.s
        H, D, Dv = s.heads, s.dim, s.vdim
        qkvg = ops.linear(h, self.qkvg.data)
        o = seqmix.lightning_scan(qkvg, cache.state, meta, H, D, Dv, self.decay)
        y = seqmix.rms_gate(o, self.norm.data, self.eps, qkvg[:, 2 * H * D + H * Dv:], h.dtype)
        return ops.linear(y, self.o.data)


MIXERS = {"attention": WindowAttention, "latent_attention": LatentAttention, "lightning": LightningAttention}


class DenseFF(nn.Module):
    """``W_down · relu(W_up h)²``."""

    def __init__(self, width: int, ff: int, ctx, dtype, device):
        super().__init__()
        self.up, self.down = _matrix(ff, width, ctx, dtype, device), _matrix(width, ff, ctx, dtype, device)

    def forward(self, h):
        return ops.linear(seqmix.relu2(ops.linear(h, self.up.data)), self.down.data)


class MixerLayer(nn.Module):
    def __init__(self, spec: MixerSpec, width: int, eps: float, mult: float, ctx: ParallelContext, dtype, device):
        super().__init__()
        self.spec, self.eps, self.mult, self.dtype = spec, eps, mult, dtype
        self.norm1, self.norm1b = Norm(width, ctx, device), Norm(width, ctx, device)
        self.norm2, self.norm2b = Norm(width, ctx, device), Norm(width, ctx, device)
        self.shift = _param((width,), ctx, device)
        self.mixer = MIXERS[spec.kind](spec, width, eps, ctx, dtype, device)
        self.ff = DenseFF(width, spec.ff, ctx, dtype, device) if spec.ff else None

    def cache(self, num_blocks, num_slots, dtype, device) -> LayerCache:
        c = self.mixer.cache(num_blocks, num_slots, dtype, device)
        c.shift = torch.zeros(num_slots, self.shift.data.shape[0], dtype=torch.float32, device=device)
        return c

    def forward(self, x, restart, meta, cache: LayerCache):
        """``x``: fp32 stream ``[T, W]``, updated in place (a fresh tensor is returned when ``restart`` — the term added in
        front of a repeated pass — is given)."""
        eps, m = self.eps, self.mult
        h, x = seqmix.ln_shift(x, restart, self.norm1.w.data, self.norm1.b.data, eps, self.shift.data, cache.shift, meta, self.dtype)
        y = self.mixer(h, meta, cache)
        if self.ff is None:
            seqmix.add_ln(x, y, self.norm1b.w.data, self.norm1b.b.data, eps, m)
            return x
        h = seqmix.add_ln(x, y, self.norm1b.w.data, self.norm1b.b.data, eps, m, self.norm2.w.data, self.norm2.b.data, self.dtype)
        seqmix.add_ln(x, self.ff(h), self.norm2b.w.data, self.norm2b.b.data, eps, m)
        return x
