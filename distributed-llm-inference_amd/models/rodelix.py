"""Rodelix: a decoder-only stack whose layers each pick one of three sequence mixers (sliding-window
attention, latent attention, lightning linear attention — ``models/mixers.py``), with layer norms before and
after every sublayer, token shift in front of every mixer, an optional repeated span of layers and
soft-capped logits.

The configuration comes from the checkpoint's ``config.json`` (``config.rodelix_config``): per layer the
mixer type with its sizes and the feed-forward width; ``loop`` (layers ``start … stop-1`` run ``times``
times with the same weights, every pass on its own cache and state, every pass but the first preceded by
adding the embedding output to the stream); ``residual_mult``; ``logit_softcap``; ``norm.eps``.

Checkpoint tensors: ``embed``, ``head``, ``final.norm[.b]``, and per layer ``l<i>.norm{1,1b,2,2b}[.b]``,
``l<i>.shift``, ``l<i>.mix.*`` and ``l<i>.mlp.{up,down}``; q/k/v(/g) and q/dkv projections are stored
separately and fused here into one GEMM per mixer.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..config import KV_BLOCK_SIZE, ModelConfig
from ..ops import seqmix
from ..parallel.state import ParallelContext
from .layers import Weight
from .mixers import MixerLayer, Norm


class RodelixForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, ctx: ParallelContext, dtype, device):
        super().__init__()
        if ctx.tp_size != 1:
            raise NotImplementedError("Rodelix stacks run on one GPU per replica (no tensor-parallel sharding of the mixers)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"Rodelix runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.ctx, self.dtype = cfg, ctx, dtype
        W = cfg.hidden_size
        self.embed = Weight((cfg.vocab_size, W), None, ctx, dtype, device)
        self.layers = nn.ModuleList(MixerLayer(s, W, cfg.rms_eps, cfg.residual_mult, ctx, dtype, device)
                                    for s in cfg.layer_specs)
        self.final_norm = Norm(W, ctx, device)
        self.head = Weight((cfg.vocab_size, W), None, ctx, dtype, device)
        self.runs = cfg.layer_runs
        self.restarts = any(again for _, again in self.runs)

    # ---- cache: one LayerCache per layer RUN (a repeated layer has one per pass)
    def allocate_caches(self, num_blocks: int, num_slots: int, device):
        return [self.layers[i].cache(num_blocks, num_slots, self.dtype, device) for i, _ in self.runs]

    def bytes_per_block(self) -> int:
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(sum(self.cfg.layer_specs[i].cache_row) for i, _ in self.runs) * KV_BLOCK_SIZE * item

    def bytes_per_slot(self) -> int:
        W = self.cfg.hidden_size
        return sum(4 * (W + (s.heads * s.dim * s.vdim if s.stateful else 0))
                   for s in (self.cfg.layer_specs[i] for i, _ in self.runs))

    def forward(self, input_ids: torch.Tensor, meta, caches) -> torch.Tensor:
        x0 = F.embedding(input_ids, self.embed.data).float()
        x = x0.clone() if self.restarts else x0            # the stream is updated in place; the restart term must survive
        for (i, again), cache in zip(self.runs, caches):
            x = self.layers[i](x, x0 if again else None, meta, cache)
        return seqmix.layer_norm(x, self.final_norm.w.data, self.final_norm.b.data, self.cfg.rms_eps, self.dtype)

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(h, self.head.data)
        cap = self.cfg.logit_softcap
        return seqmix.softcap(logits, cap) if cap > 0 else logits.float()

    # ---- parameters: (name, holder, init kind, checkpoint tensors fused along dim 0 or None)
    def named_weight_sources(self):
        yield "embed", self.embed, "normal", None
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            for nm in ("norm1", "norm1b", "norm2", "norm2b"):
                n = getattr(l, nm)
                yield p + nm, n.w, "ones", None
                yield p + nm + ".b", n.b, "zeros", None
            yield p + "shift", l.shift, "half", None
            yield from l.mixer.weights(p + "mix.")
            if l.ff is not None:
                yield p + "mlp.up", l.ff.up, "normal", None
                yield p + "mlp.down", l.ff.down, "normal", None
        yield "final.norm", self.final_norm.w, "ones", None
        yield "final.norm.b", self.final_norm.b, "zeros", None
        yield "head", self.head, "normal", None

    def named_weights(self):
        for name, w, kind, _src in self.named_weight_sources():
            yield name, w, kind

    def checkpoint_sources(self) -> dict:
        """Fused parameter name → the checkpoint tensors concatenated (dim 0) into it."""
        return {name: src for name, _w, _k, src in self.named_weight_sources() if src}
