"""Vibunex: a decoder-only stack of gated parallel layers (``models/mixers.py``: ``GatedParallelLayer``).

Every layer reads two scalar-gain RMS norms of the same fp32 stream: the first feeds a sink attention and a
time-mix recurrence side by side (outputs summed with fixed weights), the second a sigmoid-routed mixture of
squared-ReLU experts with a gated shared expert; each sublayer's result passes a sigmoid gate computed from
its own input before ``residual_mult`` times their sum is added to the stream.  A scalar-gain RMS norm and the
LM head close the stack.

The configuration comes from the checkpoint's ``config.json`` (``config.vibunex_config``); the rank of the
decay projection is the shape of its tensor.  Checkpoint tensors: ``embed``, ``head``, ``final.norm``, and per
layer ``l<i>.norm{1,2}``, ``l<i>.rg{1,2}[.b]``, ``l<i>.mix.left.*``, ``l<i>.mix.right.*``,
``l<i>.mlp.{router,e<k>.up,e<k>.down,shared.up,shared.down,shared.sg}``.  Projections that read the same input
are fused here into one GEMM (q/k/v/gate/residual gate; shared up/residual gate), the four wide time-mix
projections into one batched product, the experts into stacked tensors.
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
from .mixers import GatedParallelLayer, _param


class VibunexForCausalLM(nn.Module):
    def __init__(self, cfg: ModelConfig, ctx: ParallelContext, dtype, device):
        super().__init__()
        if ctx.tp_size != 1:
            raise NotImplementedError("Vibunex stacks run on one GPU per replica (no tensor-parallel sharding of the mixers)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"Vibunex runs in bfloat16 or float32, not {dtype}")
        self.cfg, self.ctx, self.dtype = cfg, ctx, dtype
        W = cfg.hidden_size
        self.embed = Weight((cfg.vocab_size, W), None, ctx, dtype, device)
        self.layers = nn.ModuleList(GatedParallelLayer(s, W, cfg.rms_eps, cfg.residual_mult, ctx, dtype, device)
                                    for s in cfg.layer_specs)
        self.final_norm = _param((1,), ctx, device)
        self.head = Weight((cfg.vocab_size, W), None, ctx, dtype, device)

    # ---- cache: pages of the attention part, state + previous-input rows of the recurrent part, per layer
    def allocate_caches(self, num_blocks: int, num_slots: int, device):
        return [l.cache(num_blocks, num_slots, self.dtype, device) for l in self.layers]

    def bytes_per_block(self) -> int:
        item = torch.empty((), dtype=self.dtype).element_size()
        return sum(sum(s.cache_row) for s in self.cfg.layer_specs) * KV_BLOCK_SIZE * item

    def bytes_per_slot(self) -> int:
        W = self.cfg.hidden_size
        return sum(4 * (W + s.state_shape[0] * s.state_shape[1] * s.state_shape[2]) for s in self.cfg.layer_specs)

    def forward(self, input_ids: torch.Tensor, meta, caches) -> torch.Tensor:
        x = F.embedding(input_ids, self.embed.data).float()
        for layer, cache in zip(self.layers, caches):
            x = layer(x, None, meta, cache)
        return seqmix.rms_scale(x, self.final_norm.data, None, self.cfg.rms_eps, self.dtype)[0]

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return ops.linear(h, self.head.data).float()

    # ---- parameters: (name, holder, init kind, checkpoint tensors: concatenated along dim 0, or — a list of lists — stacked)
    def named_weight_sources(self):
        yield "embed", self.embed, "normal", None
        for i, l in enumerate(self.layers):
            yield from l.weights(f"l{i}.")
        yield "final.norm", self.final_norm, "ones", None
        yield "head", self.head, "normal", None

    def named_weights(self):
        for name, w, kind, _src in self.named_weight_sources():
            yield name, w, kind

    def checkpoint_sources(self) -> dict:
        return {name: src for name, _w, _k, src in self.named_weight_sources() if src}
