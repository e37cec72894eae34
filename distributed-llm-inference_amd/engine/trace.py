"""Trace replay: feed given token ids through the engine step by step and write logits — no sampling, no
scheduling policy (the trace dictates which requests bring how many tokens in which step), everything else the
engine's own: model registry and loader, block manager with its page pool and state slots, the runner's step
buffer, kernels, cache and state.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N  < steps.jsonl

Input, one JSON object per line: ``{"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}], "end": [...]}``.
``entries``: the next tokens of each request (a request is admitted at its first entry and may skip steps); ``want``:
indices among these tokens whose logits are written; ``end``: requests whose pages and state slot are released after
the step.  All entries of a step run as ONE batch (single-token entries as decode rows in front, longer ones as prefill
chunks).  A step that wants logits writes ``<out>/<step>.f32`` (little-endian fp32 ``[wanted, vocab]``, in entry / want
order); every step prints ``done <step>``.  The page pool holds ``--max-tokens`` tokens (whole pages per request) and
there are ``--max-seqs`` state slots: both are reused as requests end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

from ..config import (CacheConfig, EngineConfig, KV_BLOCK_SIZE, SamplingParams, SchedulerConfig, load_model_config)
from .request import Request, RequestStatus, ScheduledBatch


class TraceReplayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, max_seqs: int = 4, device: str = "auto"):
        from .engine import LLMEngine
        mcfg = load_model_config(model_dir, dtype)
        # pool: max_tokens rounded up to whole pages, plus one page per sequence for requests whose count is not
        # a multiple of the page size
        pages = (max_tokens + KV_BLOCK_SIZE - 1) // KV_BLOCK_SIZE
        budget = max(pages * KV_BLOCK_SIZE, KV_BLOCK_SIZE)
        cfg = EngineConfig(model=mcfg, cache=CacheConfig(num_blocks=pages, enable_prefix_caching=False),
                           sched=SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=budget, max_model_len=budget,
                                                 token_alignment=0),
                           device=device, weights_path=model_dir, use_hip_graphs=False, async_scheduling=False,
                           tune_gemms=False)
        self.engine = LLMEngine(cfg)
        self.runner, self.bm = self.engine.runner, self.engine.bm
        self.live: dict[str, Request] = {}
        self.vocab = mcfg.vocab_size

    def step(self, entries, end=()) -> np.ndarray:
        """Run one step; returns fp32 ``[wanted, vocab]`` in entry / want order."""
        reqs, counts = [], []
        for e in entries:
            toks = np.asarray(e["tokens"], dtype=np.int32)
            if toks.size == 0:
                continue
            if toks.min() < 0 or toks.max() >= self.vocab:
                raise ValueError(f"token id outside the vocabulary in request {e['id']!r}")
            r = self.live.get(e["id"])
            if r is None:
                r = Request(e["id"], next(self.engine._seq_ids), toks, SamplingParams(max_tokens=1))
                r.status = RequestStatus.RUNNING
                self.live[e["id"]] = r
            else:
                if r.num_tokens + toks.size > r.tokens.size:
                    grown = np.empty(max(2 * r.tokens.size, r.num_tokens + toks.size), dtype=np.int32)
                    grown[:r.num_tokens] = r.tokens[:r.num_tokens]
                    r.tokens = grown
                r.tokens[r.num_tokens:r.num_tokens + toks.size] = toks
                r.num_tokens += toks.size
            if not self.bm.allocate(r.seq_id, r.num_tokens):
                raise RuntimeError(f"no page or state slot left for request {e['id']!r} "
                                   f"({self.bm.num_free} pages, {self.bm.num_free_state_slots} slots free)")
            reqs.append((r, int(toks.size), list(e.get("want", ()))))
        out = np.zeros((0, self.vocab), dtype=np.float32)
        if reqs:
            # batch order of the engine: single-token rows first, then the chunks; logits go back to entry order
            order = sorted(range(len(reqs)), key=lambda i: (reqs[i][1] != 1, i))
            num_new = np.asarray([reqs[i][1] for i in order], dtype=np.int32)
            starts = np.concatenate([[0], np.cumsum(num_new)])
            row_of = {i: int(starts[k]) for k, i in enumerate(order)}
            rows = [row_of[i] + w for i, (_r, n, want) in enumerate(reqs) for w in want]
            for i, (_r, n, want) in enumerate(reqs):
                if any(w < 0 or w >= n for w in want):
                    raise ValueError("a wanted index lies outside its entry's tokens")
            batch = ScheduledBatch([reqs[i][0] for i in order], num_new, int((num_new == 1).sum()), int(num_new.sum()),
                                   np.zeros(len(order), dtype=bool))
            out = self.runner.forward_logits(batch, self.bm, rows).numpy()
            for r, n, _ in reqs:
                r.num_computed += n
        for rid in end:
            r = self.live.pop(rid, None)
            if r is not None:
                self.bm.free_seq(r.seq_id)
        return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the page pool holds")
    ap.add_argument("--max-seqs", type=int, default=4, help="state slots = most live requests")
    ap.add_argument("--device", default="auto", choices=["auto", "cuda", "cpu"])
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    rep = TraceReplayer(a.model, a.dtype, a.max_tokens, a.max_seqs, a.device)
    print(f"ready device={rep.runner.device} dtype={rep.runner.dtype} pages={rep.runner.num_blocks}", flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = rep.step(st.get("entries", ()), st.get("end", ()))
        if logits.shape[0]:
            tmp = os.path.join(a.out, f".{st['step']}.part")
            logits.astype("<f4").tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
