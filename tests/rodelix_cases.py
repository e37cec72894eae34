"""The Rodelix test cases, parametrised by device and dtype (see ``rodelix_common``).  Each case builds its own small
configuration and checkpoint, replays schedules through the engine and compares every position's logits with the oracle."""
from __future__ import annotations

import copy

import numpy as np
import torch

import rodelix_oracle as oracle
from rodelix_common import (ATTN, FULL, LATENT, LIGHT, Rig, TOL, alone, chunks, expect, make_cfg, rel_err, tokens,
                            write_checkpoint)


def _setup(tmp, cfg, dtype, device, seed=0, edit=None, **rig):
    W = write_checkpoint(tmp, cfg, seed, bf16=dtype == "bfloat16", edit=edit)
    return W, Rig(tmp, dtype, device, **rig)


def _check(got, want, dtype, what=""):
    e = rel_err(got, want)
    assert e < TOL[dtype], f"{what}: relative error {e:.3e} over {TOL[dtype]:.1e}"


# ---------------------------------------------------------------- each mechanism alone
def case_mechanism(tmp, device, dtype, kind):
    layer = {"attention": ATTN, "lightning": LIGHT, "latent_attention": LATENT}[kind]
    cfg = make_cfg([layer], width=72)
    W, rig = _setup(tmp, cfg, dtype, device, seed=3)
    toks = tokens(140, cfg["vocab"], 1)
    want = expect(cfg, W, toks)
    got = rig.run({"a": toks}, alone("a", len(toks), [len(toks)]))["a"]
    _check(got, want, dtype, f"{kind} whole prompt")
    got = rig.run({"b": toks}, alone("b", len(toks), [31, 2, 1, 40, 1, 1, 7]))["b"]
    _check(got, want, dtype, f"{kind} in portions")


# ---------------------------------------------------------------- prefill against token-by-token, portions down to two
def case_prefill_decode_portions(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=5)
    toks = tokens(100, FULL["vocab"], 2)
    want = expect(FULL, W, toks)
    for name, sizes in (("whole", [100]), ("one by one", [1]), ("portions", [2, 3, 64, 5, 2, 17]), ("page edges", [32, 32, 1, 31, 4])):
        got = rig.run({name: toks}, alone(name, len(toks), sizes))[name]
        _check(got, want, dtype, name)


# ---------------------------------------------------------------- unequal requests in one batch against each alone
def case_mixed_batch(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=7, max_tokens=512)
    reqs = {"s1": tokens(1, FULL["vocab"], 10), "s23": tokens(23, FULL["vocab"], 11), "m70": tokens(70, FULL["vocab"], 12),
            "l130": tokens(130, FULL["vocab"], 13)}
    want = {i: expect(FULL, W, t) for i, t in reqs.items()}
    plan = {"s1": [1], "s23": [2, 1, 1, 16, 1, 1, 1], "m70": chunks(70, [33, 1, 1, 2, 1]), "l130": chunks(130, [40, 3, 1, 1, 64, 1])}
    sched, k = [], 0
    while any(plan.values()):
        step = []
        for i in ("l130", "s23", "m70", "s1"):
            if plan[i] and (k % 3 != 2 or i != "s23"):       # a request may sit out a step
                step.append((i, plan[i].pop(0)))
        k += 1
        if step:
            sched.append(step)
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} in mixed batches")


# ---------------------------------------------------------------- pages and state slots freed and used again
def case_reuse(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=9, max_tokens=160, max_seqs=2)      # five pages, two slots
    reqs = {f"r{j}": tokens(n, FULL["vocab"], 20 + j) for j, n in enumerate([70, 45, 64, 33, 80, 5])}
    want = {i: expect(FULL, W, t) for i, t in reqs.items()}
    sched = ([[("r0", 40), ("r1", 45)], [("r0", 30)]] +                                # r1 ends first, r0 later
             [[("r2", 30), ("r3", 2)], [("r3", 31), ("r2", 1)], [("r2", 33)]] +        # both slots and freed pages again
             [[("r4", 64)], [("r4", 1), ("r5", 5)], [("r4", 15)]])
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} after reuse")
    bm = rig.rep.bm
    assert bm.num_free == bm.num_blocks and bm.num_free_state_slots == 2


# ---------------------------------------------------------------- window edges: one token inside / outside must show
def _peaky(Wt):
    for k in Wt:
        if k.endswith("mix.temp"):
            Wt[k] = torch.full_like(Wt[k], 7.0)
        if k.endswith("mix.r1"):
            Wt[k] = Wt[k] * 0.05


def case_window_edges(tmp, device, dtype, heads=4, kv_heads=2):
    layer = copy.deepcopy(ATTN)
    layer["mixer"].update(heads=heads, kv_heads=kv_heads)
    layer["mixer"]["mask"]["size"] = 33                       # crosses a 32-token page by one
    cfg = make_cfg([layer, layer], width=64)
    W, rig = _setup(tmp, cfg, dtype, device, seed=11, edit=_peaky)
    toks = tokens(120, cfg["vocab"], 3)
    want = expect(cfg, W, toks)
    # the oracle itself must tell a window that is one token off in either direction, or the test shows nothing
    for off in (-1, 1):
        other = copy.deepcopy(cfg)
        for l in other["layers"]:
            l["mixer"]["mask"]["size"] += off
        assert rel_err(expect(other, W, toks)[40:], want[40:]) > 5 * TOL[dtype]
    got = rig.run({"p": toks}, alone("p", 120, [120]))["p"]
    _check(got, want, dtype, "window in a prompt")
    got = rig.run({"d": toks}, alone("d", 120, [30, 1, 1, 1, 1, 1, 1, 2, 31] + [1] * 60))["d"]
    _check(got, want, dtype, "window passing over decoded tokens")


# ---------------------------------------------------------------- a key far back among hundreds
def case_far_key(tmp, device, dtype):
    lat = copy.deepcopy(LATENT)
    lat["mixer"]["scale"] = 1.5                               # peaked softmax: single keys carry weight
    cfg = make_cfg([lat, LIGHT, lat], width=64)
    W, rig = _setup(tmp, cfg, dtype, device, seed=13)
    toks = tokens(330, cfg["vocab"], 4)
    want = expect(cfg, W, toks)
    changed = list(toks)
    changed[1] = (toks[1] + 17) % cfg["vocab"]
    assert rel_err(expect(cfg, W, changed)[-20:], want[-20:]) > 5 * TOL[dtype]       # position 1 reaches the last rows
    got = rig.run({"p": toks}, alone("p", 330, [300] + [1] * 30))["p"]
    _check(got, want, dtype, "far keys, prompt then decoding")
    got = rig.run({"c": toks}, alone("c", 330, [64, 63, 2, 129]))["c"]
    _check(got, want, dtype, "far keys, portions")


# ---------------------------------------------------------------- first tokens, very short requests, long decoding
def case_first_tokens_and_long_decode(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=15)
    for n in (1, 2, 3):
        toks = tokens(n, FULL["vocab"], 30 + n)
        got = rig.run({"x": toks}, alone("x", n, [1]))["x"]
        _check(got, expect(FULL, W, toks), dtype, f"{n}-token request")
    toks = tokens(190, FULL["vocab"], 5)
    got = rig.run({"long": toks}, alone("long", 190, [20] + [1] * 170))["long"]
    _check(got, expect(FULL, W, toks), dtype, "170 decoded tokens")


# ---------------------------------------------------------------- other sizes
def other_size_configs():
    a = copy.deepcopy(ATTN)
    a["mixer"].update(heads=3, kv_heads=3, dim=40, vdim=72, mask={"size": 200})            # window longer than the prompt
    a1 = copy.deepcopy(ATTN)
    a1["mixer"].update(heads=1, kv_heads=1, dim=16, vdim=16, mask={"size": 1})             # sees only itself
    a1["mlp"] = None
    l1 = copy.deepcopy(LIGHT)
    l1["mixer"].update(heads=1, dim=72, vdim=8, decay=[1.0])
    l2 = copy.deepcopy(LIGHT)
    l2["mixer"].update(heads=2, dim=8, vdim=136, decay=[0.3, 0.9])
    l2["mlp"] = None
    m1 = copy.deepcopy(LATENT)
    m1["mixer"].update(heads=5, dim=8, rot_dim=4, vdim=8, kv_rank=24, rot={"base": 100.0, "dims": 4})
    m1["mlp"] = {"kind": "dense", "ff": 40}
    m2 = copy.deepcopy(LATENT)
    m2["mixer"].update(heads=1, dim=32, rot_dim=16, vdim=64, kv_rank=80, rot={"base": 1e6, "dims": 2})
    wide = copy.deepcopy(LATENT)
    wide["mixer"].update(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=528, rot={"base": 1000.0, "dims": 8})   # latent wider than 512
    tall = copy.deepcopy(LIGHT)
    tall["mixer"].update(heads=1, dim=264, vdim=8, decay=[0.97])                                                # more than 256 state rows
    many = copy.deepcopy(LATENT)
    many["mixer"].update(heads=17, dim=8, rot_dim=8, vdim=16, kv_rank=32, rot={"base": 300.0, "dims": 6})      # two groups of heads
    fan = copy.deepcopy(ATTN)
    fan["mixer"].update(heads=8, kv_heads=1, dim=16, vdim=32, mask={"size": 45})                                  # eight query heads on one key head
    fan2 = copy.deepcopy(ATTN)
    fan2["mixer"].update(heads=24, kv_heads=2, dim=8, vdim=16, mask={"size": 9})
    return {
        "many query heads per key head": make_cfg([fan, fan2], width=64, vocab=90, loop=(0, 1, 2)),
        "seventeen latent heads": make_cfg([many, LIGHT], width=64, vocab=77),
        "wide latent, tall state": make_cfg([wide, tall], width=40, vocab=50),
        "square heads, long window": make_cfg([a, l1], width=88, vocab=97, mult=1.0, cap=None),
        "single heads, whole stack three times": make_cfg([a1, m2, l2], width=48, vocab=130, loop=(0, 3, 3), eps=1e-3),
        "loop at the end": make_cfg([m1, l2, a], width=54, vocab=64, loop=(2, 3, 2), mult=0.1, cap=3.0),
    }


def case_other_sizes(tmp, device, dtype, name):
    cfg = other_size_configs()[name]
    W, rig = _setup(tmp, cfg, dtype, device, seed=17)
    toks = tokens(75, cfg["vocab"], 6)
    want = expect(cfg, W, toks)
    _check(rig.run({"w": toks}, alone("w", 75, [75]))["w"], want, dtype, name + " whole")
    _check(rig.run({"c": toks}, alone("c", 75, [2, 30, 1, 1, 33, 1]))["c"], want, dtype, name + " portions")


# ---------------------------------------------------------------- greedy generation through the engine's own entry point
def case_generate(tmp, device, dtype, graphs=False):
    from dli_amd.config import CacheConfig, EngineConfig, SamplingParams, SchedulerConfig, resolve_model
    from dli_amd.engine.engine import LLMEngine
    W = write_checkpoint(tmp, FULL, 19, bf16=dtype == "bfloat16")
    mcfg, wpath = resolve_model(str(tmp), dtype)
    # with graphs: room for the start-up self-test's synthetic mixed step (5 decode rows + a 40-token prompt)
    seqs, lens = (8, (5, 61, 30, 90, 2, 17, 33, 64, 1, 45, 8)) if graphs else (3, (5, 61, 30, 90, 2))
    eng = LLMEngine(EngineConfig(model=mcfg, weights_path=wpath, device=device, cache=CacheConfig(num_blocks=8 * seqs),
                                 sched=SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=64, max_model_len=256,
                                                       long_prefill_chunk=40, token_alignment=0),
                                 use_hip_graphs=graphs, graph_batch_sizes=(1, 2, 4, 8), tune_gemms=False))
    if graphs:
        eng.warmup()
    prompts = [tokens(n, FULL["vocab"], 40 + n) for n in lens]                     # more requests than slots: some wait
    n_new = 12
    outs = eng.generate(None, SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True), prompt_ids=prompts)
    for p, o in zip(prompts, outs):
        assert len(o) == n_new
        seq = list(p)
        for tok in o:                                             # teacher-forced: every generated token is the oracle's argmax
            logits = oracle.forward(FULL, W, seq)[0][-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > (1e-3 if dtype == "float32" else 0.3):   # skip near-ties
                assert int(torch.argmax(logits)) == tok
            seq.append(tok)
    assert eng.bm.num_free == eng.bm.num_blocks and eng.bm.num_free_state_slots == seqs
    if graphs:
        assert eng.runner.stats["graph_steps"] > 0, eng.runner.selftest
    return eng
