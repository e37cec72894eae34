"""The Vibunex test cases, parametrised by device and dtype.  Each case builds its own small configuration, writes a
checkpoint from the plain oracle's random weights (``vibunex_oracle``), replays step schedules through the engine
(``rodelix_common.Rig``: the engine's runner, block manager, cache, state slots and kernels) and compares every position's
logits with the oracle.  The same cases run on the CPU path (``test_vibunex.py``) and on the GPU kernels
(``test_vibunex_gpu.py``)."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

import vibunex_oracle as oracle
from rodelix_common import Rig, TOL, alone, chunks, rel_err, tokens

LAYER = {"type": "parallel",
         "mixer": {"left_scale": 0.7, "right_scale": 1.1,
                   "left": {"heads": 6, "kv_heads": 3, "dim": 24, "vdim": 16, "scale": 0.3,
                            "rot": {"base": 8000.0, "dims": 12, "scaling": {"factor": 3.0, "original": 48, "fast": 8.0, "slow": 2.0}}},
                   "right": {"heads": 3, "dim": 20, "lora": 6}},
         "mlp": {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 5, "top": 2, "scale": 1.7}, "shared": {"ff": 56}}}
LAYER_B = {"type": "parallel",
           "mixer": {"left_scale": 1.2, "right_scale": 0.4,
                     "left": {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 40, "scale": 0.5, "rot": {"base": 300.0, "dims": 16}},
                     "right": {"heads": 2, "dim": 36, "lora": 9}},
           "mlp": None}


def make_cfg(layers, width=72, vocab=157, mult=0.4, eps=1e-5):
    return {"architecture": "Vibunex", "vocab": vocab, "width": width, "residual_mult": mult, "norm": {"eps": eps},
            "layers": [copy.deepcopy(l) for l in layers]}


FULL = make_cfg([LAYER, LAYER_B, LAYER])


def write_checkpoint(path, cfg, seed=0, bf16=False, edit=None):
    """config.json (without the decay rank: the product takes it from the tensor's shape) + model.safetensors; returns the
    weights as stored (fp32 values) for the oracle."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    W = oracle.random_weights(cfg, seed)
    if edit:
        edit(W)
    if bf16:
        W = {k: v.to(torch.bfloat16) for k, v in W.items()}
    stored = copy.deepcopy(cfg)
    for l in stored["layers"]:
        l["mixer"]["right"].pop("lora", None)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(stored, fh)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return {k: v.float() for k, v in W.items()}


def expect(cfg, W, toks):
    return oracle.forward(cfg, W, toks)[0].numpy()


def _setup(tmp, cfg, dtype, device, seed=0, edit=None, **rig):
    W = write_checkpoint(tmp, cfg, seed, bf16=dtype == "bfloat16", edit=edit)
    return W, Rig(tmp, dtype, device, **rig)


def _row_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


def _check(got, want, dtype, what="", strict=False):
    """fp32: every row within the tolerance.  bf16: rounding moves a token whose router scores nearly tie to another expert
    now and then (that row, and less so the rows after it, then differ by far more than rounding), so the bound holds for
    the bulk of the rows: the median well inside it and at most one row in seven outside; what a cut, a page or a slot can
    break shows in the fp32 run of the same case on the same templated kernels."""
    e = _row_err(got, want)
    if dtype == "float32" or strict:                          # strict: a stack without a router has no such rows
        assert e.max() < TOL[dtype], f"{what}: relative error {e.max():.3e} over {TOL[dtype]:.1e}"
    else:
        assert np.median(e) < TOL[dtype] / 4 and (e > TOL[dtype]).mean() <= 1 / 7, \
            f"{what}: median {np.median(e):.3e}, {(e > TOL[dtype]).mean():.0%} of the rows over {TOL[dtype]:.1e}"


# ---------------------------------------------------------------- each mechanism alone
def case_mechanism(tmp, device, dtype, kind):
    layer = copy.deepcopy(LAYER)
    if kind == "attention":
        layer["mixer"]["right_scale"], layer["mlp"] = 0.0, None
    elif kind == "time_mix":
        layer["mixer"]["left_scale"], layer["mlp"] = 0.0, None
    else:                                                     # the routed feed-forward: both mixers silenced
        layer["mixer"]["left_scale"] = layer["mixer"]["right_scale"] = 0.0
    cfg = make_cfg([layer, layer], width=64)
    W, rig = _setup(tmp, cfg, dtype, device, seed=3)
    toks = tokens(110, cfg["vocab"], 1)
    want = expect(cfg, W, toks)
    _check(rig.run({"a": toks}, alone("a", len(toks), [len(toks)]))["a"], want, dtype, f"{kind} whole prompt")
    _check(rig.run({"b": toks}, alone("b", len(toks), [31, 2, 1, 40, 1, 1, 7]))["b"], want, dtype, f"{kind} in portions")


# ---------------------------------------------------------------- prefill against token-by-token, portions down to two
def case_prefill_decode_portions(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=5)
    toks = tokens(100, FULL["vocab"], 2)
    want = expect(FULL, W, toks)
    for name, sizes in (("whole", [100]), ("one by one", [1]), ("portions", [2, 3, 64, 5, 2, 17]), ("page edges", [32, 32, 1, 31, 4])):
        _check(rig.run({name: toks}, alone(name, len(toks), sizes))[name], want, dtype, name)


# ---------------------------------------------------------------- unequal requests in one batch against each alone
def case_mixed_batch(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=7, max_tokens=512)
    reqs = {"s1": tokens(1, FULL["vocab"], 10), "s23": tokens(23, FULL["vocab"], 11), "m70": tokens(70, FULL["vocab"], 12),
            "l130": tokens(130, FULL["vocab"], 13)}
    want = {i: expect(FULL, W, t) for i, t in reqs.items()}
    plan = {"s1": [1], "s23": [2, 1, 1, 16, 1, 1, 1], "m70": chunks(70, [33, 1, 1, 2, 1]), "l130": chunks(130, [40, 3, 1, 1, 64, 1])}
    sched, k = [], 0
    while any(plan.values()):
        step = [(i, plan[i].pop(0)) for i in ("l130", "s23", "m70", "s1") if plan[i] and (k % 3 != 2 or i != "s23")]
        k += 1
        if step:
            sched.append(step)
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} in mixed batches")


def case_mixed_batch_on_tiles(tmp, device, dtype):
    """Chunks of two sequences beside decode rows of others in one step, with heads of 64 (on the GPU in bf16: the chunks
    take the matrix-core tile kernel, the single tokens the per-token kernel)."""
    cfg = other_size_configs()["matrix-core tiles, heads of 64 in two groups, no feed-forward"]
    W, rig = _setup(tmp, cfg, dtype, device, seed=21, max_tokens=640)
    reqs = {"a": tokens(150, cfg["vocab"], 50), "b": tokens(97, cfg["vocab"], 51), "c": tokens(40, cfg["vocab"], 52),
            "d": tokens(3, cfg["vocab"], 53)}
    want = {i: expect(cfg, W, t) for i, t in reqs.items()}
    sched = [[("a", 70), ("c", 33)], [("a", 1), ("b", 64), ("c", 1), ("d", 1)], [("a", 50), ("b", 1), ("c", 1), ("d", 2)],
             [("a", 1), ("b", 32), ("c", 5)], [("a", 28)]]
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} beside the others", strict=True)


# ---------------------------------------------------------------- pages and state slots freed and used again
def case_reuse(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=9, max_tokens=160, max_seqs=2)      # five pages, two slots
    reqs = {f"r{j}": tokens(n, FULL["vocab"], 20 + j) for j, n in enumerate([70, 45, 64, 33, 80, 5])}
    want = {i: expect(FULL, W, t) for i, t in reqs.items()}
    sched = ([[("r0", 40), ("r1", 45)], [("r0", 30)]] +
             [[("r2", 30), ("r3", 2)], [("r3", 31), ("r2", 1)], [("r2", 33)]] +
             [[("r4", 64)], [("r4", 1), ("r5", 5)], [("r4", 15)]])
    got = rig.run(reqs, sched)
    for i in reqs:
        _check(got[i], want[i], dtype, f"request {i} after reuse")
    bm = rig.rep.bm
    assert bm.num_free == bm.num_blocks and bm.num_free_state_slots == 2


# ---------------------------------------------------------------- sink, head mixing, rotation: leaving one out must show
def _loud_sink(Wt):
    for k in Wt:
        if k.endswith("left.sink"):
            Wt[k] = Wt[k] + 3.0                               # the sink takes a large share of every softmax


def case_sink_talk_rotation(tmp, device, dtype):
    cfg = make_cfg([LAYER, LAYER], width=64)
    W, rig = _setup(tmp, cfg, dtype, device, seed=11, edit=_loud_sink)
    toks = tokens(90, cfg["vocab"], 3)
    want = expect(cfg, W, toks)
    # the oracle itself must tell these faults, or the test shows nothing
    no_sink = {k: (v - 60.0 if k.endswith("left.sink") else v) for k, v in W.items()}
    no_talk = {k: (torch.eye(v.shape[0]) if k.endswith("left.talk") else v) for k, v in W.items()}
    plain = copy.deepcopy(cfg)
    for l in plain["layers"]:
        del l["mixer"]["left"]["rot"]["scaling"]
    for name, other in (("sink", expect(cfg, no_sink, toks)), ("head mixing", expect(cfg, no_talk, toks)),
                        ("stretched frequencies", expect(plain, W, toks))):
        if dtype == "float32":
            assert rel_err(other[8:], want[8:]) > 5 * TOL[dtype], name
        elif name != "stretched frequencies":                 # bf16: the two large effects stand clear of its rounding
            assert rel_err(other[8:], want[8:]) > 2 * TOL[dtype], name
    _check(rig.run({"p": toks}, alone("p", 90, [90]))["p"], want, dtype, "prompt")
    _check(rig.run({"d": toks}, alone("d", 90, [30, 2, 31] + [1] * 27))["d"], want, dtype, "portions and decoding")


# ---------------------------------------------------------------- a key far back among hundreds; memory of the recurrence
def _far_edit(Wt):
    for k in list(Wt):
        if k.endswith("left.q") or k.endswith("left.k"):
            Wt[k] = Wt[k] * 2.5                               # peaked softmax: single keys carry weight
        if k.endswith("left.sink"):
            Wt[k] = Wt[k] - 4.0
        if k.endswith("right.w0"):
            Wt[k] = Wt[k] - 5.0                               # decay close to one: the state remembers the first tokens


def case_far_key(tmp, device, dtype):
    layer = copy.deepcopy(LAYER)
    layer["mixer"]["left"]["scale"] = 1.0
    for which in ("left_scale", "right_scale"):               # each mixer alone must carry position 1 to the end
        cfg = make_cfg([layer, layer], width=64)
        for l in cfg["layers"]:
            l["mixer"]["right_scale" if which == "left_scale" else "left_scale"] = 0.0
        sub = os.path.join(str(tmp), which)
        W, rig = _setup(sub, cfg, dtype, device, seed=13, edit=_far_edit)
        toks = tokens(330, cfg["vocab"], 4)
        want = expect(cfg, W, toks)
        changed = list(toks)
        changed[1] = (toks[1] + 17) % cfg["vocab"]
        assert rel_err(expect(cfg, W, changed)[-20:], want[-20:]) > 5 * TOL[dtype], which
        _check(rig.run({"p": toks}, alone("p", 330, [300] + [1] * 30))["p"], want, dtype, f"far keys ({which}), prompt then decoding")
        _check(rig.run({"c": toks}, alone("c", 330, [64, 63, 2, 129]))["c"], want, dtype, f"far keys ({which}), portions")


# ---------------------------------------------------------------- first tokens, very short requests, long decoding
def case_first_tokens_and_long_decode(tmp, device, dtype):
    W, rig = _setup(tmp, FULL, dtype, device, seed=15)
    for n in (1, 2, 3):
        toks = tokens(n, FULL["vocab"], 30 + n)
        _check(rig.run({"x": toks}, alone("x", n, [1]))["x"], expect(FULL, W, toks), dtype, f"{n}-token request")
    toks = tokens(190, FULL["vocab"], 5)
    _check(rig.run({"long": toks}, alone("long", 190, [20] + [1] * 170))["long"], expect(FULL, W, toks), dtype, "170 decoded tokens")


# ---------------------------------------------------------------- other sizes
def other_size_configs():
    def layer(left, right, mlp, ls=0.9, rs=0.8):
        return {"type": "parallel", "mixer": {"left_scale": ls, "right_scale": rs, "left": left, "right": right}, "mlp": mlp}

    square = layer({"heads": 3, "kv_heads": 3, "dim": 40, "vdim": 8, "scale": 0.2, "rot": {"base": 100.0, "dims": 40}},
                   {"heads": 1, "dim": 72, "lora": 3},
                   {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 3, "top": 1, "scale": 1.0}, "shared": None})
    single = layer({"heads": 1, "kv_heads": 1, "dim": 16, "vdim": 64, "scale": 1.0,
                    "rot": {"base": 1e6, "dims": 2, "scaling": {"factor": 8.0, "original": 16, "fast": 4.0, "slow": 1.0}}},
                   {"heads": 5, "dim": 8, "lora": 1},
                   {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 7, "top": 7, "scale": 0.3}, "shared": {"ff": 8}}, 1.0, 1.0)
    fan = layer({"heads": 16, "kv_heads": 2, "dim": 8, "vdim": 24, "scale": 0.35, "rot": {"base": 5000.0, "dims": 4}},
                {"heads": 2, "dim": 100, "lora": 20},
                {"kind": "moe", "expert": {"ff": 130}, "router": {"experts": 12, "top": 3, "scale": 2.0}, "shared": {"ff": 16}})
    norot = layer({"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 32, "scale": 0.18, "rot": {"base": 10000.0, "dims": 0}},
                  {"heads": 4, "dim": 16, "lora": 5}, None)
    tile64 = layer({"heads": 20, "kv_heads": 5, "dim": 64, "vdim": 64, "scale": 0.15,
                    "rot": {"base": 1e4, "dims": 32, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}},
                   {"heads": 2, "dim": 64, "lora": 8}, None)
    tile128 = layer({"heads": 4, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 0.1, "rot": {"base": 1e4, "dims": 64}},
                    {"heads": 1, "dim": 128, "lora": 8}, None)
    grouped = layer({"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.15, "rot": {"base": 1e4, "dims": 16}},
                    {"heads": 2, "dim": 32, "lora": 4},
                    {"kind": "moe", "expert": {"ff": 128}, "router": {"experts": 6, "top": 2, "scale": 1.2}, "shared": {"ff": 64}})
    return {
        "matrix-core tiles, heads of 64 in two groups, no feed-forward": make_cfg([tile64, tile64], width=96, vocab=80),
        "matrix-core tiles, heads of 128, one query head per key head, no feed-forward": make_cfg([tile128], width=64, vocab=70),
        "experts as grouped products": make_cfg([grouped, grouped], width=128, vocab=90),
        "square heads, one expert of three, no shared expert": make_cfg([square, LAYER_B], width=88, vocab=97, mult=1.0),
        "single heads, every expert chosen": make_cfg([single, single], width=48, vocab=130, eps=1e-3),
        "eight query heads per key head, wide recurrence": make_cfg([fan, norot], width=56, vocab=64, mult=0.2),
        "no rotation, no feed-forward": make_cfg([norot], width=40, vocab=50),
    }


def case_other_sizes(tmp, device, dtype, name):
    cfg = other_size_configs()[name]
    W, rig = _setup(tmp, cfg, dtype, device, seed=17)
    toks = tokens(75, cfg["vocab"], 6)
    want = expect(cfg, W, toks)
    strict = not any(l.get("mlp") for l in cfg["layers"])
    _check(rig.run({"w": toks}, alone("w", 75, [75]))["w"], want, dtype, name + " whole", strict)
    _check(rig.run({"c": toks}, alone("c", 75, [2, 30, 1, 1, 33, 1]))["c"], want, dtype, name + " portions", strict)
    if "matrix-core" in name:                                 # tiles that start inside a page, with hundreds of keys behind them
        toks = tokens(300, cfg["vocab"], 8)
        want = expect(cfg, W, toks)
        _check(rig.run({"l": toks}, alone("l", 300, [45, 130, 17, 64, 43, 1]))["l"], want, dtype, name + " long portions", strict)


# ---------------------------------------------------------------- greedy generation through the engine's own entry point
def case_generate(tmp, device, dtype, graphs=False):
    from dli_amd.config import CacheConfig, EngineConfig, SamplingParams, SchedulerConfig, resolve_model
    from dli_amd.engine.engine import LLMEngine
    W = write_checkpoint(tmp, FULL, 19, bf16=dtype == "bfloat16")
    mcfg, wpath = resolve_model(str(tmp), dtype)
    seqs, lens = (8, (5, 61, 30, 90, 2, 17, 33, 64, 1, 45, 8)) if graphs else (3, (5, 61, 30, 90, 2))
    eng = LLMEngine(EngineConfig(model=mcfg, weights_path=wpath, device=device, cache=CacheConfig(num_blocks=8 * seqs),
                                 sched=SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=64, max_model_len=256,
                                                       long_prefill_chunk=40, token_alignment=0),
                                 use_hip_graphs=graphs, graph_batch_sizes=(1, 2, 4, 8), tune_gemms=False))
    if graphs:
        eng.warmup()
    prompts = [tokens(n, FULL["vocab"], 40 + n) for n in lens]                     # more requests than slots: some wait
    n_new = 10
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
