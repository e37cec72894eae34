"""Vibunex stacks on the gfx950 kernels (``csrc/kernels/dualmix.hip``), fp32 and bf16, against the plain oracle: the
cases of ``vibunex_cases`` on ``cuda``, plus generation with captured decode / mixed-step hipGraphs."""
import pytest
import torch

import vibunex_cases as cases

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(autouse=True)
def _needs_gpu():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from dli_amd import ops
    ops.hip()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["attention", "time_mix", "routed_ff"])
def test_each_mechanism_alone(tmp_path, kind, dtype):
    cases.case_mechanism(tmp_path, "cuda", dtype, kind)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_decode_and_portions(tmp_path, dtype):
    cases.case_prefill_decode_portions(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_requests_in_one_batch(tmp_path, dtype):
    cases.case_mixed_batch(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_chunks_beside_single_tokens_with_heads_of_64(tmp_path, dtype):
    cases.case_mixed_batch_on_tiles(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_and_slots_used_again(tmp_path, dtype):
    cases.case_reuse(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sink_head_mixing_and_rotation_show(tmp_path, dtype):
    cases.case_sink_talk_rotation(tmp_path, "cuda", dtype)


def test_far_keys(tmp_path):
    cases.case_far_key(tmp_path, "cuda", "float32")            # the effect of one far token is below bf16 rounding


def test_first_tokens_and_long_decoding(tmp_path):
    cases.case_first_tokens_and_long_decode(tmp_path, "cuda", "float32")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(cases.other_size_configs()))
def test_other_sizes(tmp_path, name, dtype):
    cases.case_other_sizes(tmp_path, "cuda", dtype, name)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_eager(tmp_path, dtype):
    cases.case_generate(tmp_path, "cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_with_hip_graphs(tmp_path, dtype):
    eng = cases.case_generate(tmp_path, "cuda", dtype, graphs=True)
    st = eng.runner.selftest
    assert st.get("graph_vs_eager", {}).get("ok", True) and st.get("mixed_graph_vs_eager", {}).get("ok", True), st


def test_tiles_against_the_per_token_kernel(tmp_path, monkeypatch):
    """bf16 prompts through the matrix-core tile kernel and through the per-token kernel give the same logits up to the
    rounding of the mixed weights."""
    import numpy as np
    from dli_amd.ops import seqmix
    from rodelix_common import alone, tokens
    cfg = cases.other_size_configs()["matrix-core tiles, heads of 64 in two groups, no feed-forward"]
    W, rig = cases._setup(tmp_path, cfg, "bfloat16", "cuda", seed=23)
    toks = tokens(200, cfg["vocab"], 9)
    tiled = rig.run({"a": toks}, alone("a", 200, [70, 130]))["a"]
    monkeypatch.setattr(seqmix, "TILE_ATTENTION", False)
    plain = rig.run({"b": toks}, alone("b", 200, [70, 130]))["b"]
    assert not np.array_equal(tiled, plain), "both runs took the same kernel"
    cases._check(tiled, plain, "bfloat16", "tile kernel against the per-token kernel", strict=True)
    cases._check(tiled, cases.expect(cfg, W, toks), "bfloat16", "tile kernel against the oracle", strict=True)


def test_grouped_experts_against_the_row_kernels():
    """The routed experts as grouped GEMMs on the matrix cores against the any-shape row kernels, same routing."""
    from dli_amd import ops
    lib = ops.hip()
    torch.manual_seed(1)
    T, W, F, E, K = 300, 256, 384, 7, 3
    h = torch.randn(T, W, device="cuda").bfloat16()
    up = (torch.randn(E, F, W, device="cuda") / W ** 0.5).bfloat16()
    down = (torch.randn(E, W, F, device="cuda") / F ** 0.5).bfloat16()
    ids = torch.stack([torch.randperm(E, device="cuda")[:K] for _ in range(T)]).int()
    wts = torch.rand(T, K, device="cuda")
    try:
        grouped = lib.dm_relu2_experts(h, ids, wts, up, down).float()
        lib.dm_set_grouped_experts(False)
        rows = lib.dm_relu2_experts(h, ids, wts, up, down).float()
    finally:
        lib.dm_set_grouped_experts(True)
    want = torch.zeros(T, W, device="cuda")
    for k in range(K):
        a = torch.relu(torch.einsum("tw,tfw->tf", h.float(), up[ids[:, k].long()].float())) ** 2
        want += wts[:, k:k + 1] * torch.einsum("tf,twf->tw", a.bfloat16().float(), down[ids[:, k].long()].float())
    for got, name in ((grouped, "grouped"), (rows, "rows")):
        err = ((got - want).norm() / want.norm()).item()
        assert err < 1e-2, f"{name}: {err}"
    assert not torch.equal(grouped, rows), "both calls took the same kernels"


class _NamedOps:
    """The kernel library with every call announced (flushed) and finished before the next: a fault then names its op."""

    def __init__(self, lib):
        self._lib = lib

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if not callable(fn):
            return fn

        def call(*a, **k):
            print(f"    op {name}", flush=True)
            out = fn(*a, **k)
            torch.cuda.synchronize()
            return out
        return call


@pytest.mark.skip(reason="a benchmark run of a stack with these layer sizes ended in an illegal memory access after the start-up "
                         "checks had passed; the kernel was not identified, so nothing of that size runs on a GPU until it is")
def test_layer_sizes_of_a_real_model_against_the_cpu_path(tmp_path, monkeypatch):
    """One layer at the sizes of a real model (width 2048, 16 query / 4 key heads of 128, 32 recurrent heads of 64, 8 experts
    of 5632, shared 1024): a 2 × 1100-token prefill step, decode steps of 2 rows and a mixed step, kernels against the CPU
    path of the same ops (which the other tests pin to the oracle)."""
    import numpy as np
    from dli_amd.ops import seqmix
    from rodelix_common import Rig, tokens
    layer = {"type": "parallel",
             "mixer": {"left_scale": 0.7, "right_scale": 0.7,
                       "left": {"heads": 16, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                                "rot": {"base": 1000000.0, "dims": 64, "scaling": {"factor": 8.0, "original": 8192, "fast": 16.0, "slow": 2.0}}},
                       "right": {"heads": 32, "dim": 64, "lora": 64}},
             "mlp": {"kind": "moe", "expert": {"ff": 5632}, "router": {"experts": 8, "top": 2, "scale": 1.0}, "shared": {"ff": 1024}}}
    cfg = cases.make_cfg([layer], width=2048, vocab=512, mult=0.5)
    print("  writing the checkpoint", flush=True)
    cases.write_checkpoint(tmp_path, cfg, seed=31, bf16=True)
    reqs = {"a": tokens(1104, 512, 1), "b": tokens(1103, 512, 2), "c": tokens(70, 512, 3)}
    sched = [[("a", 1100), ("b", 1100)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1), ("c", 70)], [("a", 1), ("b", 1)], [("a", 1)]]
    print("  cpu path", flush=True)
    want = Rig(tmp_path, "bfloat16", "cpu", max_tokens=2560).run(reqs, sched)
    print("  gpu path", flush=True)
    rig = Rig(tmp_path, "bfloat16", "cuda", max_tokens=2560)
    lib = seqmix._hip()
    monkeypatch.setattr(seqmix, "_hip", lambda: _NamedOps(lib))
    got = rig.run(reqs, sched)
    for i in reqs:
        e = cases._row_err(got[i], want[i])
        assert np.median(e) < 2e-2 and (e > 6e-2).mean() < 0.1, f"{i}: median {np.median(e):.3e}, worst {e.max():.3e}"
