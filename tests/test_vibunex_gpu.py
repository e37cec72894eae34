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
