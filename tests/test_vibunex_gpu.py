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


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys(tmp_path, dtype):
    cases.case_far_key(tmp_path, "cuda", dtype)


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
