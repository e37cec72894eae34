"""Vibunex stacks on the CPU path of the ops (fp32 torch references behind the same model, runner, block manager and
engine code as on the GPU) against the plain oracle ``vibunex_oracle``; plus the configuration reader and single ops
against the oracle's functions.  The GPU kernels run the same cases in ``test_vibunex_gpu.py``."""
import math

import pytest
import torch

import vibunex_cases as cases
import vibunex_oracle as oracle


@pytest.mark.parametrize("kind", ["attention", "time_mix", "routed_ff"])
def test_each_mechanism_alone(tmp_path, kind):
    cases.case_mechanism(tmp_path, "cpu", "float32", kind)


def test_prefill_decode_and_portions(tmp_path):
    cases.case_prefill_decode_portions(tmp_path, "cpu", "float32")


def test_unequal_requests_in_one_batch(tmp_path):
    cases.case_mixed_batch(tmp_path, "cpu", "float32")


def test_chunks_beside_single_tokens_with_heads_of_64(tmp_path):
    cases.case_mixed_batch_on_tiles(tmp_path, "cpu", "float32")


def test_pages_and_slots_used_again(tmp_path):
    cases.case_reuse(tmp_path, "cpu", "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sink_head_mixing_and_rotation_show(tmp_path, dtype):
    cases.case_sink_talk_rotation(tmp_path, "cpu", dtype)


def test_far_keys(tmp_path):
    cases.case_far_key(tmp_path, "cpu", "float32")


def test_first_tokens_and_long_decoding(tmp_path):
    cases.case_first_tokens_and_long_decode(tmp_path, "cpu", "float32")


@pytest.mark.parametrize("name", sorted(cases.other_size_configs()))
def test_other_sizes(tmp_path, name):
    cases.case_other_sizes(tmp_path, "cpu", "float32", name)


def test_greedy_generation_through_the_engine(tmp_path):
    cases.case_generate(tmp_path, "cpu", "float32")


def test_config_reader(tmp_path):
    from dli_amd.config import get_model_config, load_model_config, resolve_model
    cases.write_checkpoint(tmp_path, cases.FULL, 1)
    cfg = load_model_config(str(tmp_path), "float32")
    assert cfg.arch == "vibunex" and cfg.stateful and len(cfg.layer_specs) == 3
    s = cfg.layer_specs[0]
    assert s.kind == "parallel" and [p.kind for p in s.parts] == ["sink_attention", "time_mix"]
    assert s.parts[1].lora == 6                                # from the tensor's shape: the stored configuration has no rank
    assert s.parts[0].rot_scaling == (3.0, 48.0, 8.0, 2.0) and s.part_scales == (0.7, 1.1)
    assert (s.experts, s.top, s.ff, s.shared_ff, s.router_scale) == (5, 2, 40, 56, 1.7)
    assert cfg.layer_specs[1].ff == 0 and cfg.layer_specs[1].parts[0].rot_scaling == ()
    assert s.cache_row == (3 * 24, 3 * 16) and s.state_shape == (3, 20, 20)
    assert resolve_model(str(tmp_path))[1] == str(tmp_path)
    assert get_model_config("tiny-vibunex").arch == "vibunex"


def test_stretched_frequencies_against_the_oracle():
    from dli_amd.ops import seqmix
    for rot in ({"base": 8000.0, "dims": 12, "scaling": {"factor": 3.0, "original": 48, "fast": 8.0, "slow": 2.0}},
                {"base": 500.0, "dims": 32, "scaling": {"factor": 16.0, "original": 4096, "fast": 24.0, "slow": 1.5}},
                {"base": 10000.0, "dims": 6}):
        want, mag = oracle.stretched_frequencies(rot)
        sc = rot.get("scaling")
        got, gmag = seqmix.stretched_inv_freq(rot["base"], rot["dims"], (sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else ())
        assert torch.allclose(got, torch.tensor(want, dtype=torch.float64), rtol=1e-12) and math.isclose(mag, gmag)


def test_router_picks_and_weights_against_the_oracle():
    from dli_amd.ops import seqmix
    torch.manual_seed(0)
    h, R = torch.randn(40, 24), torch.randn(9, 24)
    R[3] = R[1]                                               # a tie: the lower index wins
    ids, wts, extra = seqmix.sigmoid_route(h, R, 8, 3, 2.0)
    s = torch.sigmoid(h.double() @ R.double().t())
    for t in range(40):
        order = sorted(range(8), key=lambda e: -float(s[t, e]))[:3]
        assert ids[t].tolist() == order
        assert torch.allclose(wts[t].double(), s[t, order] * 2.0, atol=1e-6)
    assert torch.allclose(extra.double(), s[:, 8], atol=1e-6)
