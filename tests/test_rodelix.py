"""Rodelix stacks on the CPU path of the ops (fp32 torch references behind the same model, runner, block manager and
engine code as on the GPU) against the plain oracle ``rodelix_oracle``; plus the configuration reader and the state slots
of the block manager.  The GPU kernels run the same cases in ``test_rodelix_gpu.py``."""
import json

import numpy as np
import pytest

import rodelix_cases as cases
from rodelix_common import FULL, write_checkpoint


@pytest.mark.parametrize("kind", ["attention", "lightning", "latent_attention"])
def test_each_mechanism_alone(tmp_path, kind):
    cases.case_mechanism(tmp_path, "cpu", "float32", kind)


def test_prefill_decode_and_portions(tmp_path):
    cases.case_prefill_decode_portions(tmp_path, "cpu", "float32")


def test_unequal_requests_in_one_batch(tmp_path):
    cases.case_mixed_batch(tmp_path, "cpu", "float32")


def test_pages_and_slots_used_again(tmp_path):
    cases.case_reuse(tmp_path, "cpu", "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads", [(4, 2), (8, 1)])
def test_window_edges(tmp_path, heads, kv_heads, dtype):
    cases.case_window_edges(tmp_path, "cpu", dtype, heads, kv_heads)


def test_far_keys(tmp_path):
    cases.case_far_key(tmp_path, "cpu", "float32")



def test_first_tokens_and_long_decoding(tmp_path):
    cases.case_first_tokens_and_long_decode(tmp_path, "cpu", "float32")


@pytest.mark.parametrize("name", sorted(cases.other_size_configs()))
def test_other_sizes(tmp_path, name):
    cases.case_other_sizes(tmp_path, "cpu", "float32", name)


def test_bfloat16_model_on_cpu(tmp_path):
    cases.case_prefill_decode_portions(tmp_path, "cpu", "bfloat16")


def test_greedy_generation_through_the_engine(tmp_path):
    cases.case_generate(tmp_path, "cpu", "float32")


def test_config_reader(tmp_path):
    from dli_amd.config import load_model_config, resolve_model
    write_checkpoint(tmp_path, FULL, 1)
    cfg = load_model_config(str(tmp_path))
    assert cfg.arch == "rodelix" and cfg.hidden_size == FULL["width"] and cfg.vocab_size == FULL["vocab"]
    assert [s.kind for s in cfg.layer_specs] == [l["type"] for l in FULL["layers"]]
    assert [i for i, _ in cfg.layer_runs] == [0, 1, 2, 1, 2, 3] and [r for _, r in cfg.layer_runs] == [False] * 3 + [True] + [False] * 2
    assert cfg.layer_specs[0].window == 37 and cfg.layer_specs[2].rot_dims == 8 and cfg.layer_specs[2].ff == 0
    assert cfg.layer_specs[1].decay == (0.55, 0.93, 0.999) and cfg.stateful
    got, weights = resolve_model(str(tmp_path), "float32")
    assert weights == str(tmp_path) and got.dtype == "float32"
    bad = dict(FULL, architecture="Nonesuch")
    (tmp_path / "config.json").write_text(json.dumps(bad))
    with pytest.raises(ValueError):
        load_model_config(str(tmp_path))


def test_state_slots_of_the_block_manager():
    from dli_amd.runtime.block_manager import BlockManager
    bm = BlockManager(8, 32, False, 2)
    assert bm.allocate(1, 40) and bm.allocate(2, 10)
    assert {bm.state_slot(1), bm.state_slot(2)} == {0, 1}
    free = bm.num_free
    assert not bm.can_allocate(3, 1) and not bm.allocate(3, 1)        # pages are there, no slot is
    assert not bm.has_seq(3) and bm.num_free == free                  # a refused sequence leaves nothing behind
    slot1 = bm.state_slot(1)
    bm.free_seq(1)
    assert bm.allocate(3, 70) and bm.state_slot(3) == slot1
    assert bm.allocate(3, 100) and bm.state_slot(3) == slot1          # growing keeps the slot
    out = np.zeros(2, dtype=np.int32)
    bm.fill_state_slots(np.array([3, 2], dtype=np.int64), out)
    assert out.tolist() == [bm.state_slot(3), bm.state_slot(2)]
    with pytest.raises(RuntimeError):
        bm.fork(3, 9)
    with pytest.raises(ValueError):
        BlockManager(8, 32, True, 2)                                  # shared prefixes cannot carry state
    bm.free_seq(2), bm.free_seq(3)
    assert bm.num_free == 8 and bm.num_free_state_slots == 2
