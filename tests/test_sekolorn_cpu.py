"""Sekolorn on the framework's CPU path (PyTorch ops, fp32) against the plain oracle in
tests/oracles: every mechanism alone, then the whole model through the engine's scheduler
bookkeeping, block manager, state slots and model runner."""

import pytest
import torch

import sekolorn_cases as K
import sekolorn_common as C

DEV, DT = "cpu", torch.float32


@pytest.mark.parametrize("case", [K.case_post_norm, K.case_route, K.case_route_group_limit,
                                  K.case_ungated_moe, K.case_latent_prep,
                                  K.case_latent_attention_needle, K.case_wkv],
                         ids=lambda f: f.__name__)
def test_mechanism(case):
    case(DEV, DT)


def test_latent_attention_more_heads():
    K.case_latent_attention_needle(DEV, DT, 5, 24, 8)


def test_schedules_config_a():
    K.case_schedules(DEV, DT, C.config_a)


def test_schedules_config_b():
    K.case_schedules(DEV, DT, C.config_b, seed=7)


def test_schedules_config_d():
    K.case_schedules(DEV, DT, C.config_d, seed=11)


def test_long_decode():
    K.case_long_decode(DEV, DT)


def test_generate_through_engine():
    K.case_generate(DEV, DT)


def test_generate_config_c():
    K.case_generate(DEV, DT, C.config_c)


def test_state_slots_pool():
    from enterprise_inference_amd.engine.block_manager import StateSlots
    s = StateSlots(3)
    assert [s.acquire(i) for i in (10, 11, 12, 13)] == [0, 1, 2, -1]
    assert s.acquire(11) == 1 and s.num_free() == 0
    s.release(11)
    s.release(10)
    assert s.acquire(14) == 0 and s.acquire(15) == 1 and s.slot_of(12) == 2 and s.slot_of(10) == -1


def test_config_reader(tmp_path):
    """config.json + the checkpoint's header give every size (the decay branch's rank is a
    tensor shape only)."""
    import json

    from safetensors.torch import save_file

    from enterprise_inference_amd.config import ModelConfig
    cfg = C.config_b()
    for L in cfg["layers"]:
        L["mixer"].pop("decay_rank", None)
    W = C.random_weights(C.config_b(), 1)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()},
              str(tmp_path / "model.safetensors"))
    mc = ModelConfig.from_pretrained(str(tmp_path))
    assert mc.architecture == "Sekolorn" and mc.hidden_size == 48 and mc.vocab_size == 70
    assert mc.extra["layers"][1]["mixer"]["decay_rank"] == 6
    assert mc.num_hidden_layers == 2 and mc.layer_norm_eps == 1e-6
