"""Vedadra on the framework's CPU path (PyTorch ops, fp32) against the plain oracle in
tests/oracles: every mechanism alone, then the whole model through the engine."""

import pytest
import torch

import vedadra_cases as K
import vedadra_common as C

F32 = torch.float32


@pytest.mark.parametrize("case", [K.case_group_norm, K.case_qk_norm_cache], ids=lambda f: f.__name__)
def test_mechanism(case):
    case("cpu", F32)


@pytest.mark.parametrize("kind,keep", [("talking", 0), ("differential", 0), ("differential", 5)])
def test_window_needle(kind, keep):
    K.case_window_needle("cpu", F32, kind, keep=keep, n=120)


@pytest.mark.parametrize("cfg", [C.config_a, C.config_b, C.config_c], ids=lambda f: f.__name__)
def test_layers(cfg):
    K.case_layers("cpu", F32, cfg)


@pytest.mark.parametrize("cfg", [C.config_a, C.config_b], ids=lambda f: f.__name__)
def test_schedules(cfg):
    K.case_schedules("cpu", F32, cfg)


def test_long_decode():
    K.case_long_decode("cpu", F32)


def test_generate_through_engine():
    K.case_generate("cpu", F32)


def test_config_reader_and_registry():
    from enterprise_inference_amd.config import ModelConfig
    from enterprise_inference_amd.models import get_model_class
    mc = ModelConfig.from_hf_dict(C.config_a())
    assert mc.architecture == "Vedadra" and mc.extra["loop"]["times"] == 3
    assert mc.extra["norm"]["groups"] == 3
    model = get_model_class("Vedadra")(mc, dtype=F32)
    assert [r[0] for r in model.runs] == [0, 1, 0, 1, 0, 1, 2]
    assert [r[1] for r in model.runs] == [False, False, True, False, True, False, False]
    assert len(model.allocate_cache(2, 16, 0, F32, "cpu")) == 7
    with pytest.raises(ValueError):
        model.load_weights([("l0.mix.nonsense", torch.zeros(1))])
