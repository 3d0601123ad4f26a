"""Sekolorn on the MI355X path (HIP kernels; fp32 and bf16 activations) against the plain oracle
in tests/oracles: every kernel alone, then the whole model through the engine."""

import pytest
import torch

import sekolorn_cases as K
import sekolorn_common as C

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _cfg(fn, dtype):
    """fp32 runs the configuration as it is; bf16 with every expert chosen (C.all_experts)."""
    return fn if dtype == torch.float32 else (lambda: C.all_experts(fn()))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("case", [K.case_post_norm, K.case_route, K.case_route_group_limit,
                                  K.case_ungated_moe, K.case_combine_post_norm, K.case_latent_prep,
                                  K.case_latent_attention_needle, K.case_wkv],
                         ids=lambda f: f.__name__)
def test_kernel(case, dtype):
    case("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(5, 24, 8), (20, 72, 16), (16, 256, 32), (16, 264, 24), (2, 512, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_latent_attention_shapes(shape, dtype):
    """Head counts below, at and above a 16-head slice; latent widths of every MFMA variant
    (bf16 runs the MFMA form at these widths, fp32 the scalar form)."""
    K.case_latent_attention_needle("cuda", dtype, *shape)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(4, 256, 256, 9, 2), (4, 128, 128, 40, 2), (3, 256, 256, 230, 2),
                                   (2, 128, 256, 300, 1)], ids=lambda s: "x".join(map(str, s)))
def test_ungated_moe_forms(shape, dtype):
    """(E, I, H, T, k) that select, in bf16, the grouped weight-streaming form, the grouped MFMA
    form (both without a host read-back) and the per-expert library form."""
    K.case_ungated_moe("cuda", dtype, *shape)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_schedules_config_a(dtype):
    K.case_schedules("cuda", dtype, _cfg(C.config_a, dtype))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_schedules_config_b(dtype):
    K.case_schedules("cuda", dtype, _cfg(C.config_b, dtype), seed=7)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_schedules_config_d(dtype):
    K.case_schedules("cuda", dtype, _cfg(C.config_d, dtype), seed=11)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_schedules_config_e(dtype):
    K.case_schedules("cuda", dtype, _cfg(C.config_e, dtype), seed=13)


def test_generate_graph_decode_config_e():
    K.case_generate("cuda", torch.bfloat16, _cfg(C.config_e, torch.bfloat16), expect_graphs=True)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_long_decode(dtype):
    K.case_long_decode("cuda", dtype, _cfg(C.config_b, dtype))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_generate_through_engine(dtype):
    K.case_generate("cuda", dtype, _cfg(C.config_a, dtype))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_generate_graph_decode(dtype):
    """A graph-eligible configuration: the bf16 engine captures decode graphs (state slots and
    block tables are read from the graph's header on every replay); every decoded token of
    every replay is checked against the oracle."""
    K.case_generate("cuda", dtype, _cfg(C.config_c, dtype), expect_graphs=dtype == torch.bfloat16)


def test_native_library_loaded():
    from enterprise_inference_amd import _native
    _native.kernels()
    assert any("libeia_kernels.so" in p for p in _native.loaded_native_libraries())
