"""Vedadra on the MI355X path (HIP kernels; fp32 and bf16 activations) against the plain oracle
in tests/oracles: every kernel alone, then the whole model through the engine."""

import pytest
import torch

import vedadra_cases as K
import vedadra_common as C

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
IDS = ["fp32", "bf16"]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("case", [K.case_group_norm, K.case_qk_norm_cache], ids=lambda f: f.__name__)
def test_kernel(case, dtype):
    case("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [
    # kind, H, G, D, Dv, window, kept first tokens, tokens, page
    ("talking", 4, 2, 16, 16, 40, 0, 150, 16),
    ("talking", 1, 1, 24, 24, 7, 0, 90, 16),
    ("talking", 8, 2, 64, 64, 130, 0, 300, 64),
    ("talking", 16, 4, 128, 128, 200, 0, 420, 64),
    ("differential", 4, 1, 16, 24, 40, 5, 150, 16),
    ("differential", 2, 2, 10, 6, 3, 0, 80, 16),
    ("differential", 4, 2, 32, 64, 64, 4, 300, 64),
    ("differential", 8, 2, 64, 128, 150, 6, 400, 64),
    # bf16: the matrix-core form's variants (1, 2, 4 heads per wave; partial last wave; head sizes
    # that are not multiples of 32; 32-token pages; kept tokens beyond one 32-key block)
    ("talking", 3, 1, 80, 80, 70, 0, 260, 64),
    ("talking", 6, 3, 48, 48, 33, 0, 200, 32),
    ("talking", 12, 4, 32, 32, 100, 0, 300, 32),
    ("talking", 2, 2, 128, 128, 31, 0, 130, 32),
    ("talking", 8, 8, 64, 64, 50, 0, 200, 32),
    ("talking", 16, 16, 32, 32, 50, 0, 200, 32),
    ("talking", 16, 16, 128, 128, 50, 0, 140, 32),
    ("differential", 5, 1, 40, 80, 44, 7, 260, 64),
    ("differential", 1, 1, 24, 16, 64, 40, 300, 32),
    ("differential", 3, 3, 128, 112, 90, 33, 350, 64),
], ids=lambda s: "-".join(map(str, s)))
def test_window_needle(shape, dtype):
    kind, H, G, D, Dv, size, keep, n, bs = shape
    K.case_window_needle("cuda", dtype, kind, H, G, D, Dv, size, keep, n, bs)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("cfg", [C.config_a, C.config_b, C.config_c], ids=lambda f: f.__name__)
def test_layers(cfg, dtype):
    K.case_layers("cuda", dtype, cfg)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("cfg", [C.config_a, C.config_b, C.config_c], ids=lambda f: f.__name__)
def test_schedules(cfg, dtype):
    K.case_schedules("cuda", dtype, cfg, seed=7)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_schedules_pages_of_32(dtype):
    """Pages of 32 tokens: the bf16 run takes the matrix-core attention form end to end."""
    K.case_schedules("cuda", dtype, C.config_c, seed=3, block_size=32)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_long_decode(dtype):
    K.case_long_decode("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_generate_through_engine(dtype):
    K.case_generate("cuda", dtype, C.config_a, expect_graphs=True)


def test_generate_graph_decode_config_c():
    K.case_generate("cuda", torch.bfloat16, C.config_c, expect_graphs=True)


@pytest.mark.parametrize("shape", [(1, 2048, 1024), (32, 4096, 1024), (7, 512, 256), (48, 8192, 2048)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gated_gelu_gemm(shape):
    """The decode-sized [gate; up] GEMM with the tanh form of GELU in its epilogue (or, where it
    splits K, in the reduce kernel) against the plain fp32 product."""
    from enterprise_inference_amd.models.layers import MergedColumnParallelLinear
    M, I, K = shape
    g = torch.Generator().manual_seed(M + I)
    lin = MergedColumnParallelLinear(K, [I, I], dtype=torch.bfloat16, device="cuda")
    lin.weight.data.copy_((torch.randn(2 * I, K, generator=g) * K ** -0.5).to(torch.bfloat16))
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).cuda()
    got = lin.forward_act_and_mul(x, "gelu_tanh").float().cpu()
    y = x.float().cpu() @ lin.weight.float().cpu().t()
    want = torch.nn.functional.gelu(y[:, :I], approximate="tanh") * y[:, I:]
    assert torch.allclose(got, want, atol=2e-2, rtol=2e-2), float((got - want).abs().max())


def test_native_library_loaded():
    from enterprise_inference_amd import _native
    lib = _native.kernels()
    assert hasattr(lib, "eia_window_attn") and hasattr(lib, "eia_gnorm")
    assert any("libeia_kernels" in p for p in _native.loaded_native_libraries())
