"""Gapidra on the MI355X path (HIP kernels; fp32 and bf16 activations) against the plain oracle
in tests/oracles: every kernel alone, then the whole model through the engine."""

import pytest
import torch

import gapidra_cases as K
import gapidra_common as C

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
IDS = ["fp32", "bf16"]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("case", [K.case_residual_rms_step, K.case_xielu, K.case_sigmoid_gate,
                                  K.case_qk_rope_cache, K.case_latent_prep],
                         ids=lambda f: f.__name__)
def test_kernel(case, dtype):
    case("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [
    # H, G, D, Dv, window, tokens, page
    (4, 2, 16, 8, 40, 150, 16),
    (1, 1, 24, 24, 7, 90, 16),
    (3, 3, 10, 6, 0, 120, 16),
    # bf16: the matrix-core form's variants (head sizes up to 64, wider, values wider than keys;
    # one and several kv heads; a partial last workgroup of heads; 32-token pages; no window)
    (8, 2, 64, 64, 130, 300, 64),
    (6, 1, 80, 112, 100, 260, 64),
    (5, 5, 32, 80, 33, 200, 32),
    (16, 4, 128, 128, 200, 420, 64),
    (4, 4, 48, 16, 0, 200, 32),
], ids=lambda s: "-".join(map(str, s)))
def test_sigmoid_needle(shape, dtype):
    H, G, D, Dv, size, n, bs = shape
    K.case_sigmoid_needle("cuda", dtype, H, G, D, Dv, size, n, bs)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [
    # H, D, rot_dim, rotated entries, Dv, kv_rank, window, tokens, page, interpolation
    (3, 10, 6, 4, 14, 20, 40, 150, 16, None),
    (1, 6, 4, 4, 5, 12, 0, 100, 16, C.YARN),
    (4, 32, 16, 16, 48, 64, 33, 200, 16, None),
    (6, 16, 8, 8, 24, 96, 100, 300, 64, C.YARN),
    (16, 16, 32, 16, 16, 128, 70, 260, 32, None),
    (20, 8, 16, 16, 8, 256, 0, 200, 64, None),
], ids=lambda s: "-".join(map(str, s[:9])))
def test_latent_needle(shape, dtype):
    H, D, rd, rdims, Dv, R, size, n, bs, scaling = shape
    K.case_latent_needle("cuda", dtype, H, D, rd, rdims, Dv, R, size, n, bs, scaling)


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
    """Pages of 32 tokens: the bf16 run takes the matrix-core attention forms end to end."""
    K.case_schedules("cuda", dtype, C.config_c, seed=3, block_size=32)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_long_decode(dtype):
    K.case_long_decode("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_generate_through_engine(dtype):
    K.case_generate("cuda", dtype, C.config_a, expect_graphs=True)


def test_generate_graph_decode_config_c():
    K.case_generate("cuda", torch.bfloat16, C.config_c, expect_graphs=True)


def test_native_library_loaded():
    from enterprise_inference_amd import _native
    lib = _native.kernels()
    assert hasattr(lib, "eia_qk_rope_cache") and hasattr(lib, "eia_add_rms")
    assert any("libeia_kernels" in p for p in _native.loaded_native_libraries())
