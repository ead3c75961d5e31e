"""Daburax on the MI355X path (HIP kernels; fp32 and bf16 activations) against the plain oracle
in tests/oracles: every kernel alone, then the whole model through the engine."""

import pytest
import torch

import daburax_cases as K
import daburax_common as C

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
IDS = ["fp32", "bf16"]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("case", [K.case_hyper_step, K.case_bigram_embed, K.case_route],
                         ids=lambda f: f.__name__)
def test_kernel(case, dtype):
    case("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [
    # H, D, Dv, rotated entries, half-split pairs, tokens
    (3, 10, 6, 4, True, 75),
    (2, 8, 12, 8, False, 40),
    (1, 32, 32, 0, True, 50),
    (2, 64, 48, 32, True, 90),
    (2, 24, 128, 24, True, 40),
    (1, 160, 96, 64, False, 30),
], ids=lambda s: "-".join(map(str, s)))
def test_retention_scan(shape, dtype):
    H, D, Dv, dims, half, T = shape
    K.case_retention_scan("cuda", dtype, H, D, Dv, dims, half, T)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(2, 6, 10, 70), (1, 32, 16, 40), (3, 48, 64, 80),
                                   (2, 128, 72, 30), (1, 40, 200, 20)],
                         ids=lambda s: "-".join(map(str, s)))
def test_memory_scan(shape, dtype):
    H, D, Dv, T = shape
    K.case_memory_scan("cuda", dtype, H, D, Dv, T)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(3, 10, 6, 4, True, 150), (2, 64, 48, 32, True, 140),
                                   (2, 128, 128, 128, False, 135), (1, 24, 128, 0, True, 200)],
                         ids=lambda s: "-".join(map(str, s)))
def test_retention_scan_chunk_parallel(shape, dtype):
    H, D, Dv, dims, half, T = shape
    K.case_retention_scan("cuda", dtype, H, D, Dv, dims, half, T, chunked=True)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(2, 6, 10, 150), (3, 48, 64, 140), (2, 128, 72, 135),
                                   (1, 128, 128, 200)], ids=lambda s: "-".join(map(str, s)))
def test_memory_scan_chunk_parallel(shape, dtype):
    H, D, Dv, T = shape
    K.case_memory_scan("cuda", dtype, H, D, Dv, T, chunked=True)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [
    # H, G, D, Dv, window, tokens, page
    (4, 2, 16, 8, 0, 150, 16),
    (1, 1, 24, 24, 0, 90, 16),
    (3, 3, 10, 6, 40, 120, 16),
    # bf16: the matrix-core form's variants (one and several kv heads, a partial last workgroup
    # of heads, values wider and narrower than keys, 32- and 64-token pages, key partitions)
    (8, 2, 64, 64, 0, 300, 64),
    (6, 1, 80, 112, 0, 260, 64),
    (5, 5, 32, 80, 0, 200, 32),
    (16, 4, 128, 128, 200, 420, 64),
    (4, 4, 48, 16, 0, 700, 32),
], ids=lambda s: "-".join(map(str, s)))
def test_sink_needle(shape, dtype):
    H, G, D, Dv, size, n, bs = shape
    K.case_sink_needle("cuda", dtype, H, G, D, Dv, n, bs, size)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [
    # W, ff, experts, identity, top, groups, keep, shared ff, tokens
    (46, 20, 6, 2, 3, 4, 2, 12, 21),            # per-expert form
    (128, 64, 6, 2, 2, 2, 1, 64, 40),           # grouped matrix-core form
    (256, 256, 14, 2, 2, 4, 2, 256, 32),        # grouped weight-streaming form (decode-sized)
    (256, 256, 3, 1, 2, 2, 1, 0, 700),          # many rows per expert
    (512, 128, 8, 0, 2, 1, 1, 128, 9),
], ids=lambda s: "-".join(map(str, s)))
def test_expert_block(shape, dtype):
    W, ff, E, ident, top, cnt, keep, shared, T = shape
    K.case_expert_block("cuda", dtype, W, ff, E, ident, top, cnt, keep, shared, T)


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
def test_schedules_odd_shared_row(dtype):
    K.case_schedules("cuda", dtype, C.config_d, seed=5, block_size=32)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_long_decode(dtype):
    K.case_long_decode("cuda", dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_generate_through_engine(dtype):
    K.case_generate("cuda", dtype, C.config_a)


def test_generate_graph_decode_config_c():
    K.case_generate("cuda", torch.bfloat16, C.config_c, expect_graphs=True)


def test_native_library_loaded():
    from enterprise_inference_amd import _native
    lib = _native.kernels()
    assert hasattr(lib, "eia_linear_scan") and hasattr(lib, "eia_hyper_step")
    assert hasattr(lib, "eia_bigram_embed")
    assert any("libeia_kernels" in p for p in _native.loaded_native_libraries())
