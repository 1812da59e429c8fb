"""Bisuzen on the GPU: the HIP kernels of liblvmix.so, alone and through the engine, against the oracle."""
import pytest

from tests import _bisuzen as K
from tests import _bisuzen_cases as C

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_mechanisms(gpu, dtype):
    C.case_residual_dyt(DEV, dtype)
    C.case_qk_prep(DEV, dtype)
    C.case_glu_act(DEV, dtype)
    C.case_lightning(DEV, dtype)
    C.case_moe_ff(DEV, dtype)


def test_moe_route(gpu):
    C.case_moe_route(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
def test_masked_attention(gpu, dtype):
    C.case_masked_attention(DEV, dtype)


def test_matrix_core_attention_agrees_with_the_vector_kernel(gpu):
    """The same bf16 cases with the vector kernel forced: both kernels see the same keys and sinks."""
    from light_vllm_amd import mix_ops
    old, mix_ops.WINDOW_ATTN_KERNEL = mix_ops.WINDOW_ATTN_KERNEL, "valu"
    try:
        C.case_masked_attention(DEV, "bfloat16")
    finally:
        mix_ops.WINDOW_ATTN_KERNEL = old


def test_layer_by_layer(gpu, tmp_path):
    C.case_layer_by_layer(DEV, tmp_path)
    C.case_layer_by_layer(DEV, tmp_path / "odd", cfg=K.CFG_ODD)
    C.case_layer_by_layer(DEV, tmp_path / "wide", cfg=K.CFG_WIDE)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_schedules(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["CFG_ODD", "CFG_WIDE", "CFG_ONE_PASS", "CFG_NO_LOOP"])
def test_engine_other_sizes(gpu, tmp_path, name, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path, cfg=getattr(K, name), seed=9)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", [101, 102, 104, 105, 107, 108])
def test_engine_random_configs(gpu, tmp_path, seed, dtype):
    C.case_engine_random_config(DEV, dtype, tmp_path, seed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_long_windows(gpu, tmp_path, dtype):
    C.case_engine_long_windows(DEV, dtype, tmp_path)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_reuse_of_pages_and_slots(gpu, tmp_path, dtype):
    C.case_engine_reuse(DEV, dtype, tmp_path)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_long_decode(gpu, tmp_path, dtype):
    C.case_engine_long_decode(DEV, dtype, tmp_path)


def test_generate(gpu, tmp_path):
    C.case_generate(DEV, tmp_path)


def test_generate_from_graphs(gpu, tmp_path):
    C.case_generate(DEV, tmp_path, enforce_eager=False)


def test_generate_bf16_graphs_like_eager(gpu, tmp_path):
    C.case_generate_bf16_graphs_like_eager(DEV, tmp_path)
