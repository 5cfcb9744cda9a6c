"""Kagalorn on the GPU: the HIP kernels of liblvmix.so, alone and through the engine, against the oracle."""
import pytest

from tests import _kagalorn as K
from tests import _kagalorn_cases as C

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_mechanisms(gpu, dtype):
    C.case_hyper_connection_and_norm(DEV, dtype)
    C.case_clamped_glu(DEV, dtype)
    C.case_head_norm_gate(DEV, dtype)
    C.case_qk_norm_store(DEV, dtype)
    C.case_sink_and_gate(DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_delta_rule_portions(gpu, dtype):
    C.case_delta_rule_portions(DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_pool_beacons(gpu, dtype):
    C.case_window_pool_beacons(DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_schedules(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_odd_sizes(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path, cfg=K.CFG_ODD, seed=9)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_wide_heads(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path, cfg=K.CFG_WIDE, seed=11)


def test_matrix_core_attention_agrees_with_the_vector_kernel(gpu, tmp_path):
    """The same bf16 schedules with the vector kernel forced: both kernels serve one model alike."""
    from light_vllm_amd import mix_ops
    old, mix_ops.WINDOW_ATTN_KERNEL = mix_ops.WINDOW_ATTN_KERNEL, "valu"
    try:
        C.case_engine_schedules(DEV, "bfloat16", tmp_path, cfg=K.CFG_WIDE, seed=11)
        C.case_window_pool_beacons(DEV, "bfloat16")
    finally:
        mix_ops.WINDOW_ATTN_KERNEL = old


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_reuse_of_pages_and_slots(gpu, tmp_path, dtype):
    C.case_engine_reuse(DEV, dtype, tmp_path)


def test_engine_long_decode(gpu, tmp_path):
    C.case_engine_long_decode(DEV, "float32", tmp_path)


def test_generate_greedy(gpu, tmp_path):
    C.case_generate(DEV, tmp_path)


def test_generate_under_preemption(gpu, tmp_path):
    C.case_generate_preemption(DEV, tmp_path)


def test_generate_greedy_from_graphs(gpu, tmp_path):
    """Steps of single tokens replay captured hipGraphs (buckets of 1, 2 and 4 sequences here, padded rows
    included, many replays between eager prompt steps): the completions are the oracle's all the same."""
    C.case_generate(DEV, tmp_path, enforce_eager=False)
