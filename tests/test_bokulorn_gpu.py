"""Bokulorn on the GPU: the HIP kernels of liblvmix.so, alone and through the engine, against the oracle."""
import pytest

from tests import _bokulorn as K
from tests import _bokulorn_cases as C

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_mechanisms(gpu, dtype):
    C.case_residual_norm(DEV, dtype)
    C.case_latent_prep_and_query(DEV, dtype)
    C.case_latent_out_gate(DEV, dtype)
    C.case_head_norm_gate_sigmoid(DEV, dtype)
    C.case_softmax_without_sink(DEV, dtype)
    C.case_channel_decay_acts_on_rows(DEV, dtype)
    C.case_moe_ff(DEV, dtype)


def test_moe_route(gpu):
    C.case_moe_route(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
def test_channel_delta_portions(gpu, dtype):
    C.case_channel_delta_portions(DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_attention_beacons(gpu, dtype):
    C.case_latent_attention_beacons(DEV, dtype)


def test_layer_by_layer(gpu, tmp_path):
    C.case_layer_by_layer(DEV, tmp_path)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_schedules(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_odd_sizes(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path, cfg=K.CFG_ODD, seed=9)


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_wide_sizes(gpu, tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path, cfg=K.CFG_WIDE, seed=11)


def test_matrix_core_attention_agrees_with_the_vector_kernel(gpu, tmp_path):
    """The same bf16 schedules and beacons with the vector kernel forced: both kernels serve one model alike."""
    from light_vllm_amd import mix_ops
    old, mix_ops.WINDOW_ATTN_KERNEL = mix_ops.WINDOW_ATTN_KERNEL, "valu"
    try:
        C.case_engine_schedules(DEV, "bfloat16", tmp_path, cfg=K.CFG_WIDE, seed=11)
        C.case_latent_attention_beacons(DEV, "bfloat16")
    finally:
        mix_ops.WINDOW_ATTN_KERNEL = old


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", [101, 102, 103, 104])
def test_engine_random_configs(gpu, tmp_path, seed, dtype):
    C.case_engine_random_config(DEV, dtype, tmp_path, seed)


def test_masked_experts_serve_the_model_like_the_gathered_ones(gpu, tmp_path):
    """The bf16 schedules above take the gathered form of the feed-forward (sizes in multiples of 32); here the
    masked form is forced on the same model."""
    from light_vllm_amd.layers import moe
    old, moe.MOE_KERNEL = moe.MOE_KERNEL, "masked"
    try:
        C.case_engine_schedules(DEV, "bfloat16", tmp_path, cfg=K.CFG_WIDE, seed=11)
    finally:
        moe.MOE_KERNEL = old


def test_sorted_experts_serve_the_model_like_the_gathered_ones(gpu, tmp_path):
    """The form that large eager steps take (vendor GEMMs on rows sorted by expert), forced on the same small model."""
    from light_vllm_amd.layers import moe
    old, moe.MOE_KERNEL = moe.MOE_KERNEL, "sorted"
    try:
        C.case_engine_schedules(DEV, "bfloat16", tmp_path, cfg=K.CFG_WIDE, seed=11)
    finally:
        moe.MOE_KERNEL = old


@pytest.mark.parametrize("dtype", DTYPES)
def test_engine_reuse_of_pages_and_slots(gpu, tmp_path, dtype):
    C.case_engine_reuse(DEV, dtype, tmp_path)


def test_engine_long_decode(gpu, tmp_path):
    C.case_engine_long_decode(DEV, "float32", tmp_path)


def test_generate_greedy(gpu, tmp_path):
    C.case_generate(DEV, tmp_path)


def test_generate_greedy_from_graphs(gpu, tmp_path):
    """Steps of single tokens replay captured hipGraphs (padded rows included, many replays between eager prompt
    steps): the completions are the oracle's all the same."""
    C.case_generate(DEV, tmp_path, enforce_eager=False)


def test_generate_bf16_from_graphs_like_eager(gpu, tmp_path):
    C.case_generate_bf16_graphs_like_eager(DEV, tmp_path)
