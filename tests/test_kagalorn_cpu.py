"""Kagalorn on the CPU: the engine's host logic (ragged scheduling, pages, pooled entries, state slots,
checkpoint placement) with the package's torch restatement of the kernels, against the oracle."""
import pytest

from tests import _kagalorn as K
from tests import _kagalorn_cases as C

DEV = "cpu"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mechanisms(dtype):
    C.case_hyper_connection_and_norm(DEV, dtype)
    C.case_clamped_glu(DEV, dtype)
    C.case_head_norm_gate(DEV, dtype)
    C.case_qk_norm_store(DEV, dtype)
    C.case_sink_and_gate(DEV, dtype)


def test_delta_rule_portions():
    C.case_delta_rule_portions(DEV, "float32")


def test_window_pool_beacons():
    C.case_window_pool_beacons(DEV, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_schedules(tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path)


def test_engine_odd_sizes(tmp_path):
    C.case_engine_schedules(DEV, "float32", tmp_path, cfg=K.CFG_ODD, seed=9)


def test_engine_wide_heads(tmp_path):
    C.case_engine_schedules(DEV, "float32", tmp_path, cfg=K.CFG_WIDE, seed=11)


def test_engine_reuse_of_pages_and_slots(tmp_path):
    C.case_engine_reuse(DEV, "float32", tmp_path)


def test_engine_long_decode(tmp_path):
    C.case_engine_long_decode(DEV, "float32", tmp_path)


def test_generate_greedy(tmp_path):
    C.case_generate(DEV, tmp_path)


def test_generate_under_preemption(tmp_path):
    C.case_generate_preemption(DEV, tmp_path)


def test_config_reader_rejects_what_it_does_not_know():
    from light_vllm_amd.models.kagalorn import KagalornConfig
    good = {k: v for k, v in K.CFG_MAIN.items()}
    KagalornConfig.from_dict(good)
    for bad in ({**good, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]},
                {**good, "layers": [{"type": "delta", "mixer": {"heads": 2}, "mlp": None}]},
                {k: v for k, v in good.items() if k != "norm"}):
        with pytest.raises(ValueError):
            KagalornConfig.from_dict(bad)


def test_checkpoint_must_cover_the_model(tmp_path):
    import torch
    from oracle import kagalorn_oracle as oracle
    from light_vllm_amd.models.kagalorn import KagalornConfig, KagalornForCausalLM
    cfg = KagalornConfig.from_dict(K.CFG_MAIN)
    torch.set_default_dtype(torch.float32)
    model = KagalornForCausalLM(cfg)
    weights = oracle.random_weights(K.CFG_MAIN, 1)
    assert set(model.weight_targets()) == set(weights)
    model.load_weights(weights.items())
    few = dict(weights); few.pop("l1.mix.A_log")
    with pytest.raises(KeyError):
        model.load_weights(few.items())
    with pytest.raises(KeyError):
        model.load_weights({**weights, "l9.norm1": weights["l0.norm1"]}.items())
