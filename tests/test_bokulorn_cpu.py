"""Bokulorn on the CPU: the engine's host logic (ragged scheduling, pages, state slots, shared-weight layers,
checkpoint placement) with the package's torch restatement of the kernels, against the oracle."""
import pytest

from tests import _bokulorn as K
from tests import _bokulorn_cases as C

DEV = "cpu"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mechanisms(dtype):
    C.case_residual_norm(DEV, dtype)
    C.case_latent_prep_and_query(DEV, dtype)
    C.case_latent_out_gate(DEV, dtype)
    C.case_head_norm_gate_sigmoid(DEV, dtype)
    C.case_softmax_without_sink(DEV, dtype)
    C.case_channel_decay_acts_on_rows(DEV, dtype)
    C.case_moe_ff(DEV, dtype)


def test_moe_route():
    C.case_moe_route(DEV)


def test_channel_delta_portions():
    C.case_channel_delta_portions(DEV, "float32")


def test_latent_attention_beacons():
    C.case_latent_attention_beacons(DEV, "float32")


def test_layer_by_layer(tmp_path):
    C.case_layer_by_layer(DEV, tmp_path)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_schedules(tmp_path, dtype):
    C.case_engine_schedules(DEV, dtype, tmp_path)


def test_engine_odd_sizes(tmp_path):
    C.case_engine_schedules(DEV, "float32", tmp_path, cfg=K.CFG_ODD, seed=9)


def test_engine_wide_sizes(tmp_path):
    C.case_engine_schedules(DEV, "float32", tmp_path, cfg=K.CFG_WIDE, seed=11)


@pytest.mark.parametrize("seed", [101, 102])
def test_engine_random_configs(tmp_path, seed):
    C.case_engine_random_config(DEV, "float32", tmp_path, seed)


def test_engine_reuse_of_pages_and_slots(tmp_path):
    C.case_engine_reuse(DEV, "float32", tmp_path)


def test_engine_long_decode(tmp_path):
    C.case_engine_long_decode(DEV, "float32", tmp_path)


def test_generate_greedy(tmp_path):
    C.case_generate(DEV, tmp_path)


def test_config_reader(tmp_path):
    from light_vllm_amd.models.bokulorn import BokulornConfig
    good = dict(K.CFG_MAIN)
    cfg = BokulornConfig.from_dict(good)
    assert cfg.source_of(3) == 0 and cfg.source_of(4) == 1 and cfg.embedding_scale == 3.5
    lat = dict(K.LAT_A)
    dele = {k: v for k, v in K.DEL_A.items() if k != "decay_rank"}
    for bad in ({**good, "layers": [{"type": "attention", "mixer": lat, "mlp": None}]},
                {**good, "layers": [{"type": "latent_attention", "mixer": {"heads": 2}, "mlp": None}]},
                {**good, "layers": [{"type": "latent_attention", "mixer": lat, "mlp": {"kind": "dense", "ff": 8}}]},
                {**good, "layers": [{"type": "latent_attention", "mixer": lat, "mlp": None, "weights_of": 0}]},
                {**good, "layers": [{"type": "channel_delta", "mixer": dele, "mlp": None}]},      # no rank, no tensor to read it from
                {**good, "layers": [{"type": "latent_attention", "mixer": lat, "mlp": None},
                                    {"type": "latent_attention_2", "mixer": K.LAT_B, "mlp": None, "weights_of": 0}]},
                {k: v for k, v in good.items() if k != "norm"}):
        with pytest.raises(ValueError):
            BokulornConfig.from_dict(bad)


def test_ranks_come_from_the_checkpoint(tmp_path):
    """The thin factors' ranks are not in config.json: the reader takes them from the tensors' shapes."""
    from oracle import bokulorn_oracle as oracle
    from light_vllm_amd.models.bokulorn import BokulornConfig
    weights = oracle.random_weights(K.CFG_MAIN, 1)
    bare = {**K.CFG_MAIN, "layers": [{**L, "mixer": {k: v for k, v in L["mixer"].items() if not k.endswith("_rank") or k in ("q_rank", "kv_rank")}}
                                     for L in K.CFG_MAIN["layers"]]}
    path = K.write_model(tmp_path / "bare", bare, weights)
    cfg = BokulornConfig.from_pretrained(path)
    assert cfg.layers[1]["mixer"]["decay_rank"] == 5 and cfg.layers[4]["mixer"]["gate_rank"] == 6


def test_checkpoint_must_cover_the_model():
    import torch
    from oracle import bokulorn_oracle as oracle
    from light_vllm_amd.models.bokulorn import BokulornConfig, BokulornForCausalLM
    cfg = BokulornConfig.from_dict(K.CFG_MAIN)
    model = BokulornForCausalLM(cfg)
    weights = oracle.random_weights(K.CFG_MAIN, 1)
    assert set(model.weight_targets()) == set(weights)
    model.load_weights(weights.items())
    assert model.layers[3].mix.uk is model.layers[0].mix.uk and model.layers[3].mix.cache is not model.layers[0].mix.cache
    assert model.layers[4].mlp.up_weight is model.layers[1].mlp.up_weight
    few = dict(weights); few.pop("l1.mix.A_log")
    with pytest.raises(KeyError):
        model.load_weights(few.items())
    with pytest.raises(KeyError):
        model.load_weights({**weights, "l3.norm1": weights["l0.norm1"]}.items())
    assert {n for n, _ in model.random_weights(0)} == set(weights)
