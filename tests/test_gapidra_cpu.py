"""Gapidra on the framework's CPU path (PyTorch ops, fp32) against the plain oracle in
tests/oracles: every mechanism alone, then the whole model through the engine."""

import pytest
import torch

import gapidra_cases as K
import gapidra_common as C

F32 = torch.float32


@pytest.mark.parametrize("case", [K.case_residual_rms_step, K.case_xielu, K.case_sigmoid_gate,
                                  K.case_qk_rope_cache, K.case_latent_prep],
                         ids=lambda f: f.__name__)
def test_mechanism(case):
    case("cpu", F32)


def test_frequencies():
    K.case_frequencies()


@pytest.mark.parametrize("size", [40, 0])
def test_sigmoid_needle(size):
    K.case_sigmoid_needle("cpu", F32, size=size, n=120)


@pytest.mark.parametrize("size", [40, 0])
def test_latent_needle(size):
    K.case_latent_needle("cpu", F32, size=size, n=120)


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
    from enterprise_inference_amd.models.mixers import (LatentAttentionMixer,
                                                        SigmoidWindowAttentionMixer)
    mc = ModelConfig.from_hf_dict(C.config_a())
    assert mc.architecture == "Gapidra" and mc.extra["embedding"]["scale"] == 3.0
    model = get_model_class("Gapidra")(mc, dtype=F32)
    kinds = [type(L.mix) for L in model.layers]
    assert kinds == [LatentAttentionMixer, SigmoidWindowAttentionMixer,
                     SigmoidWindowAttentionMixer, LatentAttentionMixer]
    assert model.layers[2].mlp is None and model.layers[0].mlp is not None
    assert model.layers[0].mix.window == 9 and model.layers[2].mix.window == 1
    assert model.layers[1].mix.rot_amp > 1.0 and model.layers[2].mix.rot_amp == 1.0
    assert len(model.allocate_cache(2, 16, 0, F32, "cpu")) == 4
    mb = get_model_class("Gapidra")(ModelConfig.from_hf_dict(C.config_b()), dtype=F32)
    assert mb.embed_scale == 1.0 and mb.layers[0].mix.window == 0 and mb.layers[1].mix.rot_dims == 0
    with pytest.raises(ValueError):
        model.load_weights([("l0.mix.nonsense", torch.zeros(1))])
    with pytest.raises(ValueError):
        model.load_weights([("l0.mix.q", torch.zeros(3, 46))])
