"""Daburax on the framework's CPU path (PyTorch ops, fp32) against the plain oracle in
tests/oracles: every mechanism alone, then the whole model through the engine."""

import pytest
import torch

import daburax_cases as K
import daburax_common as C

F32 = torch.float32


@pytest.mark.parametrize("case", [K.case_hyper_step, K.case_bigram_embed, K.case_route,
                                  K.case_retention_scan, K.case_memory_scan],
                         ids=lambda f: f.__name__)
def test_mechanism(case):
    case("cpu", F32)


def test_frequencies():
    K.case_frequencies()


def test_expert_block():
    K.case_expert_block("cpu", F32)
    K.case_expert_block("cpu", F32, W=32, ff=8, E=3, ident=0, top=1, cnt=1, keep=1, shared=0)


def test_retention_scan_interleaved_pairs_whole_head():
    K.case_retention_scan("cpu", F32, H=2, D=8, Dv=12, dims=8, half=False, T=40)


@pytest.mark.parametrize("size", [0, 40])
def test_sink_needle(size):
    K.case_sink_needle("cpu", F32, size=size, n=120)


@pytest.mark.parametrize("cfg", [C.config_a, C.config_b, C.config_c, C.config_d],
                         ids=lambda f: f.__name__)
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
    from enterprise_inference_amd.models.mixers import ParallelMixer, RetentionMixer
    mc = ModelConfig.from_hf_dict(C.config_a())
    assert mc.architecture == "Daburax" and mc.extra["streams"] == 2
    assert mc.extra["residual_mult"] == 0.7 and mc.extra["embedding"]["bigram"]["buckets"] == 37
    model = get_model_class("Daburax")(mc, dtype=F32)
    assert [type(L.mix) for L in model.layers] == [RetentionMixer, ParallelMixer, RetentionMixer,
                                                   ParallelMixer]
    assert model.layers[1].mlp is None and model.layers[0].mlp.identity == 2
    plain = get_model_class("Daburax")(ModelConfig.from_hf_dict(C.config_b()), dtype=F32)
    assert plain.streams == 0 and plain.bigram is None and plain.mult == 1.0
    assert not any(".hc" in n for n, _ in plain.named_parameters())


def test_every_tensor_has_a_place():
    """Every checkpoint name of a configuration lands in a parameter, every parameter is named
    by the checkpoint, and an unknown name is refused."""
    from enterprise_inference_amd.config import ModelConfig
    from enterprise_inference_amd.models import get_model_class
    for cfg in (C.config_a(), C.config_b(), C.config_c(), C.config_d()):
        model = get_model_class("Daburax")(ModelConfig.from_hf_dict(cfg), dtype=F32)
        W = C.random_weights(cfg, 1)
        loaded = set(model.load_weights(W.items()))
        assert loaded == {n for n, _ in model.named_parameters()}
        with pytest.raises(ValueError):
            model.load_weights([("l0.mix.nothing", torch.zeros(1))])
