"""Kerarax through the engine on the CPU backend (fp32) against the plain oracle, and
each mechanism of models/mixers.py alone against the oracle's function for it."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import kerarax_cases as C  # noqa: E402
import kerarax_engine_cases as E  # noqa: E402
import kerarax_mechanism_cases as K  # noqa: E402


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt(name, tmp_path):
    E.whole_prompt(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "c"])
def test_layers(name, tmp_path):
    E.layers_of_a_prompt(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_prefill_then_decode(name, tmp_path):
    E.prefill_then_decode(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "c"])
def test_portions(name, tmp_path):
    E.portions_of_a_prompt(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_mixed_batches_and_reuse(name, tmp_path):
    E.mixed_batches_and_reuse(name, "cpu", "float32", tmp_path)


def test_peaked_and_flat_scores(tmp_path):
    E.peaked_and_flat_scores("cpu", "float32", tmp_path)


def test_long_decode(tmp_path):
    E.long_decode("cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation(name, tmp_path):
    E.greedy_generation(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("case", K.CASES)
def test_mechanism(case):
    K.run(case, "cpu", torch.float32)


def test_registry_and_config(tmp_path):
    from fasttalk_llm_microservice_amd.models import kerarax as KX
    from fasttalk_llm_microservice_amd.models.config import resolve_model
    from fasttalk_llm_microservice_amd.models.registry import architecture_of

    d, cfg, _ = C.make_model("a", 1, tmp_path)
    mc = resolve_model(d)
    assert architecture_of(mc).name == "kerarax" and mc.vocab_size == cfg["vocab"]
    assert [r[0] for r in mc.runs()] == [0, 1, 2] and mc.layers[1]["mlp"] is None
    assert mc.layers[2]["mlp"]["shared"] is None and mc.logit_softcap == 7.0
    assert architecture_of(resolve_model("kerarax-tiny")).name == "kerarax"
    assert architecture_of(resolve_model("bagasun-tiny")).name == "bagasun"
    assert architecture_of(resolve_model("tiny")).name == "llama"
    # the written configuration parses back to itself; an unknown mixer is refused
    assert KX.config_from_dict(KX.config_to_dict(mc), mc.name) == mc
    bad = {**cfg, "layers": [{**cfg["layers"][0], "type": "mamba2"}]}
    with pytest.raises(ValueError):
        KX.config_from_dict(bad)


def test_cache_and_state_per_layer(tmp_path):
    """Every layer owns paged keys, paged values and a history of projected rows per state
    slot, sized by its own heads and taps."""
    d, cfg, _ = C.make_model("a", 2, tmp_path)
    eng = C.make_engine(d, "cpu", pages=8, seqs=3)
    per_run = eng.runner.kv.per_run
    assert len(per_run) == 3
    for (kc, vc, hist), l in zip(per_run, cfg["layers"]):
        m = l["mixer"]
        assert kc.shape == (8, 16, m["kv_heads"] * m["dim"]) and vc.shape == (8, 16, m["kv_heads"] * m["vdim"])
        ch = (m["heads"] + m["kv_heads"]) * m["dim"] + m["kv_heads"] * m["vdim"]
        assert hist.shape == (3, m["conv"] - 1, ch) and hist.dtype == torch.float32
