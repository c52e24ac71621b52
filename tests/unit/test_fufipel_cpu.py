"""Fufipel through the engine on the CPU backend (fp32) against the plain oracle, and
each mechanism of models/mixers.py alone against the oracle's function for it."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import fufipel_cases as C  # noqa: E402
import fufipel_engine_cases as E  # noqa: E402
import fufipel_mechanism_cases as K  # noqa: E402


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt(name, tmp_path):
    E.whole_prompt(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
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


def test_peaked_scores(tmp_path):
    E.peaked_scores("cpu", "float32", tmp_path)


def test_slow_decay_long_decode(tmp_path):
    E.slow_decay_long_decode("cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation(name, tmp_path):
    E.greedy_generation(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("case", K.CASES)
def test_mechanism(case):
    K.run(case, "cpu", torch.float32)


def test_registry_and_config(tmp_path):
    from fasttalk_llm_microservice_amd.models import fufipel as FX
    from fasttalk_llm_microservice_amd.models.config import resolve_model
    from fasttalk_llm_microservice_amd.models.registry import architecture_of

    d, cfg, _ = C.make_model("a", 1, tmp_path)
    mc = resolve_model(d)
    assert architecture_of(mc).name == "fufipel" and mc.vocab_size == cfg["vocab"]
    assert [r[0] for r in mc.runs()] == [0, 1, 2, 3, 4] and mc.layers[2]["mlp"] is None
    assert mc.layers[2]["mixer"]["kv_from"] == 0 and mc.bigram == (37, 5, 3) and mc.logit_scale == 1.5
    assert architecture_of(resolve_model("fufipel-tiny")).name == "fufipel"
    assert architecture_of(resolve_model("kerarax-tiny")).name == "kerarax"
    assert architecture_of(resolve_model("tiny")).name == "llama"
    # the written configuration parses back to itself; unknown mixers and bad borrowers are refused
    assert FX.config_from_dict(FX.config_to_dict(mc), mc.name) == mc
    for bad in ({**cfg, "layers": [{**cfg["layers"][0], "type": "mamba2"}]},
                {**cfg, "layers": [cfg["layers"][2]]},                       # borrows from itself / a later layer
                {**cfg, "layers": [cfg["layers"][1], cfg["layers"][2]]}):    # borrows from another mixer type
        with pytest.raises(ValueError):
            FX.config_from_dict(bad)


def test_cache_and_state_per_layer(tmp_path):
    """Attention layers own paged keys and values, or share the pages of the layer they
    borrow from; side-by-side layers own pages and an fp32 state per slot; the previous
    token has one entry per slot."""
    d, cfg, _ = C.make_model("a", 2, tmp_path)
    eng = C.make_engine(d, "cpu", pages=8, seqs=3)
    kv = eng.runner.kv
    assert len(kv.per_run) == 5 and kv.extra["last_token"].shape == (3,)
    m = cfg["layers"][0]["mixer"]
    assert kv.per_run[0][0].shape == (8, 16, m["kv_heads"] * m["dim"])
    assert kv.per_run[2] is kv.per_run[0] and kv.per_run[4] is kv.per_run[0]
    (kc, vc), st = kv.per_run[1]
    a, b = cfg["layers"][1]["mixer"]["left"], cfg["layers"][1]["mixer"]["right"]
    assert kc.shape == (8, 16, a["kv_heads"] * a["dim"]) and vc.shape == (8, 16, a["kv_heads"] * a["vdim"])
    assert st.shape == (3, b["heads"], b["dim"], b["vdim"]) and st.dtype == torch.float32
    per_token = sum(x["kv_heads"] * (x["dim"] + x["vdim"]) for x in (m, a, cfg["layers"][3]["mixer"]["left"])) * 4
    assert eng.runner.model.kv_bytes_per_token(4) == per_token == eng.runner.model.cfg.kv_bytes_per_token(4)
