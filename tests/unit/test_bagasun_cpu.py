"""Bagasun through the engine on the CPU backend (fp32) against the plain oracle, and
each mechanism of models/mixers.py alone against the oracle's function for it."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bagasun_cases as C  # noqa: E402
import bagasun_engine_cases as E  # noqa: E402
import bagasun_mechanism_cases as K  # noqa: E402


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt(name, tmp_path):
    E.whole_prompt(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_prefill_then_decode(name, tmp_path):
    E.prefill_then_decode(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "c"])
def test_portions(name, tmp_path):
    E.portions_of_a_prompt(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_mixed_batches_and_reuse(name, tmp_path):
    E.mixed_batches_and_reuse(name, "cpu", "float32", tmp_path)


def test_peaked_keys_and_window_edges(tmp_path):
    E.peaked_keys_and_window_edges("cpu", "float32", tmp_path)


def test_long_decode(tmp_path):
    E.long_decode_persistent_state("cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation(name, tmp_path):
    E.greedy_generation(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("case", K.CASES)
def test_mechanism(case):
    K.run(case, "cpu", torch.float32)


def test_registry_and_runs(tmp_path):
    from fasttalk_llm_microservice_amd.models.config import resolve_model
    from fasttalk_llm_microservice_amd.models.registry import architecture_of

    d, cfg, _ = C.make_model("a", 1, tmp_path)
    mc = resolve_model(d)
    assert architecture_of(mc).name == "bagasun" and mc.vocab_size == cfg["vocab"]
    assert [r[0] for r in mc.runs()] == [0, 1, 2, 0, 2]
    assert architecture_of(resolve_model("bagasun-tiny")).name == "bagasun"
    assert architecture_of(resolve_model("nulazen-tiny")).name == "nulazen"
    assert architecture_of(resolve_model("tiny")).name == "llama"


def test_borrowed_weights_own_state(tmp_path):
    """A layer on borrowed weights keeps a cache / state of its own: one entry per run,
    distinct tensors, although the two runs share one mixer object."""
    d, cfg, _ = C.make_model("a", 2, tmp_path)
    eng = C.make_engine(d, "cpu")
    m = eng.runner.model
    assert m.layers[3] is None and m.layers[4] is None
    per_run = eng.runner.kv.per_run
    assert len(per_run) == 5
    assert per_run[0][0].data_ptr() != per_run[3][0].data_ptr()
    assert per_run[2][0].data_ptr() != per_run[4][0].data_ptr()
    # a chain of borrowers resolves to the layer that owns weights; a type mismatch is refused
    from fasttalk_llm_microservice_amd.models import bagasun as B
    import copy
    c2 = copy.deepcopy(cfg)
    c2["layers"].append(dict(c2["layers"][3], weights_of=3))
    assert B.config_from_dict(c2).runs()[-1][0] == 0
    c2["layers"][-1]["type"] = "attention"
    with pytest.raises(ValueError):
        B.config_from_dict(c2)


def test_layer_taps_match_oracle(tmp_path):
    """The fp32 residual after every layer run against the oracle's."""
    d, cfg, P = C.make_model("c", 3, tmp_path)
    eng = C.make_engine(d, "cpu")
    t = C.tokens(21, cfg["vocab"], 7)
    eng.runner.model.layer_tap = taps = []
    C.replay(eng, {"r": t}, [[("r", len(t))]])
    eng.runner.model.layer_tap = None
    import bagasun_oracle as O
    want = []
    O.forward(cfg, P, t, want)
    assert len(taps) == len(want) == 4
    for a, b in zip(taps, want):
        torch.testing.assert_close(a, b, rtol=2e-4, atol=2e-4)
