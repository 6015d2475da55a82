"""Nulazen through the engine on the CPU backend (fp32) against the plain oracle, and
each mechanism of models/mixers.py alone against the oracle's function for it."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import nulazen_cases as C  # noqa: E402
import nulazen_engine_cases as E  # noqa: E402
import nulazen_mechanism_cases as K  # noqa: E402


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


def test_far_key_and_page_borders(tmp_path):
    E.far_key_and_page_borders("cpu", "float32", tmp_path)


def test_long_decode(tmp_path):
    E.long_decode_persistent_state("cpu", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation(name, tmp_path):
    E.greedy_generation(name, "cpu", "float32", tmp_path)


@pytest.mark.parametrize("case", K.CASES)
def test_mechanism(case):
    K.run(case, "cpu", torch.float32)


def test_registry_picks_the_class(tmp_path):
    from fasttalk_llm_microservice_amd.models.config import resolve_model
    from fasttalk_llm_microservice_amd.models.registry import architecture_of

    d, cfg, _ = C.make_model("b", 1, tmp_path)
    mc = resolve_model(d)
    assert architecture_of(mc).name == "nulazen" and mc.vocab_size == cfg["vocab"]
    assert architecture_of(resolve_model("tiny")).name == "llama"
    assert architecture_of(resolve_model("nulazen-tiny")).name == "nulazen"
    assert len(mc.runs()) == 2 and len(resolve_model("nulazen-tiny").runs()) == 5


def test_state_slots_gate_admission(tmp_path):
    """The scheduler admits no more sequences than there are state slots, and a
    preempted / finished sequence's slot is handed on."""
    from fasttalk_llm_microservice_amd.engine.sampling_params import SamplingParams

    d, cfg, _ = C.make_model("b", 2, tmp_path)
    eng = C.make_engine(d, "cpu", seqs=2, pages=8)
    prompts = [C.tokens(n, cfg["vocab"], n) for n in (4, 6, 3, 9, 2)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))
    assert [len(o) for o in outs] == [5] * 5
    assert eng.scheduler.slots.num_free() == 2 and eng.bm.num_free() == 8


def test_replay_order_and_idle_steps(tmp_path):
    """Wanted rows come back in the caller's order whatever the step's row order is; a
    request may sit out a step; an entry without tokens and a step without entries run
    nothing; a finished request's id can be used again."""
    import numpy as np

    d, cfg, P = C.make_model("b", 3, tmp_path)
    eng = C.make_engine(d, "cpu", seqs=2, pages=8)
    ta, tb = C.tokens(9, cfg["vocab"], 1), C.tokens(6, cfg["vocab"], 2)
    wa, wb = C.oracle(cfg, P, ta), C.oracle(cfg, P, tb)
    eng.replay_step([("a", ta[:4], [3, 0])])
    lg = eng.replay_step([("a", ta[4:5], [0]), ("b", tb[:5], [4, 1, 2])])          # a decodes beside b's prompt
    np.testing.assert_allclose(lg, np.stack([wa[4], wb[4], wb[1], wb[2]]), rtol=2e-4, atol=3e-4)
    assert eng.replay_step([("a", [], [])]).shape == (0, cfg["vocab"])
    assert eng.replay_step([], []).shape[0] == 0
    lg = eng.replay_step([("b", tb[5:], [0])], end=["b"])                          # a sits this step out
    np.testing.assert_allclose(lg[0], wb[5], rtol=2e-4, atol=3e-4)
    lg = eng.replay_step([("b", tb[:2], [1]), ("a", ta[5:], [3])], end=["a", "b"])  # a new request named b
    np.testing.assert_allclose(lg, np.stack([wb[1], wa[8]]), rtol=2e-4, atol=3e-4)
    assert eng.scheduler.slots.num_free() == 2 and eng.bm.num_free() == 8
