"""Bagasun through the engine with the HIP kernels (fp32 sharp, bf16 loose) against the
plain oracle, each mechanism alone, and greedy generation through LLMEngine.generate."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import bagasun_cases as C  # noqa: E402
import bagasun_engine_cases as E  # noqa: E402
import bagasun_mechanism_cases as K  # noqa: E402

pytestmark = pytest.mark.gpu
CASES = [("a", "float32"), ("b", "float32"), ("c", "float32"), ("a", "bfloat16"), ("c", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompt(name, dtype, tmp_path):
    E.whole_prompt(name, "cuda", dtype, tmp_path)


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefill_then_decode(name, dtype, tmp_path):
    E.prefill_then_decode(name, "cuda", dtype, tmp_path)


@pytest.mark.parametrize("name", ["a", "c"])
def test_portions(name, tmp_path):
    E.portions_of_a_prompt(name, "cuda", "float32", tmp_path)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_and_reuse(name, dtype, tmp_path):
    E.mixed_batches_and_reuse(name, "cuda", dtype, tmp_path)


def test_peaked_keys_and_window_edges(tmp_path):
    E.peaked_keys_and_window_edges("cuda", "float32", tmp_path)


def test_long_decode(tmp_path):
    E.long_decode_persistent_state("cuda", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_greedy_generation(name, tmp_path):
    E.greedy_generation(name, "cuda", "float32", tmp_path)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_greedy_generation_graphs(name, tmp_path):
    """Decode steps replayed from captured graphs and queued ahead of the host."""
    E.greedy_generation(name, "cuda", "float32", tmp_path, graphs=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", K.CASES)
def test_mechanism(case, dtype):
    K.run(case, "cuda", dtype)


def test_bf16_generation_runs(tmp_path):
    from fasttalk_llm_microservice_amd.engine.sampling_params import SamplingParams

    d, cfg, _ = C.make_model("c", 3, tmp_path)
    eng = C.make_engine(d, "cuda", "bfloat16", seqs=3)
    outs = eng.generate([C.tokens(n, cfg["vocab"], n) for n in (3, 20, 1, 7)],
                        SamplingParams(temperature=0.8, top_p=0.9, max_tokens=9, ignore_eos=True, seed=1))
    assert [len(o) for o in outs] == [9] * 4 and all(0 <= t < cfg["vocab"] for o in outs for t in o)
