"""Generation parameters: the reference's defaults, checks and choice of sampling mode."""
import pytest

from atoma_infer_amd.sampling import DEFAULT_RANDOM_SEED, GenerateParameters, ValidationError, uniform, validate


def plan(**kw):
    return validate(GenerateParameters(**kw), 10, 4096, 8192)


def test_defaults_follow_the_reference():
    """backends/vllm/src/validation.rs:226-315, types.rs:84-85."""
    p = plan()
    assert p.temperature == 1.0 and p.top_k == 0 and p.top_p == 1.0 and p.repetition_penalty == 1.0
    assert p.random_seed == DEFAULT_RANDOM_SEED == 1_283_768_955 and p.max_new_tokens == 100
    assert p.greedy and p.mode == "ArgMax"          # temperature 1.0 means argmax (llm_service.rs:346-348)
    assert plan(max_new_tokens=None).max_new_tokens == 8192 - 10   # validation.rs:133-137


def test_mode_selection():
    """backends/vllm/src/llm_service.rs:346-372."""
    assert plan(temperature=0.7).mode == "All"
    assert plan(temperature=0.7, do_sample=False).mode == "ArgMax"
    assert plan(temperature=0.7, top_p=0.9).mode == "TopP"
    assert plan(temperature=0.7, top_k=5).mode == "TopK"
    assert plan(temperature=0.7, top_k=5, top_p=0.9).mode == "TopKThenTopP"
    assert plan(temperature=1.0, top_k=5).mode == "ArgMax"


@pytest.mark.parametrize("kw", [
    {"temperature": 0.0}, {"temperature": -1.0}, {"repetition_penalty": 0.0}, {"frequency_penalty": 2.5},
    {"top_p": 1.0}, {"top_p": 0.0}, {"typical_p": 1.5}, {"top_k": 0}, {"max_new_tokens": 0},
    {"stop": ["a", "b"]}, {"top_n_tokens": 5}, {"truncate": 0}, {"truncate": 5000}, {"best_of": 2},
    {"max_new_tokens": 9000}, {"repetition_penalty": 1.2},
])
def test_invalid_parameters_are_refused(kw):
    with pytest.raises(ValidationError):
        plan(**kw)


def test_input_length_checks():
    with pytest.raises(ValidationError):
        validate(GenerateParameters(), 0, 4096, 8192)
    with pytest.raises(ValidationError):
        validate(GenerateParameters(), 5000, 4096, 8192)
    assert plan(repetition_penalty=1.2, repeat_last_n=16).repeat_last_n == 16


def test_uniform_is_a_pure_function_in_the_unit_interval():
    xs = [uniform(42, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in xs)
    assert xs == [uniform(42, i) for i in range(2000)]
    assert abs(sum(xs) / len(xs) - 0.5) < 0.03 and len(set(xs)) > 1990
    assert uniform(42, 0) != uniform(43, 0)
