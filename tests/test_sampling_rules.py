"""Which strategy a request gets and which tokens its penalties count: the host-side rules of
sampling (no GPU)."""
from xinfer_amd.config.engine_config import GenerationConfig, SamplingParams
from xinfer_amd.sampling.sampler import (PENALTY_CONTEXT, Strategy, penalties_apply, penalty_context,
                                         resolve_strategy)


def test_penalties_count_the_last_128_sampled_tokens_and_never_the_prompt():
    """/root/reference/src/core/runner.rs:1887-1901 and 1950-1962: the list holds what was sampled;
    nothing is counted until it has more than 128 entries, then its last 128."""
    assert PENALTY_CONTEXT == 128
    prompt = list(range(1000, 1300))                       # 300 prompt tokens, never counted
    for generated in (0, 1, 2, 127, 128):
        assert penalty_context(prompt + list(range(generated)), len(prompt)) == []
    assert penalty_context(prompt + list(range(129)), len(prompt)) == list(range(1, 129))
    assert penalty_context(prompt + list(range(500)), len(prompt)) == list(range(372, 500))
    assert penalty_context(list(range(129)), 0) == list(range(1, 129))
    # a long prompt and few sampled tokens: the prompt's tail is not taken in their place
    assert penalty_context(prompt + [7, 7, 7], len(prompt)) == []


def test_a_penalty_of_exactly_one_or_zero_is_off():
    """/root/reference/src/utils/logits_processor.rs:399-401."""
    ctx = [5, 5, 9]
    assert not penalties_apply(Strategy(0.7, 0, 1.0, 0.0, 0.0), ctx)
    assert not penalties_apply(Strategy(0.7, 0, 1.0, 1.0, 0.0), ctx)
    assert not penalties_apply(Strategy(0.7, 0, 1.0, 1.0, 1.0), ctx)
    assert penalties_apply(Strategy(0.7, 0, 1.0, 0.5, 0.0), ctx)
    assert penalties_apply(Strategy(0.7, 0, 1.0, 1.0, 0.3), ctx)         # the other one switches both on
    assert penalties_apply(Strategy(0.7, 0, 1.0, -0.5, 0.0), ctx)
    assert not penalties_apply(Strategy(0.7, 0, 1.0, 0.5, 0.5), [5])      # one token is not enough (:399)
    assert not penalties_apply(Strategy(0.7, 0, 1.0, 0.5, 0.5), [])


def test_strategy_precedence():
    """/root/reference/src/core/runner.rs:1803-1854: a request's temperature 0 is greedy; a request's
    own parameters come first; then generation_config.json if it has a temperature and a top-k or
    top-p; else top-k 32, top-p 0.95, temperature 0.7."""
    gen = GenerationConfig(temperature=0.6, top_p=0.8, top_k=20, frequency_penalty=0.2)
    assert resolve_strategy(SamplingParams(), None) == Strategy(0.7, 32, 0.95)
    assert resolve_strategy(SamplingParams(), gen) == Strategy(0.6, 20, 0.8, 0.2, 0.0)
    assert resolve_strategy(SamplingParams(), GenerationConfig(temperature=0.6)) == Strategy(0.7, 32, 0.95)
    assert resolve_strategy(SamplingParams(temperature=0.0), gen).greedy
    assert resolve_strategy(SamplingParams(temperature=0.9), gen) == Strategy(0.9, 0, 1.0, 0.2, 0.0)
    assert resolve_strategy(SamplingParams(top_k=5), gen).greedy          # parameters of its own, no temperature
    assert resolve_strategy(SamplingParams(temperature=0.5, top_k=5, presence_penalty=0.4), gen) == \
        Strategy(0.5, 5, 1.0, 0.2, 0.4)
