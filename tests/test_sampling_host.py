"""Sampling options and the host side of the sampler (no GPU)."""
import pytest

from palm_infra_amd.sampling import GREEDY, SamplingError, SamplingParams, SequenceSampling, penalty_counts, uniform


def test_defaults_are_the_reference_ones():
    p = SamplingParams()            # engine/sampler.h:7-17
    assert (p.temperature, p.top_k, p.top_p, p.min_p, p.repeat_penalty, p.repeat_last_n, p.presence_penalty,
            p.frequency_penalty, p.seed) == (0.6, 50, 0.9, 0.0, 1.0, 64, 0.0, 0.0, 42)
    p.validate()
    assert not p.greedy and not p.penalties_enabled
    assert GREEDY.plain_argmax and SamplingParams(temperature=1.0, top_k=1).plain_argmax
    assert not SamplingParams(temperature=0.0, repeat_penalty=1.1).plain_argmax
    assert not SamplingParams(repeat_penalty=1.1, repeat_last_n=0).penalties_enabled


@pytest.mark.parametrize("kw,msg", [
    (dict(temperature=-0.1), "temperature"), (dict(temperature=2.5), "temperature"), (dict(temperature=float("nan")), "temperature"),
    (dict(top_k=-1), "top_k"), (dict(top_p=1.5), "top_p"), (dict(min_p=-0.1), "min_p"), (dict(repeat_penalty=0.0), "repeat_penalty"),
    (dict(repeat_last_n=-2), "repeat_last_n"), (dict(presence_penalty=2.5), "presence_penalty"),
    (dict(frequency_penalty=-3.0), "frequency_penalty"), (dict(seed=-1), "seed"),
])
def test_ranges(kw, msg):       # engine/sampler.cpp:222-260, tests/test_sampler.cpp:223-238
    with pytest.raises(SamplingError, match=msg):
        SamplingParams(**kw).validate()


def test_uniform_numbers_depend_on_seed_stream_and_draw_only():
    a = [uniform(42, 3, d) for d in range(200)]
    assert a == [uniform(42, 3, d) for d in range(200)]
    assert all(0.0 <= u < 1.0 for u in a)
    assert a != [uniform(42, 4, d) for d in range(200)] and a != [uniform(43, 3, d) for d in range(200)]
    assert 0.4 < sum(a) / len(a) < 0.6 and len(set(a)) > 190


def test_history_window_counts_match_the_plain_penalties():
    hist = [4, 9, 4, 4, 2, 300, -1]
    assert penalty_counts(hist, 3, 100) == {2: 1}              # 300 and -1 are not tokens of a 100-vocabulary
    assert penalty_counts(hist, -1, 100) == {4: 3, 9: 1, 2: 1}
    assert penalty_counts(hist, 0, 100) == {}
    s = SequenceSampling(stream=1)
    s.accept([1, 2, -5, 3])
    assert s.history == [1, 2, 3]
    s.draws = 4
    s.reset()
    assert s.history == [] and s.draws == 0
