"""Sampling options and the per-request random numbers (CPU)."""
import pytest

from pulse_infer_amd.sampling.params import SamplingParams, uniform_for


def test_uniform_numbers_depend_only_on_seed_and_counter():
    a = [uniform_for(7, i) for i in range(2000)]
    assert a == [uniform_for(7, i) for i in range(2000)]
    assert all(0.0 <= u < 1.0 for u in a)
    assert abs(sum(a) / len(a) - 0.5) < 0.03 and len(set(a)) > 1990
    assert a[:5] != [uniform_for(8, i) for i in range(5)]
    # neighbouring seeds and counters are not correlated in the obvious way
    assert len({uniform_for(s, 0) for s in range(100)}) == 100


def test_options_are_checked():
    assert SamplingParams().greedy and not SamplingParams(temperature=0.7).greedy
    assert SamplingParams(temperature=-1.0).greedy
    for bad in (dict(top_k=-1), dict(top_p=1.5), dict(top_p=-0.1), dict(presence_penalty=-1.0)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
