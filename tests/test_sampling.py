"""The framework's host-side sampling pieces against the plain sampler."""
import pytest

from kappai_amd.sampling import RandomStream, RequestSampler, Sampler, SamplingParams
from plain import sampler as S


def test_random_stream_equals_the_plain_one():
    for seed in (1, 42, 2 ** 40 + 3):
        a, b = RandomStream(seed), S.Rng(seed)
        assert [a.uniform() for _ in range(100)] == [b.uniform() for _ in range(100)]
    assert RandomStream(0).s != RandomStream(0).s        # seed 0: entropy


def test_params():
    assert SamplingParams().temperature == pytest.approx(0.8) and SamplingParams().top_k == 40
    assert SamplingParams.greedy().is_greedy() and SamplingParams(top_k=1).is_greedy()
    assert SamplingParams().is_filtered(1000)
    assert not SamplingParams(top_k=0, top_p=1.0, min_p=0.0).is_filtered(1000)
    assert not SamplingParams(top_k=2000, top_p=1.0, min_p=0.0).is_filtered(1000)
    with pytest.raises(ValueError):
        SamplingParams(repeat_penalty=0).validate()
    s = RequestSampler(SamplingParams(repeat_last_n=3, repeat_penalty=1.5, seed=4))
    s.observe([1, 2, 3, 4, 5])
    assert s.penalty_window() == [3, 4, 5]


def test_what_the_host_has_to_see():
    """Steps may be queued ahead of their tokens for every way of drawing that needs no earlier
    token of the row from the host: the repeat penalty looks at earlier tokens, which are kept on
    the GPU up to a window of ``HISTORY_CAP``; only a longer window needs the host's list."""
    from kappai_amd.sampling.sampler import HISTORY_CAP
    plain = [RequestSampler(SamplingParams(top_k=k, top_p=0.9)) for k in (0, 40, 5000)]
    assert Sampler.runs_on_device(plain, 65536)
    assert Sampler.runs_on_device(plain + [RequestSampler(SamplingParams(repeat_penalty=1.1))],
                                  65536)
    assert Sampler.runs_on_device(
        [RequestSampler(SamplingParams(repeat_penalty=1.1, repeat_last_n=HISTORY_CAP))], 65536)
    assert not Sampler.runs_on_device(plain + [RequestSampler(SamplingParams(
        repeat_penalty=1.1, repeat_last_n=HISTORY_CAP + 1))], 65536)
    assert Sampler.runs_on_device([RequestSampler(SamplingParams(
        repeat_penalty=1.0, repeat_last_n=HISTORY_CAP + 1))], 65536)
