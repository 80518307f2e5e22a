"""The framework's host-side sampling pieces against the plain sampler."""
import numpy as np
import pytest

from kappai_amd.sampling import RandomStream, RequestSampler, SamplingParams, filtered_draw
from plain import sampler as S


def test_random_stream_equals_the_plain_one():
    for seed in (1, 42, 2 ** 40 + 3):
        a, b = RandomStream(seed), S.Rng(seed)
        assert [a.uniform() for _ in range(100)] == [b.uniform() for _ in range(100)]
    assert RandomStream(0).s != RandomStream(0).s        # seed 0: entropy


@pytest.mark.parametrize("kw", [
    dict(temperature=0.8, top_k=40, top_p=0.9, min_p=0.1),
    dict(temperature=1.3, top_k=5, top_p=1.0, min_p=0.0),
    dict(temperature=0.5, top_k=0, top_p=0.6, min_p=0.0),
    dict(temperature=1.0, top_k=0, top_p=1.0, min_p=0.3),
    dict(temperature=2.0, top_k=3000, top_p=0.95, min_p=0.01),
])
def test_filtered_draw_equals_the_plain_one(kw):
    rng = np.random.default_rng(3)
    for trial in range(30):
        vocab = int(rng.choice([50, 700, 2500]))
        logits = (rng.normal(size=vocab) * 3).astype(np.float32)
        u = float(np.float32(rng.random()))
        p = SamplingParams(**kw)
        assert filtered_draw(logits, p, u) == S.sample_filtered(
            logits, kw["temperature"], kw["top_k"], kw["top_p"], kw["min_p"], u)


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
