"""The host sampler against the plain one, and the reference's own sampler vectors
(tests/test_orchestrator.py:175-274)."""
import numpy as np
import pytest

from plain import gemma2_plain as P
from zse_amd.sampling import SamplingParams, sample_host, uniform


def test_reference_vectors():
    assert sample_host(np.array([0.1, 0.5, 0.3, 0.9, 0.2]), SamplingParams(temperature=0.0), 0.3) == 3
    assert sample_host(np.array([-1.0, -0.5, -2.0]), SamplingParams(temperature=0.0), 0.3) == 1
    z = np.array([0.1, 5.0, 0.2, 4.0, 0.0])
    got = {sample_host(z, SamplingParams(temperature=1.0, top_k=2), uniform(i, 0)) for i in range(50)}
    assert got <= {1, 3} and got == {1, 3}
    assert sample_host(np.array([10.0, -10, -10, -10]), SamplingParams(top_p=0.5), 0.999) == 0
    z = np.array([5.0, 4.9, 0.1])
    assert sample_host(z, SamplingParams(temperature=0.0), 0.5) == 0
    assert sample_host(z, SamplingParams(temperature=0.0, repetition_penalty=2.0), 0.5, past={0}) == 1
    low = sum(sample_host(np.array([10.0, 0, 0, 0, 0]), SamplingParams(temperature=0.1), uniform(i, 0)) == 0
              for i in range(100))
    high = sum(sample_host(np.array([10.0, 0, 0, 0, 0]), SamplingParams(temperature=5.0), uniform(i + 1000, 0)) != 0
               for i in range(100))
    assert low >= 95 and high > 10


def test_greedy_takes_the_first_maximum():
    assert sample_host(np.array([1.0, 3.0, 3.0, 2.0]), SamplingParams(temperature=0.0), 0.9) == 1


def test_uniform_is_a_pure_function_in_the_unit_interval():
    u = [uniform(7, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in u) and len(set(u)) == 2000
    assert uniform(7, 5) == uniform(7, 5) and uniform(7, 5) != uniform(8, 5)
    assert abs(np.mean(u) - 0.5) < 0.03


@pytest.mark.parametrize("seed", range(5))
def test_agrees_with_the_plain_sampler(seed):
    rng = np.random.default_rng(seed)
    for _ in range(40):
        z = rng.normal(0, 3, 200)
        t = float(rng.choice([0.0, 0.3, 0.8, 1.0, 2.0]))
        k = int(rng.choice([0, 1, 5, 50, 500]))
        p = float(rng.choice([1.0, 0.95, 0.5, 0.1]))
        pen = float(rng.choice([1.0, 1.3, 2.0]))
        past = {int(i) for i in rng.integers(0, 200, 10)}
        u = float(rng.random())
        sp = SamplingParams(temperature=t, top_k=k, top_p=p, repetition_penalty=pen)
        want = P.sample(z, u, t, k, p, pen, {i: 1 for i in past})
        assert sample_host(z, sp, u, past) == want


def test_params_validate():
    for bad in (dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1), dict(repetition_penalty=0.0),
                dict(max_tokens=-1)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    assert SamplingParams(temperature=0).greedy and SamplingParams(temperature=1e-7).greedy
    assert SamplingParams(temperature=0.8).plain and not SamplingParams(top_k=5).plain
    assert SamplingParams(temperature=0, top_k=5).plain and not SamplingParams(temperature=0, repetition_penalty=1.2).plain


def test_penalty_scales_follow_how_often_a_token_appeared():
    # once: the penalty itself; n times: penalty ** (1 + log2 n) (reference orchestrator/sampler.py:64-74)
    from zse_amd.sampling.sampler import apply_repetition_penalty, penalty_scales
    sc = penalty_scales({3: 1, 5: 2, 9: 8}, 1.5)
    assert sc[3] == 1.5 and abs(sc[5] - 1.5 ** 2) < 1e-12 and abs(sc[9] - 1.5 ** 4) < 1e-12
    assert penalty_scales([4, 4, 7], 2.0) == {4: 2.0, 7: 2.0}          # a plain list counts every token once
    z = apply_repetition_penalty(np.array([2.0, -2.0, 1.0]), {0: 1, 1: 1, 7: 3}, 2.0)
    assert list(z) == [1.0, -4.0, 1.0]                                  # positive divided, negative multiplied, out of range ignored
