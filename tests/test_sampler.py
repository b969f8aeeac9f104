"""The host sampler and the random stream (no GPU): the vectors of the reference's
tests/sampling/test_sampler.cpp, and draw-for-draw agreement with the plain sampler."""

import math
import random

import numpy as np
import pytest

import plain_qwen3 as plain
from tie_amd.errors import InvalidArgument
from tie_amd.sampling import RandomStream, SamplingParams, sample

LOGITS = np.log(np.array([0.7, 0.2, 0.1], dtype=np.float32))


def frequencies(params, draws, logits=LOGITS):
    rng = RandomStream(params.seed)
    freq = [0.0] * len(logits)
    for _ in range(draws):
        freq[sample(logits, params, rng)] += 1.0 / draws
    return freq


def test_random_stream_is_the_64_bit_mersenne_twister():
    rng = RandomStream(5489)
    for _ in range(9999):
        rng.next_u64()
    assert rng.next_u64() == 9981545732273789042            # fixed by the C++ standard for mt19937_64
    a, b = RandomStream(3), plain.MT19937_64(3)
    assert [a.next_u64() for _ in range(700)] == [b() for _ in range(700)]
    u = RandomStream(1).uniform(0.0, 2.5)
    assert 0.0 <= u < 2.5


def test_greedy_takes_the_first_maximum():
    rng = RandomStream(0)
    assert sample(np.array([0.1, 2.0, -1.0], np.float32), SamplingParams(), rng) == 1
    assert sample(np.array([3.0, 1.0, 3.0], np.float32), SamplingParams(), rng) == 0


def test_temperature_one_follows_the_softmax():
    f = frequencies(SamplingParams(temperature=1.0, seed=42), 20000)
    assert f[0] == pytest.approx(0.7, rel=0.03) and f[1] == pytest.approx(0.2, rel=0.1) and f[2] == pytest.approx(0.1, rel=0.15)


def test_top_k_and_top_p_remove_the_tail():
    f = frequencies(SamplingParams(temperature=1.0, seed=7, top_k=2), 5000)
    assert f[2] == 0.0 and f[0] == pytest.approx(0.7 / 0.9, rel=0.05)
    f = frequencies(SamplingParams(temperature=1.0, seed=7, top_p=0.75), 5000)   # 0.7 alone falls short of 0.75
    assert f[2] == 0.0 and f[1] > 0.0
    f = frequencies(SamplingParams(temperature=1.0, seed=7, top_p=0.01), 500)
    assert f[0] == pytest.approx(1.0) and f[1] == 0.0 and f[2] == 0.0


def test_top_k_and_top_p_combine():
    logits = np.log(np.array([0.5, 0.3, 0.15, 0.05], dtype=np.float32))
    p = SamplingParams(temperature=1.0, top_k=3, top_p=0.7)    # top 3 total 0.95; 0.5 < 0.665 <= 0.8
    rng = RandomStream(11)
    seen = {sample(logits, p, rng) for _ in range(2000)}
    assert seen == {0, 1}


def test_the_same_seed_reproduces_the_same_draws():
    p = SamplingParams(temperature=1.0, seed=3)
    assert frequencies(p, 200) == frequencies(p, 200)


def test_validate_rejects_impossible_parameters():
    SamplingParams().validate()
    for bad in (dict(temperature=-0.1), dict(top_k=-1), dict(top_p=0.0), dict(top_p=1.5), dict(max_tokens=0),
                dict(temperature=math.nan), dict(temperature=math.inf), dict(top_p=math.nan), dict(seed=-1)):
        with pytest.raises(InvalidArgument):
            SamplingParams(**bad).validate()


def test_tiny_temperatures_are_greedy():
    rng = RandomStream(0)
    p = SamplingParams(temperature=1e-40)                      # subnormal in float32: the reciprocal is not finite
    p.validate()
    assert sample(np.array([0.0, 1.0, -2.0], np.float32), p, rng) == 1
    assert sample(np.array([0.0, -np.inf, 0.0], np.float32), p, rng) == 0
    p = SamplingParams(temperature=2e-38)                      # 1/t is finite, but logit/t would overflow
    for seed in range(200):
        rng = RandomStream(seed)
        assert sample(np.array([5.0, 6.0], np.float32), p, rng) == 1
        assert sample(np.array([10.0, 11.0, 9.0], np.float32), p, rng) == 1
        assert sample(np.array([-17.0, -13.0, -15.0], np.float32), p, rng) == 1


def test_nan_and_infinite_logits():
    rng = RandomStream(0)
    sampled = SamplingParams(temperature=1.0)
    nan_logits = np.array([1.0, np.nan, 2.0], np.float32)
    for p in (SamplingParams(), sampled):
        with pytest.raises(InvalidArgument, match="logit 1 is NaN"):
            sample(nan_logits, p, rng)
    with_inf = np.array([1.0, np.inf, 2.0, np.inf], np.float32)
    before = RandomStream(0).next_u64()
    assert sample(with_inf, SamplingParams(), rng) == 1 and sample(with_inf, sampled, rng) == 1
    assert rng.next_u64() == before                            # a certain token does not consume a random number
    assert sample(np.array([-np.inf, 0.0, -np.inf], np.float32), sampled, rng) == 1
    with pytest.raises(InvalidArgument, match="-inf"):
        sample(np.array([-np.inf, -np.inf], np.float32), sampled, rng)
    with pytest.raises(InvalidArgument, match="empty"):
        sample(np.array([], np.float32), sampled, rng)
    p = SamplingParams(temperature=1.0, top_p=0.999)
    for t in (1.0, 2e-38):
        p.temperature = t
        rng = RandomStream(3)
        assert all(sample(np.array([0.0, -np.inf, 0.0], np.float32), p, rng) != 1 for _ in range(2000))


def test_all_negative_logits_sample_by_their_softmax():
    logits = np.array([math.log(0.7) - 1000.0, math.log(0.3) - 1000.0], np.float32)
    rng = RandomStream(7)
    p = SamplingParams(temperature=1.0)
    first = sum(sample(logits, p, rng) == 0 for _ in range(20000))
    assert first / 20000 == pytest.approx(0.7, rel=0.03)


@pytest.mark.parametrize("top_k,top_p", [(0, 1.0), (10, 1.0), (0, 0.8), (20, 0.8), (3, 0.5), (500, 0.95)])
def test_draw_for_draw_agreement_with_the_plain_sampler(top_k, top_p):
    r = random.Random(top_k * 7 + int(top_p * 100))
    for trial in range(12):
        n = r.choice([5, 64, 384])
        logits = np.array([r.gauss(0, 2.5) for _ in range(n)], dtype=np.float32)
        if trial % 4 == 0:
            logits[r.randrange(n)] = logits[r.randrange(n)]    # an exact tie
        t = r.choice([0.3, 0.8, 1.0, 1.7])
        mine, theirs = RandomStream(trial), plain.MT19937_64(trial)
        p = SamplingParams(temperature=t, top_k=top_k, top_p=top_p)
        for _ in range(25):
            assert sample(logits, p, mine) == plain.sample(list(logits), t, top_k, top_p, theirs)


def test_looking_ahead_in_the_stream_takes_nothing_from_it():
    """``peek_unit`` shows what ``unit`` will return, any number of outputs ahead and across the generator's
    refill (312 outputs), and ``skip`` moves on as ``unit`` does."""
    a, b = RandomStream(9), RandomStream(9)
    want = [b.unit() for _ in range(700)]
    got = []
    for i in range(0, 700, 7):
        assert a.peek_unit(3) == want[i + 3] and a.peek_unit(0) == want[i] and a.peek_unit(1) == want[i + 1]
        got.append(a.unit())
        a.skip(2)
        assert a.peek_unit() == want[i + 3]
        got += [a.unit() for _ in range(4)]
    assert got == [w for i, w in enumerate(want) if i % 7 not in (1, 2)]
    assert a.uniform(0.0, 3.0) == b.uniform(0.0, 3.0)
