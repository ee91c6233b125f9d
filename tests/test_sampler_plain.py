"""The plain sampler against brute force and the reference's own test vectors; the parameters' checks; the
counter-based uniform numbers."""
import math
import random

import pytest

from plain import sampler_plain as S
from jllm_serve_amd.sampling import SamplingParams, uniform


def probs(z, t):
    m = max(z)
    e = [math.exp((x - m) / t) for x in z]
    s = sum(e)
    return [x / s for x in e]


def test_nucleus_keeps_the_shortest_prefix():
    # p = (0.86, 0.05, thin tail), top_p 0.9 => keep 2 (T/SmokeTest.java:536-560)
    tail = [0.09 / 98] * 98
    p = [0.86, 0.05] + tail
    z = [math.log(x) for x in p]
    assert sorted(S.kept_weights(z, 1.0, 0, 0.9, 0.0)) == [0, 1]
    # six-token nucleus at 0.88: 0.5, 0.2, 0.1, 0.05, 0.02, 0.01 then dust
    p = [0.5, 0.2, 0.1, 0.05, 0.02, 0.011] + [0.119 / 200] * 200
    z = [math.log(x) for x in p]
    assert sorted(S.kept_weights(z, 1.0, 0, 0.88, 0.0)) == [0, 1, 2, 3, 4, 5]


def test_nucleus_membership_against_brute_force():
    # random logits N(0, 4^2), V = 4096, T in {0.7, 1.3} (T/SmokeTest.java:562-618)
    rng = random.Random(3)
    for t in (0.7, 1.3):
        for top_p in (0.5, 0.9, 0.95):
            z = [rng.gauss(0, 4) for _ in range(4096)]
            p = probs(z, t)
            order = sorted(range(len(z)), key=lambda i: -p[i])
            cum, brute = 0.0, set()
            for i in order:
                brute.add(i)
                cum += p[i]
                if cum >= top_p:
                    break
            w = S.kept_weights(z, t, 0, top_p, 0.0)
            assert set(w) == brute
            seen = set()
            for n in range(4000):
                tok = S.draw(w, rng.random())
                assert tok in brute, "never samples outside the nucleus"
                seen.add(tok)
            assert all(i in seen for i in brute if p[i] >= 0.01), "every nucleus token with p >= 1 % appears"


def test_top_k_min_p_and_order():
    z = [1.0, 3.0, 2.0, 0.5, 2.5, -1.0]
    assert sorted(S.kept_weights(z, 1.0, 3, 1.0, 0.0)) == [1, 2, 4]
    # top-p is relative to the top-k candidates' mass, not the whole vocabulary's (Sampler.java:384-402)
    w = S.kept_weights(z, 1.0, 3, 0.6, 0.0)
    mass = [math.exp(3 - 3), math.exp(2.5 - 3), math.exp(2 - 3)]
    assert sorted(w) == ([1, 4] if mass[0] / sum(mass) < 0.6 else [1])
    assert sorted(S.kept_weights(z, 1.0, 0, 1.0, 0.5)) == [1, 4]  # weights >= 0.5 of the top's: e^-0.5 = 0.61, e^-1 = 0.37
    assert S.sample(z, 0.0, 0, 1.0, 0.0, 0.3) == 1 and S.sample(z, 5.0, 1, 1.0, 0.0, 0.99) == 1  # greedy, top_k 1
    assert S.argmax([0.5, 2.0, 2.0, -1.0]) == 1


def test_draw_follows_the_weights():
    z = [math.log(0.2), math.log(0.5), math.log(0.3)]
    assert [S.sample(z, 1.0, 0, 1.0, 0.0, u) for u in (0.0, 0.19, 0.21, 0.69, 0.71, 0.999)] == [0, 0, 1, 1, 2, 2]
    # temperature sharpens: at T = 0.5 the weights are squared
    w = S.kept_weights(z, 0.5, 0, 1.0, 0.0)
    assert w[0] / w[1] == pytest.approx((0.2 / 0.5) ** 2)


def test_penalties():
    z = [2.0, -2.0, 1.0, 0.5]
    out = S.apply_penalties(z, seen={0, 1}, generated={1: 2, 2: 1}, rep=2.0, pres=0.5, freq=0.25, bias={3: -100.0})
    assert out[0] == 1.0  # positive: divided
    assert out[1] == pytest.approx(-4.0 - 0.5 - 0.5)  # negative: multiplied, then presence + 2 * frequency
    assert out[2] == pytest.approx(0.5 - 0.5 - 0.25)  # generated tokens are "seen" too
    assert out[3] == -99.5


def test_params_validation_and_defaults():
    d = SamplingParams()
    assert (d.temperature, d.top_k, d.top_p, d.min_p, d.repetition_penalty, d.seed) == (0.6, 20, 0.95, 0.0, 1.0, -1)
    for bad in (dict(temperature=-1), dict(top_k=-1), dict(top_p=0), dict(top_p=1.5), dict(min_p=2), dict(repetition_penalty=0),
                dict(temperature=float("nan")), dict(presence_penalty=float("inf"))):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    assert SamplingParams(temperature=0).greedy and SamplingParams(top_k=1).greedy and not d.greedy
    assert d.plain and not SamplingParams(repetition_penalty=1.1).plain and not SamplingParams(logit_bias={3: 1.0}).plain


def test_uniform_stream():
    a = [uniform(7, i) for i in range(1000)]
    assert a == [uniform(7, i) for i in range(1000)], "same seed, same stream"
    assert a != [uniform(8, i) for i in range(1000)]
    assert all(0.0 <= x < 1.0 for x in a) and abs(sum(a) / len(a) - 0.5) < 0.03
    assert len(set(a)) == len(a)


def test_token_logprobs():
    """Pins the plain log-probabilities: they are a distribution, they do not move with a shift of all logits, the
    alternatives come most likely first with the lower index first among equals, and a hand-computed case."""
    from plain.sampler_plain import token_logprob
    z = [0.0, math.log(2.0), math.log(2.0), math.log(3.0), -50.0]
    lp, ids, tops = token_logprob(z, 1, 3)
    assert abs(lp - math.log(2.0 / 8.0)) < 1e-9          # weights 1, 2, 2, 3 (and ~0): total 8
    assert ids == [3, 1, 2] and abs(tops[0] - math.log(3.0 / 8.0)) < 1e-9 and tops[1] == tops[2]
    assert abs(sum(math.exp(token_logprob(z, t, 0)[0]) for t in range(len(z))) - 1.0) < 1e-12
    shifted = [v + 1000.0 for v in z]
    assert abs(token_logprob(shifted, 4, 0)[0] - token_logprob(z, 4, 0)[0]) < 1e-9
    assert token_logprob(z, 0, 0)[1:] == ([], [])
    with pytest.raises(ValueError):
        SamplingParams(top_logprobs=21)
