"""The plain sampler against the vectors the reference's tests hold
(tests/test_sampler.c:184-324) and against the host-side generator."""
import numpy as np
import pytest

import plain_llama as P
from xyntetik_runner_amd.sampling import SamplerState, SamplingParams, xorshift64


def test_xorshift64_vector_and_draw_range():
    assert P.xorshift64(1) == 1082269761 and xorshift64(1) == 1082269761
    s = 88172645463325252
    for _ in range(1000):
        s2, r = P.rng_f32(s)
        assert s2 == xorshift64(s) and 0.0 <= r < 1.0
        s = s2
    assert P.xorshift64(0) == 0                       # the fixed point that makes seed 0 unusable
    with pytest.raises(ValueError):
        SamplingParams(seed=0)


def test_engine_generator_matches_plain():
    st = SamplerState(SamplingParams(temperature=1.0, seed=1234))
    s = 1234
    for _ in range(50):
        s, r = P.rng_f32(s)
        assert st.draw() == r


def test_greedy_vectors():
    assert P.sample_pick([10, 9, 1, 0.5], 0.0, 0.5) == 0
    assert P.sample_pick([1, 7, 7, 3], 0.0, 0.5) == 1            # ties: lowest id
    lg = np.array([2.0, 5.0, 1.0], dtype=np.float32)
    # greedy ignores the repeat penalty (temp 0): the penalised argmax is still returned
    assert P.sample_pick(lg, 0.0, 0.1, repeat_penalty=10.0, recent=[1]) == 1
    assert P.sample_pick(lg, 1.0, 0.0, repeat_penalty=10.0, recent=[1]) == 0    # sampling applies it
    assert P.sample_pick(lg, 1.0, 0.0, repeat_penalty=10.0, recent=[1], exempt=[1]) == 1
    assert P.sample_pick(lg, 1.0, 0.0, repeat_penalty=10.0, recent=[7, -1, 1000]) == 1   # ids outside are ignored
    # the reference's own vector: token 0 was seen, a penalty of 2 halves its 10 to 5, below token 1's 9,
    # and a temperature of 0.01 leaves no choice (tests/test_sampler.c:200-206)
    for draw in (0.0, 0.3, 0.999):
        assert P.sample_pick([10.0, 9.0, 1.0, 0.5], 0.01, draw, repeat_penalty=2.0, recent=[0]) == 1


def test_temperature_follows_softmax_and_converges_to_greedy():
    V = 8192
    lg = np.full(V, -20.0, dtype=np.float32)
    lg[[5, 100, 4000]] = [6.0, 5.4, 4.8]
    z = np.exp(lg.astype(np.float64)); z /= z.sum()
    s, counts = 42, {5: 0, 100: 0, 4000: 0}
    n = 4000
    for _ in range(n):
        s, r = P.rng_f32(s)
        t = P.sample_pick(lg, 1.0, r)
        counts[t] = counts.get(t, 0) + 1
    for t in (5, 100, 4000):
        assert abs(counts[t] / n - z[t]) < 0.03
    s = 7
    for _ in range(20):
        s, r = P.rng_f32(s)
        assert P.sample_pick(lg, 0.01, r) == 5                  # temp -> 0+: the argmax


def test_filters():
    lg = np.log(np.array([0.5, 0.25, 0.15, 0.1], dtype=np.float64)).astype(np.float32)
    assert P.sample_pick(lg, 1.0, 0.99) == 3
    assert P.sample_pick(lg, 1.0, 0.99, top_k=2) == 1            # only the two best remain
    assert P.sample_pick(lg, 1.0, 0.70, top_k=2) == 1            # renormalised: 2/3, 1/3
    assert P.sample_pick(lg, 1.0, 0.60, top_k=2) == 0
    assert P.sample_pick(lg, 1.0, 0.99, top_p=0.7) == 1          # smallest prefix with mass >= 0.7: {0, 1}
    assert P.sample_pick(lg, 1.0, 0.99, top_p=0.76) == 2
    assert P.sample_pick(lg, 1.0, 0.99, min_p=0.4) == 1          # keeps p >= 0.4 * 0.5
    assert P.sample_pick(lg, 1.0, 0.99, min_p=0.25) == 2
