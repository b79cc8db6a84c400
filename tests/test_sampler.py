"""Sampler: the oracle restatement against the reference's own vectors (tests/test_sampler.cpp),
then the host library's Sampler (C++) against the oracle and the same vectors.  CPU only."""
import importlib
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
import sampler_oracle as so

fr = importlib.import_module("faster-rwkv_amd")


class HostSampler(fr.Sampler):
    def __call__(self, logits, temperature, top_k, top_p):
        return self.sample(logits, temperature, top_k, top_p)


def _oracle_sampler(seed):
    g = so.MinStdRand0(seed)
    return lambda lg, t, k, p: so.sample(lg, t, k, p, g)


def _dist(sample, logits, t, k, p, n):
    d = np.zeros(len(logits))
    for _ in range(n):
        d[sample(logits, t, k, p)] += 1
    return d / n


IMPLS = [("oracle", lambda seed: _oracle_sampler(seed)), ("host", lambda seed: HostSampler(seed))]


@pytest.mark.parametrize("name,make", IMPLS)
def test_reference_greedy_vectors(name, make):
    """tests/test_sampler.cpp:37-74."""
    s = make(3)
    assert list(_dist(s, [0, 1, 2], 1, 0, 0, 200)) == [0, 0, 1]
    assert list(_dist(s, [0, 0.5, 0.499], 1, 1, 0.999, 200)) == [0, 1, 0]
    assert list(_dist(s, [0, 0.5, 0.499], 9999, 1, 0.999, 200)) == [0, 1, 0]
    assert list(_dist(s, [0, 1, 2], 1, 999, 0, 200)) == [0, 0, 1]


@pytest.mark.parametrize("name,make", IMPLS)
def test_reference_seeded_known_answer(name, make):
    """tests/test_sampler.cpp:157-169: seed 8, 50 draws."""
    d = _dist(make(8), [3, -5, 0, 4, -1.0], 2, 0, 1, 50)
    assert np.allclose(d, [0.22, 0, 0.06, 0.70, 0.02], atol=1e-9)


@pytest.mark.parametrize("name,make", IMPLS)
def test_reference_cut_vectors(name, make):
    """tests/test_sampler.cpp:96-130: deterministic zero entries and ratios of the kept ones."""
    n = 3000 if name == "oracle" else 100000
    tol = 0.03 if name == "oracle" else 0.01
    logits = [0.4, 0.5, 0.1]
    probs = so.softmax(logits)
    s = make(11)
    assert list(_dist(s, logits, 1, 999, float(probs[1]), 200)) == [0, 1, 0]
    d = _dist(s, logits, 1, 999, float(probs[1]) + 0.001, n)
    assert d[2] == 0 and abs(d[0] - probs[0] / (probs[0] + probs[1])) < tol
    assert list(_dist(s, logits, 1, 1, 1, 200)) == [0, 1, 0]
    d = _dist(s, logits, 1, 2, 1, n)
    assert d[2] == 0 and abs(d[1] - probs[1] / (probs[0] + probs[1])) < tol
    d = _dist(s, [0, 0, 0], 9999, 0, 1, n)
    assert np.abs(d - 1 / 3).max() < tol
    d = _dist(s, logits, 1, 0, 1, n)
    assert np.abs(d - probs).max() < tol


@pytest.mark.parametrize("name,make", IMPLS)
def test_reference_python_comparison_vectors(name, make):
    """tests/test_sampler.cpp:132-155."""
    n = 3000 if name == "oracle" else 100000
    tol = 0.03 if name == "oracle" else 0.01
    s = make(5)
    d = _dist(s, [3, -5, 0, 4, -1.0], 2, 0, 0.8, n)
    assert d[1] == d[2] == d[4] == 0 and abs(d[0] - 0.378) < tol and abs(d[3] - 0.622) < tol
    d = _dist(s, [3, -5, 0, 4, -1.0], 5, 0, 1.0, n)
    assert np.abs(d - [0.293, 0.059, 0.160, 0.357, 0.139]).max() < 2 * tol


def test_minstd_rand0_known_value():
    """The C++ standard fixes the 10000th value of a default-seeded minstd_rand0 at 1043618065."""
    g = so.MinStdRand0(1)
    for _ in range(10000):
        v = g()
    assert v == 1043618065


@pytest.mark.parametrize("V,t,k,p", [(50, 1.0, 0, 0.9), (1000, 0.7, 40, 0.95), (1000, 2.0, 0, 0.5),
                                     (4096, 1.3, 5, 1.0), (65536, 1.0, 0, 0.85), (300, 0.05, 0, 1.0),
                                     (300, 1.0, 1000, 0.999), (65536, 1.0, 100, 2.0)])
def test_host_sampler_draws_the_oracles_tokens(V, t, k, p):
    """Same seed, same logits -> the same token sequence, draw by draw (distinct logits, so
    the sort order is unique)."""
    rng = np.random.default_rng(V + k)
    hs, og = HostSampler(123), so.MinStdRand0(123)
    draws = 12 if V > 10000 else 60
    for i in range(draws):
        logits = (rng.standard_normal(V) * 3).astype(np.float32)
        a = hs(logits, t, k, p)
        b = so.sample(logits, t, k, p, og)
        assert a == b, (i, a, b)


def test_empty_logits_raise():
    hs = HostSampler(1)
    with pytest.raises(fr.FrhipError):
        hs.sample(np.zeros(0, np.float32))


def test_penalties_of_the_generation_loop_against_their_closed_form():
    """chat.cpp:57-62, 77: at the draw of step s a token drawn at steps d_1 < d_2 < ... < s has had
    frequency * sum_j decay^(s - 1 - d_j) + presence subtracted from its logit (each earlier adjustment was made
    to that step's own logits, not carried over), other tokens nothing.  Checked in float64 against the oracle's
    fp32 loop for a fixed drawing pattern."""
    pres, freq, decay = 0.8, 0.8, 0.996
    pen = so.Penalties(pres, freq, decay)
    draws = [7, 3, 7, 7, 1, 3, 9, 7, 0, 3, 3, 7]
    for s, tok in enumerate(draws):
        logits = np.linspace(-1, 1, 12).astype(np.float32)
        before = logits.copy()
        pen.apply(logits)
        for t in range(12):
            ds = [d for d in range(s) if draws[d] == t]
            want = float(before[t]) - (freq * sum(decay ** (s - 1 - d) for d in ds) + pres if ds else 0.0)
            assert abs(float(logits[t]) - want) <= 1e-5, (s, t)
        pen.drawn(tok)
    # decay 1, frequency 1, presence 0: the adjustment is the plain count
    pen = so.Penalties(0.0, 1.0, 1.0)
    for tok in (2, 2, 5, 2):
        pen.drawn(tok)
    logits = np.zeros(8, np.float32)
    assert list(pen.apply(logits)) == [0, 0, -3, 0, 0, -1, 0, 0]
