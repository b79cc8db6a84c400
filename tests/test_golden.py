"""Committed fixtures (tests/golden): the reference's own known-answer vectors as data, and
regression vectors of the oracle.  CPU only; the GPU counterparts are in test_gpu_host_model.py."""
import json
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "oracle"))
sys.path.insert(0, os.path.join(HERE, "golden"))
import pyoracle as po
import sampler_oracle as so
import make_oracle_golden as mg

REF = json.load(open(os.path.join(HERE, "golden", "reference_vectors.json")))
GOLD = np.load(os.path.join(HERE, "golden", "oracle_small_models.npz"))


def _dist(logits, t, k, p, n, seed):
    g = so.MinStdRand0(seed)
    d = np.zeros(len(logits))
    for _ in range(n):
        d[so.sample(logits, t, k, p, g)] += 1
    return d / n


def test_sampler_oracle_against_the_references_fixture():
    """Every vector of tests/test_sampler.cpp that fixes a value, read from the fixture."""
    s = REF["sampler"]
    for c in s["greedy"]["cases"]:
        assert list(_dist(c["logits"], c["temperature"], c["top_k"], c["top_p"], 200, 3)) == c["dist"]
    c = s["seeded"]
    d = _dist(c["logits"], c["temperature"], c["top_k"], c["top_p"], c["n"], c["seed"])
    assert np.allclose(d, np.asarray(c["dist"], np.float32), atol=1e-7)  # EXPECT_FLOAT_EQ on float32 values
    for c in s["python_comparison"]["cases"]:
        d = _dist(c["logits"], c["temperature"], c["top_k"], c["top_p"], 4000, 5)
        assert all(d[i] == 0 for i in c["exact_zero"])
        assert np.abs(d - c["dist"]).max() < c["tol"] + 0.025  # 4000 draws instead of the reference's 100000
    c = s["uniform"]
    assert np.abs(_dist(c["logits"], c["temperature"], c["top_k"], c["top_p"], 4000, 7) - 1 / 3).max() < 0.03


def test_scalar_div_known_answer_of_the_reference():
    """tests/test_ops.cpp:9-16: 1 / 2 in binary16 is exactly 0.5."""
    c = REF["ops"]["scalar_div_fp16"]
    x = np.full(c["n"], c["fill"], np.float16)
    assert float((x / np.float16(c["divisor"]))[0]) == c["expect_first"]
    one, two = int(np.float16(c["fill"]).view(np.uint16)), int(np.float16(c["divisor"]).view(np.uint16))
    assert float(np.uint16(po.lib.orc_hdiv(one, two)).view(np.float16)) == c["expect_first"]


def test_the_references_model_logits_are_recorded_but_unusable():
    assert REF["model_logits"]["usable"] is False and "checkpoint" in REF["model_logits"]["why"]


@pytest.mark.parametrize("name", sorted(mg.CASES))
def test_oracle_reproduces_its_golden_logits(name):
    """The oracle today against the committed vectors: exact up to the last place of libm's expf."""
    one, seq = mg.logits_of(*mg.CASES[name])
    assert one.shape == GOLD[name + "_one"].shape
    assert np.abs(one - GOLD[name + "_one"]).max() <= 1e-3
    assert np.abs(seq - GOLD[name + "_seq_last"]).max() <= 1e-3
    assert np.array_equal(np.argmax(one, axis=1), np.argmax(GOLD[name + "_one"], axis=1))
