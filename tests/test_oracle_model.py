"""Model-level invariants of the oracle, the ones the reference states itself:
seq mode == a loop of one-token steps (kernels/default/model_forward_seq.cpp:34-46),
ResetStates then rerun is identical (tests/test_model.cpp:93-97), and the fp16
emulation stays close to the fp32 composition (kernels/default/att.cpp, ffn.cpp)."""
import numpy as np
import pytest

import pyoracle as po
from synth import make_model, matrix_indices, quantize_u8


def _model(version, mode, L=3, C=128, F=512, V=300, H=2, seed=3):
    dt = np.float16 if mode == po.F16 else np.float32
    params, emb = make_model(version, L, C, F, V, H, seed=seed, dtype=dt)
    return po.Model(version, mode, L, C, F, H, V, params, emb), params, emb


@pytest.mark.parametrize("version", [4, 50, 52])
def test_seq_equals_loop_of_one(version):
    m, _, _ = _model(version, po.F16)
    ids = [5, 17, 299, 0, 42, 7, 7, 123]
    lg_seq = m.run(ids)
    st_seq = [s.copy() for s in m.state]
    m.reset()
    for i in ids:
        lg_one = m.run(i)
    # same arithmetic up to fp32 summation order of the v5.2 scan vs the one-token functor
    assert np.abs(lg_seq - lg_one).max() <= (0 if version == 4 else 2e-2)
    for a, b in zip(st_seq, m.state):
        assert np.allclose(a.astype(np.float32), b.astype(np.float32), rtol=1e-3, atol=1e-3)
    if version == 4:
        for a, b in zip(st_seq, m.state):
            assert np.array_equal(a, b)


@pytest.mark.parametrize("version", [4, 50, 52])
def test_reset_then_rerun_is_bit_identical(version):
    m, _, _ = _model(version, po.F16)
    a = [m.run(i).copy() for i in (1, 2, 3)]
    m.reset()
    b = [m.run(i).copy() for i in (1, 2, 3)]
    for x, y in zip(a, b):
        assert np.array_equal(x, y)
    assert not np.array_equal(a[0], a[1])


@pytest.mark.parametrize("version", [4, 52])
def test_f16_emulation_tracks_fp32_composition(version):
    m16, params, emb = _model(version, po.F16, L=6)
    m32 = po.Model(version, po.F32, 6, 128, 512, 2, 300, [p.astype(np.float32) for p in params],
                   emb.astype(np.float32))
    for i in (3, 9, 27, 81):
        l16, l32 = m16.run(i), m32.run(i)
    # after 6 layers the fp16 path has applied one /2 rescale (model_forward.cpp:173-175);
    # layernorm before the head removes the scale, so logits stay comparable
    assert np.abs(l16 - l32).max() < 3e-2
    assert np.corrcoef(l16, l32)[0, 1] > 0.999


def test_initial_state_contract():
    """model.cpp:152-175: v4 aa=bb=0, pp=-1e30, shift states 0; v5 all zero."""
    m, _, _ = _model(4, po.F16, L=2)
    assert [s.dtype for s in m.state[:5]] == [np.float16, np.float32, np.float32, np.float32, np.float16]
    assert (m.state[3] == np.float32(-1e30)).all() and (m.state[1] == 0).all() and (m.state[0] == 0).all()
    m5, _, _ = _model(52, po.F16, L=2, C=128, H=2)
    assert m5.state[1].size == 2 * 64 * 64 and (m5.state[1] == 0).all()


def test_int8_model_is_the_fp16_model_of_dequantised_weights():
    L, C, F, V = 2, 128, 512, 300
    params, emb = make_model(4, L, C, F, V, seed=11)
    qparams = list(params)
    for i in matrix_indices(4, L):
        q, mx, rx, my, ry = quantize_u8(params[i])
        qparams[i] = po.dequant_u8(q, mx, rx, my, ry)
    m = po.Model(4, po.F16, L, C, F, 0, V, params, emb)
    mq = po.Model(4, po.F16, L, C, F, 0, V, qparams, emb)
    for i in (4, 8, 15):
        a, b = m.run(i), mq.run(i)
    assert np.abs(a - b).max() < 0.1 and np.corrcoef(a, b)[0, 1] > 0.99


def test_int8_model_one_token_steps_use_the_codes_and_seq_mode_the_binary16_matrix():
    L, C, F, V = 2, 128, 512, 300
    params, emb = make_model(4, L, C, F, V, seed=12)
    quant = {i: quantize_u8(params[i]) for i in matrix_indices(4, L)}
    deq = list(params)
    for i, parts in quant.items():
        deq[i] = po.dequant_u8(*parts)
    plain = po.Model(4, po.F16, L, C, F, 0, V, deq, emb)       # the fp16 model of w^ everywhere
    head = matrix_indices(4, L)[-1]
    body_only = po.Model(4, po.F16, L, C, F, 0, V, deq, emb, quant={i: v for i, v in quant.items() if i != head})
    ids = [5, 17, 200, 3]
    # seq mode multiplies the binary16 matrix in every layer (only the head, which sees one row, is a
    # one-token product: model_forward_seq.cpp:170-178): identical when the head's codes are not registered
    assert np.array_equal(plain.run(ids), body_only.run(ids))
    body_only.close()
    coded = po.Model(4, po.F16, L, C, F, 0, V, params, emb, quant=quant)
    plain.reset()
    a, b = plain.run(ids), coded.run(ids)
    assert not np.array_equal(a, b) and np.abs(a - b).max() < 2e-3  # the head alone differs
    plain.reset(), coded.reset()
    # one-token steps differ by the rounding of w^ only: close, not identical
    for i in ids:
        a, b = plain.run(i), coded.run(i)
    assert not np.array_equal(a, b) and np.abs(a - b).max() < 2e-2
    coded.close()
    plain.reset()
    coded2 = po.Model(4, po.F16, L, C, F, 0, V, deq, emb)
    for i in ids:
        a, b = plain.run(i), coded2.run(i)
    assert np.array_equal(a, b)  # nothing stays registered after close()


def test_config1_fp32_16_prompt_tokens_then_128_greedy_steps():
    """Benchmark configuration 1 at its stated size: RWKV-4 169M-shaped (12 layers, d_model 768, ffn 3072,
    vocabulary 50277), fp32 weights, the fp32 composition of kernels/default/att.cpp:16-45 and ffn.cpp:8-23
    (the CPU model path upstream never registered), greedy decode of 128 tokens from a seeded 16-token prompt."""
    import time
    L, C, F, V = 12, 768, 3072, 50277
    params, emb = make_model(4, L, C, F, V, seed=1235, dtype=np.float32)
    m = po.Model(4, po.F32, L, C, F, 0, V, params, emb)
    prompt = np.random.default_rng(42).integers(0, V, 16)

    def greedy(n):
        m.reset()
        for t in prompt:
            lg = m.run(int(t))
        out = []
        for _ in range(n):
            tok = int(np.argmax(lg))
            out.append(tok)
            lg = m.run(tok)
        return out, lg

    t0 = time.time()
    o1, l1 = greedy(128)
    dt = time.time() - t0
    print("config 1: %d tokens in %.2f s = %.1f tok/s on the oracle's fp32 path" % (16 + 128, dt, (16 + 128) / dt))
    o2, l2 = greedy(128)
    assert o1 == o2 and np.array_equal(l1, l2) and np.isfinite(l1).all()
    assert len(set(o1)) > 1 and all(0 <= t < V for t in o1)
