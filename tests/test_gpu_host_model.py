"""GPU parity tests through the C++ host layer: rwkv::Model("<file>.fr", "hip fp16"|"hip int8")
against the oracle on the same weights -- the path chat / bench_model take."""
import importlib
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import pyoracle as po
from hipref import greedy_against_oracle, same_token_or_near_tie
from synth import make_model, matrix_indices, quantize_u8

fr = importlib.import_module("faster-rwkv_amd")

L_, C_, F_, V_ = 12, 512, 2048, 4096


@pytest.fixture(scope="module")
def model_files(tmp_path_factory):
    d = tmp_path_factory.mktemp("fr")
    params, emb = make_model(4, L_, C_, F_, V_, seed=5)
    path = str(d / "v4.fr")
    fr.write_fr(path, "4", L_, C_, F_, 0, params, emb)
    return path, params, emb


_same_token = same_token_or_near_tie


def _oracle(params, emb, quant):
    """The oracle model; uint8: seq mode multiplies the binary16 w^ of the codes, one-token steps their
    unrounded fp32 weights (pyoracle.Model `quant=`)."""
    qd = {i: quantize_u8(params[i]) for i in matrix_indices(4, L_)} if quant else None
    return po.Model(4, po.F16, L_, C_, F_, 0, V_, params, emb, quant=qd)


@pytest.mark.parametrize("strategy", ["hip fp16", "hip int8"])
def test_model_run_matches_oracle_over_128_greedy_steps(model_files, strategy):
    path, params, emb = model_files
    m = fr.Model(path, strategy)
    assert (m.n_layer, m.n_embd, m.vocab) == (L_, C_, V_)
    om = _oracle(params, emb, strategy.endswith("int8"))
    prompt = np.random.default_rng(42).integers(0, V_, 16)
    worst, swaps = greedy_against_oracle(m.run, om.run, prompt, 128, tol=2e-2, tag=strategy)
    print(strategy, "worst |dlogit| over 128 steps:", worst, "near-tie swaps:", swaps, flush=True)
    aa = m.state(11, 1, np.float32)
    ref = om.state[11 * 5 + 1]
    assert np.abs(aa - ref).max() <= 5e-3 * np.abs(ref).max()
    m.close()


def test_python_names_of_the_reference_wrapper(model_files):
    """python/fr_python.cpp:48-56, python/fasterrwkv/__init__.py:19-25: model(ids) -> numpy logits,
    model.reset_states(), model.states(), sampler(logits, ...)."""
    path, params, emb = model_files
    m = fr.Model(path, "hip fp16")
    a = m([5, 6, 7])
    st = m.states()
    assert len(st) == L_ and [x.shape for x in st[0]] == [(C_,)] * 5
    assert st[0][0].dtype == np.float16 and st[0][1].dtype == np.float32 and np.abs(st[0][1]).max() > 0
    m.reset_states()
    assert np.all(m.states()[3][1] == 0) and np.all(m.states()[3][3] == np.float32(-1e30))  # model.cpp:152-160
    assert np.array_equal(m([5, 6, 7]), a)
    smp = fr.Sampler(seed=3)
    assert smp(a, 1.0, 1, 0.0) == int(np.argmax(a))  # top_k = 1 is the arg-max
    m.close()


def test_fused_graph_path_equals_operator_by_operator_path(model_files):
    path, _, _ = model_files
    ids = [3, 1000, 77, 77, 4095, 0, 9]
    m = fr.Model(path, "hip fp16")
    fused = [m.run(i) for i in ids]
    m.close()
    os.environ["FR_HIP_GENERIC"] = "1"
    try:
        g = fr.Model(path, "hip fp16")
        generic = [g.run(i) for i in ids]
        g.close()
    finally:
        del os.environ["FR_HIP_GENERIC"]
    for a, b in zip(fused, generic):
        assert np.array_equal(a, b)  # same kernels, same order of arithmetic


def test_reset_and_state_file_round_trip(model_files, tmp_path):
    """tests/test_model.cpp:35-51 (save -> run -> load -> run reproduces) and :93-97."""
    path, _, _ = model_files
    m = fr.Model(path, "hip fp16")
    a = [m.run(i) for i in (1, 2, 3)]
    m.reset()
    b = [m.run(i) for i in (1, 2, 3)]
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    sf = str(tmp_path / "state.bin")
    m.save_state(sf)
    c = m.run(4)
    m.run(5)
    m.load_state(sf)
    d = m.run(4)
    assert np.array_equal(c, d)
    m.close()


@pytest.mark.parametrize("strategy", ["hip fp16", "hip int8"])
def test_seq_mode_equals_one_token_steps_and_oracle(model_files, strategy):
    """kernels/default/model_forward_seq.cpp:34-46: Run(ids) == Run(id) for each id -- for
    logits AND for the state left behind (checked by continuing to decode from it)."""
    path, params, emb = model_files
    ids = [int(t) for t in np.random.default_rng(43).integers(0, V_, 200)]
    m = fr.Model(path, strategy)
    seq = m.run(ids)
    after_seq = [m.run(t) for t in (9, 8, 7)]
    m.reset()
    for i in ids:
        one = m.run(i)
    after_one = [m.run(t) for t in (9, 8, 7)]
    assert np.abs(seq - one).max() <= 2e-2
    assert int(np.argmax(seq)) == int(np.argmax(one))
    for a, b in zip(after_seq, after_one):
        assert np.abs(a - b).max() <= 2e-2
    om = _oracle(params, emb, strategy.endswith("int8"))
    ref = om.run(ids)
    assert np.abs(seq - ref).max() <= 2e-2 and int(np.argmax(seq)) == int(np.argmax(ref))
    m.close()


@pytest.mark.parametrize("spec", ["v=4,L=3,C=512,F=2048,V=2048,seed=11", "v=5.2,L=3,C=512,F=1792,V=2048,H=8,seed=12"])
@pytest.mark.parametrize("generic", [False, True])
def test_kept_binary16_image_of_uint8_weights_gives_the_same_bits(spec, generic):
    """FR_HIP_SEQ_IMAGE=1 (opt-in; unset or 0: off): prompts of
    FRHIP_SEQ_EXPAND_ROWS rows or more multiply the kept binary16 image of the uint8 weights instead
    of one expanded per call; w^ is the same, so logits (last
    row and every row) and the state left behind are the same bits.  One-token steps still read the
    codes."""
    ids = [int(t) for t in np.random.default_rng(47).integers(0, 2048, 300)]

    def run():
        m = fr.Model("synthetic:" + spec, "hip int8")
        out = [m.run(ids), m.run(ids[:250]), m.run(5), m.run(ids[:64]), m.run(6)]
        m.reset()
        out.append(m.run_full(ids[:200]))
        out += [st for layer in m.states() for st in layer]
        m.close()
        return out

    env = {"FR_HIP_SEQ_IMAGE": "1", **({"FR_HIP_GENERIC": "1"} if generic else {})}
    saved = {k: os.environ.get(k) for k in env}
    plain = None
    try:
        if generic:
            os.environ["FR_HIP_GENERIC"] = "1"
        os.environ["FR_HIP_SEQ_IMAGE"] = "0"  # the default, stated
        plain = run()
        os.environ.update(env)
        kept = run()
    finally:
        for k, v in saved.items():
            os.environ.pop(k, None) if v is None else os.environ.__setitem__(k, v)
    assert len(plain) == len(kept)
    for a, b in zip(plain, kept):
        assert np.array_equal(a, b)


_FORMS_CHILD = r"""
import hashlib, importlib, os, sys
import numpy as np
sys.path.insert(0, sys.argv[1])
fr = importlib.import_module("faster-rwkv_amd")
for spec, strategy in [("v=5.2,L=2,C=2560,F=8960,V=4096,H=40,seed=31", "hip int8"),
                       ("v=5.2,L=2,C=2560,F=8960,V=4096,H=40,seed=31", "hip fp16"),
                       ("v=4,L=2,C=2048,F=8192,V=4096,seed=32", "hip int8"),
                       ("v=5,L=2,C=768,F=2688,V=4096,H=12,seed=33", "hip fp16")]:
    m = fr.Model("synthetic:" + spec, strategy)
    h = hashlib.sha1()
    tok = 7
    for _ in range(6):
        lg = m.run(tok)
        h.update(lg.tobytes())
        tok = int(np.argmax(lg))
    m.close()
    print(h.hexdigest())
"""


def test_one_matrix_per_workgroup_and_shared_launches_give_the_same_bits():
    """The layernorm launches of several matrices exist in two forms (every workgroup serving all matrices, or one:
    rows_excl_kernel); which one runs is a matter of speed only.  FRHIP_SEG_EXCLUSIVE=0 / 1 forces the form for
    every such launch (read once per process, hence the child processes): same logits, bit for bit, as the default
    choice, for RWKV-5.2 at the 3B width (where the default picks the one-matrix form), RWKV-4 at the 1.5B width
    and a narrow RWKV-5.0 (where it does not)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    seen = {}
    for form in (None, "0", "1"):
        env = {k: v for k, v in os.environ.items() if k != "FRHIP_SEG_EXCLUSIVE"}
        if form is not None:
            env["FRHIP_SEG_EXCLUSIVE"] = form
        out = subprocess.run([sys.executable, "-c", _FORMS_CHILD, root], env=env, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr[-2000:]
        seen[form] = out.stdout.split()
        assert len(seen[form]) == 4
    assert seen[None] == seen["0"] == seen["1"]


@pytest.mark.parametrize("spec,strategy", [
    ("v=4,L=4,C=512,F=2048,V=4096,seed=21", "hip fp16"),
    ("v=4,L=4,C=512,F=2048,V=4096,seed=21", "hip int8"),
    ("v=5.2,L=3,C=512,F=1792,V=4096,H=8,seed=22", "hip fp16"),
    ("v=5,L=3,C=512,F=2048,V=4096,H=8,seed=23", "hip int8"),
])
def test_greedy_loop_kept_on_the_device_equals_the_loop_of_runs(spec, strategy):
    """fr_greedy_decode on the fused path queues the steps back to back, each step's first kernel taking
    its token from the arg-max pairs of the step before; FR_HIP_GREEDY_ON_HOST=1 is chat.cpp:56-92's
    loop (Run, arg-max on the host, Run).  Same tokens, same logits afterwards, same state: bit for bit.
    1 100 steps cross the 1 023-step batches the host waits for; a one-step and a two-step call and a
    call right after a prompt in seq mode are covered too."""
    prompt = [int(t) for t in np.random.default_rng(48).integers(0, 4096, 40)]

    def run():
        m = fr.Model("synthetic:" + spec, strategy)
        out = []
        for first, steps in ((7, 1), (8, 2), (9, 1100), (10, 33)):
            ids, _ = m.greedy(first, steps)
            out.append(ids.copy())
        out.append(m.run(11).copy())
        lg = m.run(prompt)
        ids, _ = m.greedy(int(np.argmax(lg)), 50)
        out.append(ids.copy())
        out.append(m.run(12).copy())
        out += [st for layer in m.states() for st in layer]
        m.close()
        return out

    chained = run()
    os.environ["FR_HIP_GREEDY_ON_HOST"] = "1"
    try:
        looped = run()
    finally:
        del os.environ["FR_HIP_GREEDY_ON_HOST"]
    # the loop of runs, spelled out in Python, for the first calls
    m = fr.Model("synthetic:" + spec, strategy)
    for first, steps, got in ((7, 1, chained[0]), (8, 2, chained[1])):
        t = first
        for i in range(steps):
            t = int(np.argmax(m.run(t)))
            assert t == got[i]
    m.close()
    assert len(chained) == len(looped)
    for a, b in zip(chained, looped):
        assert np.array_equal(a, b)
    assert len(set(chained[2].tolist())) > 1  # not a constant sequence


def test_synthetic_model_and_cpp_greedy_loop():
    m = fr.Model("synthetic:v=4,L=2,C=256,F=1024,V=1024,seed=7", "hip int8")
    toks, secs = m.greedy(1, 16)
    m.reset()
    again, _ = m.greedy(1, 16)
    assert np.array_equal(toks, again) and secs > 0
    assert (toks >= 0).all() and (toks < 1024).all()
    m.close()


def test_bad_arguments_surface_as_exceptions(model_files):
    path, _, _ = model_files
    with pytest.raises(fr.FrhipError):
        fr.Model(path, "hip fp32")
    m = fr.Model(path, "hip fp16")
    with pytest.raises(fr.FrhipError):
        m.run(V_ + 5)
    m.close()


def test_rwkv5_2_model_matches_oracle(tmp_path):
    """RWKV-5.2 (config-5 architecture at reduced size): fused graph path through Model::Run."""
    L5, C5, F5, V5, H5 = 6, 512, 1792, 2048, 8
    params, emb = make_model(52, L5, C5, F5, V5, H5, seed=21)
    path = str(tmp_path / "v52.fr")
    fr.write_fr(path, "5.2", L5, C5, F5, H5, params, emb)
    for strategy in ("hip fp16", "hip int8"):
        qd = {i: quantize_u8(params[i]) for i in matrix_indices(52, L5)} if strategy.endswith("int8") else None
        om = po.Model(52, po.F16, L5, C5, F5, H5, V5, params, emb, quant=qd)
        m = fr.Model(path, strategy)
        assert m.n_head == H5 and m.n_ffn == F5
        tok, worst = 11, 0.0
        for step in range(64):
            lh, lo = m.run(tok), om.run(tok)
            worst = max(worst, float(np.abs(lh - lo).max()))
            assert same_token_or_near_tie(lh, lo), "greedy token differs at step %d" % step
            tok = int(np.argmax(lo))
        print(strategy, "v5.2 worst |dlogit| over 64 steps:", worst, flush=True)
        assert worst <= 2e-2
        s_ref = om.state[5 * 3 + 1]
        s_got = m.state(5, 1, np.float32)
        assert np.abs(s_got - s_ref).max() <= 5e-3 * np.abs(s_ref).max()
        # seq-mode prefill of a prompt, then decode: same logits as the oracle's seq mode
        m.reset()
        om.reset()
        prompt = [int(t) for t in np.random.default_rng(44).integers(0, V5, 96)]
        ls, lo = m.run(prompt), om.run(prompt)
        assert np.abs(ls - lo).max() <= 2e-2 and _same_token(ls, lo)
        tok = int(np.argmax(lo))
        for step in range(8):
            ls, lo = m.run(tok), om.run(tok)
            assert np.abs(ls - lo).max() <= 2e-2
            tok = int(np.argmax(lo))
        m.close()
        om.close()


def test_rwkv5_0_model_matches_oracle(tmp_path):
    """RWKV-5.0 through Model::Run: fused one-token path, seq mode, and the operator loop."""
    L5, C5, F5, V5, H5 = 6, 512, 1792, 2048, 8
    params, emb = make_model(50, L5, C5, F5, V5, H5, seed=23)
    path = str(tmp_path / "v50.fr")
    fr.write_fr(path, "5", L5, C5, F5, H5, params, emb)
    for strategy in ("hip fp16", "hip int8"):
        qd = {i: quantize_u8(params[i]) for i in matrix_indices(50, L5)} if strategy.endswith("int8") else None
        om = po.Model(50, po.F16, L5, C5, F5, H5, V5, params, emb, quant=qd)
        m = fr.Model(path, strategy)
        assert m.n_head == H5 and m.n_ffn == F5
        tok, worst = 11, 0.0
        for step in range(48):
            lh, lo = m.run(tok), om.run(tok)
            worst = max(worst, float(np.abs(lh - lo).max()))
            assert same_token_or_near_tie(lh, lo), "greedy token differs at step %d" % step
            tok = int(np.argmax(lo))
        print(strategy, "v5.0 worst |dlogit| over 48 steps:", worst, flush=True)
        assert worst <= 2e-2
        s_ref = om.state[5 * 3 + 1]
        s_got = m.state(5, 1, np.float32)
        assert np.abs(s_got - s_ref).max() <= 5e-3 * np.abs(s_ref).max()
        m.reset()
        om.reset()
        prompt = [int(t) for t in np.random.default_rng(45).integers(0, V5, 80)]
        ls, lo = m.run(prompt), om.run(prompt)
        assert np.abs(ls - lo).max() <= 2e-2 and _same_token(ls, lo)
        tok = int(np.argmax(lo))
        for step in range(8):
            ls, lo = m.run(tok), om.run(tok)
            assert np.abs(ls - lo).max() <= 2e-2
            tok = int(np.argmax(lo))
        m.close()


def test_full_output_gives_the_logits_of_every_position(model_files):
    """ModelForwardSeq(..., full_output=true) (kernels/default/model_forward_seq.cpp:170-178): row t
    equals the logits of a run over the first t+1 tokens; the last row equals Model::Run."""
    path, params, emb = model_files
    m = fr.Model(path, "hip fp16")
    om = po.Model(4, po.F16, L_, C_, F_, 0, V_, params, emb)
    prompt = [int(t) for t in np.random.default_rng(46).integers(0, V_, 40)]
    full = m.run_full(prompt)
    assert full.shape == (40, V_)
    m.reset()
    last = m.run(prompt)
    assert np.abs(full[-1] - last).max() <= 1e-3
    for t in (0, 7, 39):
        om.reset()
        lo = om.run(prompt[: t + 1]) if t else om.run(prompt[0])
        assert np.abs(full[t] - lo).max() <= 2e-2 and int(np.argmax(full[t])) == int(np.argmax(lo))
    m.close()


def test_sampled_generation_follows_the_oracle_sampler(model_files):
    """chat.cpp's loop with a seeded Sampler: the C++ loop on the hip model picks the tokens that the
    sampler oracle picks from the same logits."""
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
    import sampler_oracle as so
    path, params, emb = model_files
    m = fr.Model(path, "hip fp16")
    toks, _ = m.generate(fr.Sampler(77), 5, 24, temperature=1.2, top_k=50, top_p=0.9)
    m.reset()
    g = so.MinStdRand0(77)
    tok = 5
    for i in range(24):
        tok = so.sample(m.run(tok), 1.2, 50, 0.9, g)
        assert tok == int(toks[i]), i
    m.close()


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 1, 0.0), (1.2, 50, 0.9)])  # chat.cpp:76-77's own settings; a sampled run
def test_generation_with_the_repetition_penalties_of_the_chat_loop(temperature, top_k, top_p):
    """chat.cpp:56-92 with its presence / frequency penalties and their decay (0.8, 0.8, 0.996: chat.cpp:22-24):
    the C++ loop on the hip model draws the tokens that the oracle's sampler draws from the same logits adjusted
    by the oracle's statement of the penalties, and the penalties change what is drawn (a vocabulary of 64 and 80
    steps: without penalties some token must repeat, and a repeated token's logit is at least 1.6 lower with them)."""
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "oracle"))
    import sampler_oracle as so
    m = fr.Model("synthetic:v=4,L=2,C=256,F=1024,V=64,seed=9", "hip fp16")
    steps = 80
    toks, _ = m.generate(fr.Sampler(77), 5, steps, temperature=temperature, top_k=top_k, top_p=top_p,
                         presence_penalty=0.8, frequency_penalty=0.8, penalty_decay=0.996)
    m.reset()
    plain, _ = m.generate(fr.Sampler(77), 5, steps, temperature=temperature, top_k=top_k, top_p=top_p)
    assert not np.array_equal(toks, plain)
    if top_k == 1:  # greedy: without penalties the device-side loop gives the same tokens, with them it is not used
        m.reset()
        assert np.array_equal(m.greedy(5, steps)[0], plain)
    m.reset()
    g, pen = so.MinStdRand0(77), so.Penalties(0.8, 0.8, 0.996)
    tok = 5
    for i in range(steps):
        tok = so.sample(pen.apply(m.run(tok)), temperature, top_k, top_p, g)
        pen.drawn(tok)
        assert tok == int(toks[i]), i
    m.close()


# ---------------------------------------------------------------------------
# committed golden vectors (tests/golden/oracle_small_models.npz): the HIP path on the same
# synthetic models, one-token steps and seq mode, within the stated tolerance of the fixture
# ---------------------------------------------------------------------------
import sys as _sys

_sys.path.insert(0, os.path.join(os.path.dirname(__file__), "golden"))
import make_oracle_golden as _mg

_GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "oracle_small_models.npz"))


@pytest.mark.parametrize("name", sorted(_mg.CASES))
def test_hip_model_against_committed_golden_logits(name, tmp_path):
    version, L, C, F, V, H, seed, quant = _mg.CASES[name]
    params, emb = make_model(version, L, C, F, V, H, seed=seed)
    path = str(tmp_path / (name + ".fr"))
    fr.write_fr(path, {4: "4", 50: "5", 52: "5.2"}[version], L, C, F, H, params, emb)
    m = fr.Model(path, "hip int8" if quant else "hip fp16")
    gold_one, gold_seq = _GOLD[name + "_one"], _GOLD[name + "_seq_last"]
    for i, t in enumerate(_GOLD["tokens"]):
        lh = m.run(int(t))
        assert np.abs(lh - gold_one[i]).max() <= 2e-2, (name, i)
        assert _same_token(lh, gold_one[i])
    m.reset()
    ls = m.run([int(t) for t in _GOLD["tokens"]])
    assert np.abs(ls - gold_seq).max() <= 2e-2 and _same_token(ls, gold_seq)
