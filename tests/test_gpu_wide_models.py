"""Shapes beyond the fused one-token kernels' register tilings, through rwkv::Model, against the oracle:

* ffn value rows longer than 9216 binary16 elements (RWKV-4 3B: 10240; RWKV-5.2 7B: 14336): the one-token
  value product consumes its rows in slices, inside the same captured graph;
* n_embd above 4096 (RWKV-4 14B: 5120 x 20480): layernorm + mixes, every product and the state update are
  separate launches.

Two layers at full width each, a small vocabulary; criterion as everywhere: logits within 2e-2 of the
fp16-emulating oracle and the same greedy token (kernels/default/model_forward.cpp:105-192,
model_forward_seq.cpp:34-46).
"""
import importlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import pyoracle as po
from hipref import greedy_against_oracle, same_token_or_near_tie
from synth import make_model, matrix_indices, quantize_u8

fr = importlib.import_module("faster-rwkv_amd")

TOL = 2e-2
V_ = 8192

CASES = {
    # name: (version tag of make_model, version string of the file, L, C, F, H)
    "rwkv4-3B-width": (4, "4", 2, 2560, 10240, 0),
    "rwkv4-14B-width": (4, "4", 2, 5120, 20480, 0),
    "rwkv5.2-7B-width": (52, "5.2", 2, 4096, 14336, 64),
}


@pytest.mark.parametrize("strategy", ["hip fp16", "hip int8"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_wide_model_prompt_decode_and_seq_mode(tmp_path, name, strategy):
    ver, vstr, L_, C_, F_, H_ = CASES[name]
    params, emb = make_model(ver, L_, C_, F_, V_, H_, seed=77)
    path = str(tmp_path / "m.fr")
    fr.write_fr(path, vstr, L_, C_, F_, H_, params, emb)
    quant = {i: quantize_u8(params[i]) for i in matrix_indices(ver, L_)} if strategy.endswith("int8") else None
    m = fr.Model(path, strategy)
    assert (m.n_layer, m.n_embd) == (L_, C_)
    om = po.Model(ver, po.F16, L_, C_, F_, H_, V_, params, emb, quant=quant)
    prompt = np.random.default_rng(5).integers(0, V_, 8)
    worst, ties = greedy_against_oracle(m.run, om.run, prompt, 24, tol=TOL, tag=name + " " + strategy)
    print(name, strategy, "worst |dlogit| over 8 + 24 one-token steps: %.3e, %d near-tie swaps" % (worst, ties), flush=True)
    # seq mode from a fresh state, then one more token from the state it leaves
    m.reset()
    om.reset()
    ids = [int(t) for t in np.random.default_rng(6).integers(0, V_, 64)]
    lh, lo = m.run(ids), om.run(ids)
    d = float(np.abs(lh - lo).max())
    print(name, strategy, "T=64 seq mode: |dlogit| %.3e" % d, flush=True)
    assert d <= TOL and same_token_or_near_tie(lh, lo)
    greedy_against_oracle(m.run, om.run, [int(np.argmax(lo))], 4, tol=TOL, tag=name + " after the prompt")
    m.close()
    om.close()
