"""Writes tests/golden/oracle_small_models.npz: logits of small synthetic models computed by the
CPU oracle (oracle/rwkv_oracle.c through pyoracle), for RWKV-4, 5.0 and 5.2, binary16 mode and
the uint8 model.

They are regression fixtures, not reference outputs: the reference's own golden logits
(tests/test_model.cpp:10-21) need a converted checkpoint that is not available offline.  What
pins the oracle's arithmetic is listed in oracle/README.md; these vectors pin the oracle (and,
in the GPU tests, the HIP path) against silent drift, at a size that runs in a second.

Run from the repository root:  python tests/golden/make_oracle_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(HERE, ".."), os.path.join(HERE, "..", "..", "oracle")]
import pyoracle as po  # noqa: E402
from synth import make_model, matrix_indices, quantize_u8  # noqa: E402

CASES = {  # name: (version, L, C, F, V, H, seed, quant)
    "v4_f16": (4, 3, 128, 512, 300, 0, 3, False),
    "v4_u8": (4, 3, 128, 512, 300, 0, 3, True),
    "v50_f16": (50, 2, 128, 448, 300, 2, 5, False),
    "v52_f16": (52, 2, 128, 448, 300, 2, 7, False),
}
TOKENS = [5, 17, 299, 0, 42, 7, 7, 123]


def logits_of(version, L, C, F, V, H, seed, quant):
    params, emb = make_model(version, L, C, F, V, H, seed=seed)
    # the int8 model: seq mode multiplies the binary16 w^ of the codes, one-token steps the unrounded
    # fp32 weights of the same formula (pyoracle.Model, `quant=`)
    qd = {i: quantize_u8(params[i].astype(np.float32)) for i in matrix_indices(version, L)} if quant else None
    m = po.Model(version, po.F16, L, C, F, H, V, params, emb, quant=qd)
    one = np.stack([m.run(t).copy() for t in TOKENS])
    m.reset()
    seq = m.run(TOKENS).copy()
    return one.astype(np.float32), seq.astype(np.float32)


def main():
    out = {"tokens": np.asarray(TOKENS, np.int32)}
    for name, cfg in CASES.items():
        one, seq = logits_of(*cfg)
        out[name + "_one"] = one
        out[name + "_seq_last"] = seq
    np.savez_compressed(os.path.join(HERE, "oracle_small_models.npz"), **out)
    print("wrote", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
